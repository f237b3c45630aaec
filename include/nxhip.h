/* nxhip.h — C ABI of libnxhip, an MI355X (gfx950) engine for the Nx backend
   contract (Nx_core.Backend_intf.S of raven-ml/raven).

   Everything here is plain C: pointers, sizes and one POD descriptor. A binding
   (OCaml foreign stubs, ctypes, ...) unpacks its tensor handle into an
   nxh_tensor and calls one entry point per primitive, exactly where the
   reference binding calls caml_nx_c_<op> (packages/nx/lib/backend_c/
   nx_backend.ml:104-168,242-264,349,395-397,482-483).

   Conventions shared by every compute entry point
   - "output first": the caller allocates the result storage (nxh_alloc) and
     passes its descriptor as the first tensor argument, as the reference does
     (nx_backend.ml:170-183).
   - strides and offset are in ELEMENTS and may be zero (broadcast) or negative
     (flip) on inputs; rank <= NXH_MAX_NDIM (nx_c.h:45-61).
   - dtype tags equal Nx's Dtype.Packed.tag (nx_c.h:130-200).
   - every call is asynchronous on the context's stream; nxh_memcpy_d2h,
     nxh_gather, nxh_scatter and nxh_synchronize wait for it.
   - return value: NXH_OK, NXH_INVALID_ARGUMENT (the reference raises
     Invalid_argument) or NXH_FAILURE (the reference raises Failure); the
     message, prefixed "<op>: " like the reference's, is read with
     nxh_last_error (nx_c.h:365-395, nx_c_engine.c:1345-1351). */

#ifndef NXHIP_H
#define NXHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NXH_MAX_NDIM 32

/* Status kinds (nx_c_engine.c:1345-1351: which statuses become
   Invalid_argument, which Failure). */
enum { NXH_OK = 0, NXH_INVALID_ARGUMENT = 1, NXH_FAILURE = 2 };

/* dtype tags, Dtype.Packed.tag order (nx_c.h:130-168, 197-200). */
typedef enum {
  NXH_F16 = 0,
  NXH_F32 = 1,
  NXH_F64 = 2,
  NXH_BF16 = 3,
  NXH_F8E4M3 = 4,
  NXH_F8E5M2 = 5,
  NXH_I4 = 6,
  NXH_U4 = 7,
  NXH_I8 = 8,
  NXH_U8 = 9,
  NXH_I16 = 10,
  NXH_U16 = 11,
  NXH_I32 = 12,
  NXH_U32 = 13,
  NXH_I64 = 14,
  NXH_U64 = 15,
  NXH_C32 = 16,
  NXH_C64 = 17,
  NXH_BOOL = 18,
  NXH_DTYPE_COUNT = 19
} nxh_dtype;

/* Unary ops, Backend_intf.S order (backend_intf.ml:240-323;
   nx_c_map.c:1184-1204). */
typedef enum {
  NXH_NEG = 0, NXH_RECIP, NXH_ABS, NXH_SIGN, NXH_SQRT, NXH_EXP, NXH_LOG,
  NXH_SIN, NXH_COS, NXH_TAN, NXH_ASIN, NXH_ACOS, NXH_ATAN, NXH_SINH, NXH_COSH,
  NXH_TANH, NXH_TRUNC, NXH_CEIL, NXH_FLOOR, NXH_ROUND, NXH_ERF,
  NXH_UNARY_COUNT
} nxh_unary_op;

/* Binary ops (backend_intf.ml:157-228; nx_c_map.c:1207-1219). */
typedef enum {
  NXH_ADD = 0, NXH_SUB, NXH_MUL, NXH_IDIV, NXH_FDIV, NXH_MOD, NXH_POW,
  NXH_ATAN2, NXH_MAX, NXH_MIN, NXH_XOR, NXH_OR, NXH_AND,
  NXH_BINARY_COUNT
} nxh_binary_op;

/* Comparisons, bool output (backend_intf.ml:197-207; nx_c_map.c:1253-1256). */
typedef enum {
  NXH_CMPEQ = 0, NXH_CMPNE, NXH_CMPLT, NXH_CMPLE, NXH_COMPARE_COUNT
} nxh_compare_op;

/* Reductions (backend_intf.ml:341-351; nx_c_fold.c:824-831). */
typedef enum {
  NXH_SUM = 0, NXH_PROD, NXH_RMAX, NXH_RMIN, NXH_REDUCE_COUNT
} nxh_reduce_op;

/* The tensor descriptor: storage pointer + the four ABI slots of the reference
   handle (nx_c.h:47-61, 406-412). `data` is a DEVICE pointer to storage
   element 0 (not to the view's first element); the first live element is at
   data + offset * elem_size. */
typedef struct {
  void *data;
  int32_t dtype; /* nxh_dtype */
  int32_t ndim;
  int64_t offset;
  int64_t shape[NXH_MAX_NDIM];
  int64_t strides[NXH_MAX_NDIM];
} nxh_tensor;

typedef struct nxh_context nxh_context;

/* ── Context (nx_backend.mli:32-39 create_context) ───────────────────────── */

/* Creates a context on the device named by the environment variable
   NX_HIP_DEVICE (default 0): one HIP stream, one caching allocator. Fails with
   NXH_FAILURE when no usable GPU is present; *ctx is then NULL and the message
   is available from nxh_last_error(NULL). */
int nxh_context_create(nxh_context **ctx);
void nxh_context_destroy(nxh_context *ctx);
/* Message of the last non-OK status returned on the calling thread. */
const char *nxh_last_error(nxh_context *ctx);
/* Device ordinal, name, CU count of the context's GPU. */
int nxh_device_info(nxh_context *ctx, int *device, char *name, size_t name_len,
                    int *compute_units);

/* ── Device buffers and transfer (backend_intf.ml:108-145 buffer / from_host /
   to_host; nx_backend.ml:54-69) ──────────────────────────────────────────── */

/* Bytes of `count` elements of dtype (packed int4/uint4: two per byte,
   nx_c.h:325-328). Returns -1 for a bad tag. */
int64_t nxh_dtype_bytes(int dtype, int64_t count);
/* Uninitialised device block from the context's caching allocator
   (Backend_intf.buffer). bytes == 0 yields a valid non-NULL pointer. */
int nxh_alloc(nxh_context *ctx, size_t bytes, void **dptr);
/* Returns a block to the allocator. Stream-ordered: kernels already queued on
   the context stream may still use it. */
int nxh_free(nxh_context *ctx, void *dptr);
/* from_host: host -> device copy; the host buffer may be reused on return. */
int nxh_memcpy_h2d(nxh_context *ctx, void *dst_device, const void *src_host,
                   size_t bytes);
/* to_host: waits for the stream, then device -> host copy. */
int nxh_memcpy_d2h(nxh_context *ctx, void *dst_host, const void *src_device,
                   size_t bytes);
int nxh_synchronize(nxh_context *ctx);
/* Allocator counters: bytes handed out, bytes cached in free lists, bytes
   obtained from the driver, number of driver allocations. */
int nxh_memory_stats(nxh_context *ctx, uint64_t *in_use, uint64_t *cached,
                     uint64_t *reserved, uint64_t *driver_allocs);
/* Returns every cached block to the driver. */
int nxh_trim(nxh_context *ctx);

/* full (backend_intf.ml:130-136; nx_backend.ml:61-64): every element of `out`
   (any strides) becomes the element whose storage bytes are at `value`
   (elem_size bytes, already encoded in the dtype's storage format). */
int nxh_fill(nxh_context *ctx, const nxh_tensor *out, const void *value);

/* ── map family (nx_c_map.c) ─────────────────────────────────────────────── */

/* caml_nx_c_<unary> (nx_c_map.c:1184-1204): out[i] = op(x[i]), computed in the
   dtype's compute type and rounded/wrapped once on store. */
int nxh_unary(nxh_context *ctx, int op, const nxh_tensor *out,
              const nxh_tensor *x);
/* caml_nx_c_<binary> (nx_c_map.c:1207-1219). */
int nxh_binary(nxh_context *ctx, int op, const nxh_tensor *out,
               const nxh_tensor *x, const nxh_tensor *y);
/* caml_nx_c_cmp{eq,ne,lt,le} (nx_c_map.c:1231-1256): bool (uint8 0/1) output,
   dispatched on the input dtype. */
int nxh_compare(nxh_context *ctx, int op, const nxh_tensor *out,
                const nxh_tensor *x, const nxh_tensor *y);
/* caml_nx_c_where (nx_c_map.c:809-839, 1224): storage-typed select. */
int nxh_where(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *cond,
              const nxh_tensor *if_true, const nxh_tensor *if_false);
/* caml_nx_c_cast (nx_c_map.c:182-218, 1261-1280): the src x dst matrix. */
int nxh_cast(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *x);

/* ── fold family (nx_c_fold.c) ───────────────────────────────────────────── */

/* caml_nx_c_reduce_{sum,prod,max,min} (nx_c_fold.c:824-831; driver
   nx_c_engine.c:1052-1170). `axes` strictly increasing; `out` is either the
   squeezed result or the keepdims-shaped one (nx_c_engine.c:1392-1420). */
int nxh_reduce(nxh_context *ctx, int op, const nxh_tensor *out,
               const nxh_tensor *x, const int32_t *axes, int n_axes);
/* No counterpart in the reference. nxh_reduce for callers that cannot allocate
   (code under HIP graph capture by the caller's own stream machinery, tight
   serving loops, harnesses that forbid hipMalloc): the same kernels, the same
   split, bit-identical results, but the partial results of a split reduction
   live in a static device array of NXH_STATIC_WORKSPACE_BYTES that every GPU
   the library runs on holds until the process ends, so the call allocates and
   frees nothing. A reduction whose partials would not fit is refused with
   Failure before anything is launched (it needs at most
   splits * outputs * sizeof(accumulator) bytes; e.g. float32 [8192,8192] over
   axis 0 takes 2 MiB). All calls on one GPU share that array: calls on one
   context are ordered by its stream, calls that overlap on one GPU from
   different contexts race. */
#define NXH_STATIC_WORKSPACE_BYTES (8u << 20)
int nxh_reduce_noalloc(nxh_context *ctx, int op, const nxh_tensor *out,
                       const nxh_tensor *x, const int32_t *axes, int n_axes);
/* caml_nx_c_arg{max,min} (nx_c_fold.c:832-833; nx_c_engine.c:1214-1254):
   int32 output; is_min = 0 for argmax, 1 for argmin. */
int nxh_argreduce(nxh_context *ctx, int is_min, const nxh_tensor *out,
                  const nxh_tensor *x, int axis);

/* ── matmul (nx_c_matmul.c:874-1108, 1271-1277) ──────────────────────────── */
int nxh_matmul(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *a,
               const nxh_tensor *b);

/* ── move family (nx_c_move.c) ───────────────────────────────────────────── */

/* caml_nx_c_copy (nx_c_move.c:191-201): copy / contiguous / assign. */
int nxh_copy(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *x);
/* caml_nx_c_gather (nx_c_move.c:342-458). Waits for the stream so that an
   out-of-bounds index is reported by this call, as in the reference. */
int nxh_gather(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *data,
               const nxh_tensor *indices, int axis);

/* caml_nx_c_scatter (nx_c_move.c:460-586): `out` already holds the template (the
   binding copies it first, nx_backend.ml:412-416). mode 0 = Set (the last update
   in row-major order of the index space wins), 1 = Add (accumulates in that
   order, in the dtype's compute type). Deterministic. Waits for the stream so
   that an out-of-bounds index is reported by this call. */
int nxh_scatter(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *indices,
                const nxh_tensor *updates, int axis, int mode);
/* caml_nx_c_pad (nx_c_move.c:203-276): out = x widened by pad_before[d] elements
   in front of every axis d (the rest of out's extent behind it), the border
   holding *fill_value (one storage element of the dtype, host memory; the
   reference passes it as a scalar tensor filled by the binding). */
int nxh_pad(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *x,
            const void *fill_value, const int64_t *pad_before);
/* caml_nx_c_cat (nx_c_move.c:278-312): the members, in order, along `axis`. */
int nxh_cat(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *const *inputs,
            int n_inputs, int axis);

/* ── scan (nx_c_fold.c:161-176, 741-837; driver nx_c_engine.c:1257-1331) ───── */

/* caml_nx_c_cumsum / cumprod / cummax / cummin: inclusive prefix scan along
   `axis`; `op` is an nxh_reduce_op. out has x's shape and dtype. */
int nxh_scan(nxh_context *ctx, int op, const nxh_tensor *out, const nxh_tensor *x, int axis);

/* ── random (nx_c_random.c) ──────────────────────────────────────────────── */

/* caml_nx_c_threefry (nx_c_random.c:36-133): Threefry-2x32, 20 rounds, on int32
   tensors of equal shape whose last axis (extent 2) holds the word pair. */
int nxh_threefry(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *key,
                 const nxh_tensor *counter);

/* ── sort (nx_c_sort.c) ──────────────────────────────────────────────────── */

/* caml_nx_c_sort (nx_c_sort.c:262-292, driver :366-470): out = x sorted along
   `axis` in the dtype's compute type; NaN-class elements last in both
   directions; complex is lexicographic. Elements that compare equal but differ
   in bits (IEEE +-0) come out in ascending original index, reversed for
   descending — one of the orders the reference's unstable sort may give. */
int nxh_sort(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *x, int axis,
             int descending);
/* caml_nx_c_argsort (nx_c_sort.c:294-312): int32 indices that sort x along
   `axis`; ties keep the first index first in both directions, NaN-class
   elements last in index order. */
int nxh_argsort(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *x, int axis,
                int descending);

/* ── windows (nx_c_move.c:588-870) ───────────────────────────────────────── */

/* caml_nx_c_unfold (nx_c_move.c:655-690, 789-822): x (leading..., spatial...)
   -> out (leading..., prod(kernel_size), L), the last n_window_dims dims of x
   being the windowed ones; taps that fall into the padding read as zero.
   `padding` is flat: before0, after0, before1, ... */
int nxh_unfold(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *x,
               int n_window_dims, const int64_t *kernel_size, const int64_t *stride,
               const int64_t *dilation, const int64_t *padding);
/* caml_nx_c_fold (nx_c_move.c:745-787, 829-866): x (leading..., prod(kernel),
   L) -> out (leading..., output_size...); taps landing on one output element
   are summed in ascending tap order in the compute type. */
int nxh_fold(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *x,
             int n_window_dims, const int64_t *output_size, const int64_t *kernel_size,
             const int64_t *stride, const int64_t *dilation, const int64_t *padding);

/* ── fused sequences of primitives ───────────────────────────────────────── */

/* Each call below equals a fixed sequence of the primitives above, as the
   reference's frontend and layers issue them, done in one pass over the data
   with every intermediate rounded to the dtype its primitive would have stored.
   They have no binding of their own in the reference: a caller that sees the
   sequence (a deferred-evaluation window in the binding) substitutes the call.
   Floating dtypes f16/bf16/f32/f64; rows (the last axis) contiguous and at most
   2^24 long (a row of up to 8192 elements is held in registers, a longer one
   is walked three times), otherwise Failure and the caller issues the
   primitives. */

/* frontend.ml:4242-4252 softmax over the last axis: max, sub, exp, sum, div.
   With `scale` (one storage element of x's dtype, host memory) x is first
   multiplied by it; with `mask` (bool, x's shape, stride-0 broadcast allowed)
   elements whose mask is 0 are replaced by *masked_value, as the mul and where
   of kaun/lib/attention.ml:67-110. out may be x's dtype or, for f32 input,
   f16/bf16 (the cast that follows in attention.ml:105-108). */
int nxh_softmax_rows(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *x,
                     const void *scale, const nxh_tensor *mask, const void *masked_value);
/* kaun/lib/layer_norm.ml:43-68: (x - mean) / sqrt(var + eps) over the last axis
   (biased variance of the centred values; statistics in float32 for 16-bit
   dtypes), then * gamma and + beta when given (rank 1, the row length). */
int nxh_layer_norm_rows(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *x,
                        const nxh_tensor *gamma, const nxh_tensor *beta, double eps);
/* kaun/lib/fn.ml:31-38: ((x * (tanh((x + x*(x*x) * c0) * c1) + c2)) * c3);
   `constants` = c0..c3 as four storage elements of x's dtype (host memory),
   the scalars the sequence would have been given. C-contiguous operands. */
int nxh_gelu_tanh(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *x,
                  const void *constants);

/* kaun/lib/attention.ml:67-110 for f16 / bf16 operands, as one kernel that never
   writes the score tensor:
     out = matmul (cast dtype (softmax (where mask (matmul (cast f32 q)
           (transpose (cast f32 k)) * scale) masked_value))) v
   q, out: [batch..., Sq, D]; k, v: [batch..., Sk, D]; D in {32, 64, 128}; rows
   contiguous and 16-byte aligned, any other strides (head-split views are fine).
   `scale` and `masked_value` are float32 elements in host memory (the scalars
   of the float32 island), scale may be NULL. Either `mask` (bool,
   [batch..., Sq, Sk], stride-0 broadcast allowed) or `causal` != 0 (mask[i][j]
   = j <= i, generated; needs Sq == Sk and *masked_value == -inf, since key
   tiles above the diagonal are skipped; any other fill is Failure and the
   caller passes the mask tensor), or neither. */
int nxh_attention(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *q,
                  const nxh_tensor *k, const nxh_tensor *v, const void *scale,
                  const nxh_tensor *mask, const void *masked_value, int causal);

/* kaun/lib/linear.ml:50-52 (matmul, then the bias add) followed by the residual
   add of kaun/examples/04-gpt2/gpt2.ml:165-176, inside the GEMM's epilogue:
     out = (matmul x w + bias) + residual
   each of the three results rounded to the dtype as its primitive would store
   it, so the value equals the op-by-op one of this library bit for bit. bias:
   rank 1 of out's last extent, or NULL; residual: out's shape, or NULL (both
   NULL is nxh_matmul). f16 / bf16 / f32 operands that take the tiled MFMA GEMM
   (K a multiple of 128 bytes of k, 16-byte aligned rows, unit-stride output
   columns); otherwise Failure and the caller issues the primitives. */
int nxh_linear(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *x,
               const nxh_tensor *w, const nxh_tensor *bias, const nxh_tensor *residual);

/* nxh_linear without a residual followed by nxh_gelu_tanh (the first half of the MLP of
   kaun/examples/04-gpt2/gpt2.ml:165-176: Fn.gelu_approx (Linear.apply fc x)), the GELU
   applied in the GEMM's epilogue:
     out = gelu_tanh (matmul x w + bias)
   with every rounding of the eleven primitives it stands for, so the value equals the
   two calls' bit for bit. bfloat16 / float16 operands whose product is made of whole
   128 x 128 tiles (or, with a row-major x, 128 x 192 ones) with 16-byte aligned rows;
   anything else is Failure and the caller issues the two calls. `constants` as for nxh_gelu_tanh. */
int nxh_linear_gelu_tanh(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *x,
                         const nxh_tensor *w, const nxh_tensor *bias, const void *constants);

/* ── Fourier transforms ──────────────────────────────────────────────────── */

/* fft / ifft (backend_intf.ml:594-598; nx_backend.ml:507-528; nx_c_fft.c:940-956,
   1173-1182): complex64 / complex128, out has x's shape and dtype. UNNORMALISED
   (nx_c_fft.c:30-32): fft is the -sign DFT, ifft the +sign DFT without 1/n.
   One 1-D pass per entry of `axes`, in that order, the first reading x, the
   later ones transforming out in place; arithmetic in double, one rounding per
   pass on store. Any length up to 2^26 (2^25 when it is not a power of two). */
int nxh_fft(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *x,
            const int32_t *axes, int n_axes, int inverse);
/* rfft (backend_intf.ml:600-608; nx_backend.ml:530-536; nx_c_fft.c:958-982):
   x f32 / f64, out complex64 / complex128 with n/2+1 bins along the LAST listed
   axis, which is transformed first (from the real lines); the other listed axes
   follow as complex passes on out. */
int nxh_rfft(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *x,
             const int32_t *axes, int n_axes);
/* irfft (backend_intf.ml:610-623; nx_backend.ml:538-548; nx_c_fft.c:997-1144):
   x complex, out f32 / f64 of length s along the last listed axis, s = s_last
   when positive, else 2 (bins - 1). The other listed axes are transformed first
   (+sign, in complex128); then each line's spectrum of length s is rebuilt from
   min(bins, s/2+1) bins by conjugate symmetry (missing bins are zero) and the
   real part of its +sign transform is stored. */
int nxh_irfft(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *x,
              const int32_t *axes, int n_axes, int64_t s_last);

/* ── linear algebra ──────────────────────────────────────────────────────── */

/* The last two dims are the matrix, earlier dims the batch (backend_intf.ml:625-
   638). Storage dtypes f16 / bf16 / f32 / f64 / fp8 / complex64 / complex128;
   arithmetic in double. Numeric failures are Failure with the reference's status
   text as the message's tail (nx_c_linalg.h:29-36; nx_backend.ml:573-591 lifts
   them to Linalg_error by that suffix): "matrix is not positive definite",
   "triangular matrix is singular", "eigenvalue iteration did not converge".
   Every call waits for the stream (the failure belongs to the call). */

/* cholesky (backend_intf.ml:640-646; nx_c_tri.c:303-400): reads the lower
   triangle; out = L (upper == 0) or U = L^H, the other triangle zero. */
int nxh_cholesky(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *x, int upper);
/* triangular_solve (backend_intf.ml:703-720; nx_c_tri.c:88-118, 459-562): b and
   out are [..., n, nrhs] (a vector right-hand side is passed as one column,
   nx_backend.ml:598-611). flags: bit 0 upper, bit 1 transpose (the conjugate
   transpose for complex), bit 2 unit diagonal. An exactly zero pivot fails. */
int nxh_triangular_solve(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *a,
                         const nxh_tensor *b, int flags);
/* qr (backend_intf.ml:648-653; nx_c_qr.c:24-80; nx_backend.ml:613-626): q is
   [..., m, k] and r [..., k, n] when reduced (k = min(m, n)), else [..., m, m]
   and [..., m, n]. LAPACK's reflector convention, so R's diagonal is real. */
int nxh_qr(nxh_context *ctx, const nxh_tensor *q, const nxh_tensor *r, const nxh_tensor *x, int reduced);
/* eigh / eigvalsh (backend_intf.ml:685-701; nx_c_eigh.c:14-21; nx_backend.ml:628-
   649): reads the lower triangle; w [..., n] float64 ascending; v (may be null:
   values only) [..., n, n] of x's dtype, column k the unit eigenvector of w[k].
   n <= 4096. */
int nxh_eigh(nxh_context *ctx, const nxh_tensor *w, const nxh_tensor *v, const nxh_tensor *x);
/* svd (backend_intf.ml:655-664; nx_backend.ml:651-677): s [..., k] float64
   descending; u [..., m, k] and vt [..., k, n] (thin) or [..., m, m] and
   [..., n, n] (full), told apart by their shapes as in the reference. k <= 4096. */
int nxh_svd(nxh_context *ctx, const nxh_tensor *u, const nxh_tensor *s, const nxh_tensor *vt, const nxh_tensor *x);
/* eig / eigvals (backend_intf.ml:666-683; nx_c_eig.c:43-62; nx_backend.ml:679-
   707): w [..., n] and v [..., n, n] complex128 whatever x's dtype; v may be
   null (values only); eigenvectors have unit 2-norm, eigenvalues come in the
   order of the Schur factor's diagonal. n <= 2048. */
int nxh_eig(nxh_context *ctx, const nxh_tensor *w, const nxh_tensor *v, const nxh_tensor *x);

/* ── deferred evaluation ─────────────────────────────────────────────────── */

/* No counterpart in the reference, whose frontend lowers softmax, layer norm, GELU,
   attention and a linear layer to runs of primitives (frontend.ml:4242-4252,
   kaun/lib/layer_norm.ml:43-68, fn.ml:31-38, attention.ml:67-110, linear.ml:50-52)
   and whose backend runs each primitive as it is called. With the mode on,
   nxh_unary / nxh_binary / nxh_compare / nxh_where / nxh_cast / nxh_reduce /
   nxh_matmul / nxh_copy, a one-element nxh_fill and an nxh_memcpy_h2d of at most
   64 KiB (whose bytes are kept) only record their call. The record is
   executed, in issue order, by the next call of any other entry point (a host
   read and nxh_synchronize included), at a recorded copy once it holds 48
   entries (so that the device works while the host records on), or when it
   reaches 2048 entries. A run that
   spells one of those sequences, and whose intermediate results are read only
   inside the run, is replaced by the fused entry point below. An intermediate
   whose block was given back with nxh_free while recorded is never written; one
   whose block is still held when the record executes is postponed: it is
   written, as recorded, just before the first call that reads it (or that
   writes something it was computed from), and never if nxh_free comes first.
   So handles that are released late (finalisers) fuse like handles released at
   once. Observable results are the eager ones, except that an error of a
   recorded primitive is returned by the call that executes it, and that a
   fused row sum may be added in another order. nxh_free of a block that
   recorded or postponed work still uses takes effect once that work has run or
   been dropped. Switching the mode (either way) executes the record first, and
   switching it off writes everything postponed. Nothing is postponed while a
   graph is being captured. */
int nxh_set_deferred(nxh_context *ctx, int on);
/* Counters since the context was created, in this order. */
enum {
  NXH_DEFER_RECORDED = 0,   /* primitives recorded */
  NXH_DEFER_ISSUED,         /* primitives issued as recorded */
  NXH_DEFER_FLUSHES,        /* executions of a non-empty record */
  NXH_DEFER_FALLBACKS,      /* fused calls that were declined (the run was issued as recorded) */
  NXH_DEFER_SOFTMAX,        /* runs replaced by nxh_softmax_rows */
  NXH_DEFER_LAYER_NORM,     /* ... nxh_layer_norm_rows */
  NXH_DEFER_GELU,           /* ... nxh_gelu_tanh */
  NXH_DEFER_ATTENTION,      /* ... nxh_attention */
  NXH_DEFER_LINEAR,         /* ... nxh_linear */
  NXH_DEFER_POSTPONED,      /* entries of fused runs left unexecuted because their result was still held */
  NXH_DEFER_MATERIALISED,   /* of those, issued later because something read the result */
  NXH_DEFER_LINEAR_GELU,    /* runs replaced by nxh_linear_gelu_tanh (counted here only) */
  NXH_DEFER_GROUPED,        /* of the nxh_linear runs, those launched together with others that read the same x */
  NXH_DEFER_STAT_COUNT
};
int nxh_deferred_stats(nxh_context *ctx, uint64_t *stats, int count);

/* ── memory-side cache policy ────────────────────────────────────────────── */

/* No counterpart in the reference (a CPU's caches need no help from a backend).
   The MI355X keeps the last 256 MB read or written in a cache in front of HBM.
   While the tensors of the recent calls add up to more than that, the
   elementwise kernels write a result that was never read back while cached the
   last few times its block was written with non-temporal stores, and read an
   operand whose block was not read again in time with non-temporal loads, so
   that what the next call reads stays cached. The decision is per call, from a
   two-bit history per block of 8 MiB or more and the order of the calls; it
   changes when data reaches HBM, never a result. mode: bit 0 allows streaming
   loads, bit 1 streaming stores; 3 is the default, 0 turns the policy off (the
   environment variable NXH_CACHE_HINTS sets the initial value). Bit 2 makes
   every access stream that a kernel can stream, whatever the history and the
   size: for tests of those code paths. */
int nxh_set_cache_policy(nxh_context *ctx, int mode);
/* Calls so far whose inputs / whose result streamed past the cache. */
int nxh_cache_policy_stats(nxh_context *ctx, uint64_t *calls_streaming_in, uint64_t *calls_streaming_out);

/* ── recorded sequences ──────────────────────────────────────────────────── */

/* The reference backend has no counterpart: its eager calls cost a C stub
   each (nx_c_stubs.c), where a GPU call costs a launch of several
   microseconds, which a forward pass of small kernels (Kaun's GPT-2,
   kaun/examples/gpt2 via rune/lib/autodiff.ml's eager path) is bound by.
   Between nxh_capture_begin and nxh_capture_end every entry point above
   records its launches into a HIP graph instead of running them;
   nxh_graph_launch then replays them all with one call, in stream order with
   whatever else is issued on the context.
   - Storage allocated during the capture is the graph's: a tensor that lives on
     (the result) is overwritten by every replay, and its block returns to the
     allocator only after both nxh_free and nxh_graph_destroy. Storage that
     existed before (weights, inputs) is read at replay time as it then is:
     write new inputs into the same buffers (nxh_copy / nxh_memcpy_h2d)
     before a replay.
   - nxh_memcpy_h2d of up to 256 KiB is recorded with a private copy of the
     bytes. nxh_memcpy_d2h, nxh_synchronize, nxh_trim and the timer fail while
     capturing (Failure), and so does an allocation the driver refuses.
   - nxh_gather / nxh_scatter cannot report an index out of bounds from inside a
     capture: the out-of-range lanes are skipped as always, and the first
     nxh_synchronize after a replay that met one fails with Failure.
   - shapes, strides and scalars are frozen at capture; warm every entry point
     once eagerly before capturing it. */
typedef struct nxh_graph nxh_graph;
int nxh_capture_begin(nxh_context *ctx);
int nxh_capture_end(nxh_context *ctx, nxh_graph **graph);
int nxh_graph_launch(nxh_context *ctx, nxh_graph *graph);
/* Waits for the stream, then releases the graph and its idle storage. */
int nxh_graph_destroy(nxh_context *ctx, nxh_graph *graph);

/* ── measurement ─────────────────────────────────────────────────────────── */

/* HIP events recorded on the context stream: start, then stop returns the
   elapsed milliseconds between them after waiting for the stop event. */
int nxh_timer_start(nxh_context *ctx);
int nxh_timer_stop(nxh_context *ctx, float *milliseconds);
/* Name of the kernel path the last compute call on this thread selected
   (e.g. "map_contig", "map_tiled", "fold_row"), for tests and profiles. */
const char *nxh_last_path(nxh_context *ctx);

#ifdef __cplusplus
}
#endif
#endif /* NXHIP_H */
