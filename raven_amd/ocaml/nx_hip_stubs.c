/* nx_hip_stubs.c — OCaml foreign stubs over the libnxhip C ABI
   (include/nxhip.h). One CAMLprim per reference stub caml_nx_c_<op>
   (packages/nx/lib/backend_c/nx_backend.ml:104-168,242-264,349,395-397,
   482-483), same "output first" convention.

   Not compiled in this repository's image (no OCaml toolchain / caml headers);
   it is the binding a maintainer adds next to nx_backend.ml.

   The OCaml tensor handle is
     { buffer : dev; shape : int array; strides : int array; offset : int;
       tag : int; dtype; context }
   and, as in the reference (nx_c.h:47-61), C reads fixed slots: 0 buffer (a
   custom block holding the device pointer), 1 shape, 2 strides, 3 offset,
   4 dtype tag. */

#include <dlfcn.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <caml/alloc.h>
#include <caml/bigarray.h>
#include <caml/custom.h>
#include <caml/fail.h>
#include <caml/memory.h>
#include <caml/mlvalues.h>
#include <caml/threads.h>

#include "nxhip.h"

/* ── libnxhip.so, resolved once ──────────────────────────────────────────── */
#define NXH_SYMBOLS(X)                                                        \
  X(context_create) X(context_destroy) X(last_error) X(alloc) X(free)         \
  X(memcpy_h2d) X(memcpy_d2h) X(synchronize) X(fill) X(unary) X(binary)       \
  X(compare) X(where) X(cast) X(reduce) X(argreduce) X(matmul) X(copy)        \
  X(gather) X(scatter) X(pad) X(cat) X(scan) X(threefry) X(dtype_bytes)       \
  X(sort) X(argsort) X(unfold) X(fold) X(fft) X(rfft) X(irfft) X(cholesky)    \
  X(triangular_solve) X(qr) X(eigh) X(svd) X(eig) X(device_info)              \
  X(memory_stats) X(trim) X(reduce_noalloc) X(softmax_rows) X(layer_norm_rows) \
  X(gelu_tanh) X(attention) X(linear) X(linear_gelu_tanh) X(set_deferred) X(deferred_stats)        \
  X(set_cache_policy) X(cache_policy_stats)                                    \
  X(capture_begin) X(capture_end) X(graph_launch) X(graph_destroy)             \
  X(timer_start) X(timer_stop) X(last_path)
static struct {
#define X(n) __typeof__(nxh_##n) *n;
  NXH_SYMBOLS(X)
#undef X
} L;
static void *lib_handle;

static void load_library(void) {
  if (lib_handle) return;
  const char *path = getenv("NXHIP_LIBRARY");
  lib_handle = dlopen(path ? path : "libnxhip.so", RTLD_NOW | RTLD_LOCAL);
  if (!lib_handle) caml_failwith("create_context: cannot load libnxhip.so");
#define X(n)                                                       \
  L.n = (__typeof__(L.n))dlsym(lib_handle, "nxh_" #n);             \
  if (!L.n) caml_failwith("create_context: libnxhip.so lacks nxh_" #n);
  NXH_SYMBOLS(X)
#undef X
}

/* ── context, device buffers and graphs as custom blocks ─────────────────────
   The collector finalises blocks in no particular order, so the context is
   counted: its own block, every buffer and every graph hold one reference, and
   whichever is finalised last destroys it (a buffer finalised after the
   context block still finds its allocator). */
typedef struct {
  nxh_context *ctx;
  long refs;
} ctx_box;
#define Box_val(v) (*(ctx_box **)Data_custom_val(v))
#define Ctx_val(v) (Box_val(v)->ctx)
typedef struct {
  ctx_box *box;
  void *ptr;
  size_t bytes;
} dev_block;
#define Dev_val(v) ((dev_block *)Data_custom_val(v))
typedef struct {
  ctx_box *box;
  nxh_graph *graph;
} graph_block;
#define Graph_val(v) ((graph_block *)Data_custom_val(v))

static ctx_box *box_retain(ctx_box *b) {
  __atomic_add_fetch(&b->refs, 1, __ATOMIC_RELAXED);
  return b;
}
static void box_release(ctx_box *b) {
  if (__atomic_sub_fetch(&b->refs, 1, __ATOMIC_ACQ_REL) == 0) {
    L.context_destroy(b->ctx); /* waits for the stream, returns every block to the driver */
    free(b);
  }
}
static void ctx_finalize(value v) { box_release(Box_val(v)); }
static void dev_finalize(value v) {
  dev_block *d = Dev_val(v);
  if (d->ptr) L.free(d->box->ctx, d->ptr); /* stream-ordered inside the library */
  d->ptr = NULL;
  box_release(d->box);
}
static void graph_finalize(value v) {
  graph_block *g = Graph_val(v);
  if (g->graph) L.graph_destroy(g->box->ctx, g->graph);
  g->graph = NULL;
  box_release(g->box);
}
static struct custom_operations ctx_ops = {"nx_hip.context", ctx_finalize,
    custom_compare_default, custom_hash_default, custom_serialize_default,
    custom_deserialize_default, custom_compare_ext_default, custom_fixed_length_default};
static struct custom_operations dev_ops = {"nx_hip.buffer", dev_finalize,
    custom_compare_default, custom_hash_default, custom_serialize_default,
    custom_deserialize_default, custom_compare_ext_default, custom_fixed_length_default};
static struct custom_operations graph_ops = {"nx_hip.graph", graph_finalize,
    custom_compare_default, custom_hash_default, custom_serialize_default,
    custom_deserialize_default, custom_compare_ext_default, custom_fixed_length_default};

/* status -> exception, the reference's split (nx_c_engine.c:1345-1351) */
static void check(nxh_context *ctx, int rc) {
  if (rc == NXH_OK) return;
  const char *msg = L.last_error(ctx);
  if (rc == NXH_INVALID_ARGUMENT) caml_invalid_argument(msg);
  caml_failwith(msg);
}

CAMLprim value caml_nx_hip_create_context(value unit) {
  CAMLparam1(unit);
  CAMLlocal1(v);
  load_library();
  nxh_context *ctx = NULL;
  int rc = L.context_create(&ctx);
  if (rc != NXH_OK) caml_failwith(L.last_error(NULL));
  ctx_box *box = (ctx_box *)malloc(sizeof *box);
  if (!box) {
    L.context_destroy(ctx);
    caml_raise_out_of_memory();
  }
  box->ctx = ctx;
  box->refs = 1;
  v = caml_alloc_custom(&ctx_ops, sizeof(ctx_box *), 0, 1);
  Box_val(v) = box;
  CAMLreturn(v);
}

CAMLprim value caml_nx_hip_alloc(value vctx, value vbytes) {
  CAMLparam2(vctx, vbytes);
  CAMLlocal1(v);
  size_t bytes = (size_t)Long_val(vbytes);
  void *p = NULL;
  check(Ctx_val(vctx), L.alloc(Ctx_val(vctx), bytes, &p));
  /* caml_alloc_custom_mem lets the GC account for the device bytes */
  v = caml_alloc_custom_mem(&dev_ops, sizeof(dev_block), bytes);
  Dev_val(v)->box = box_retain(Box_val(vctx));
  Dev_val(v)->ptr = p;
  Dev_val(v)->bytes = bytes;
  CAMLreturn(v);
}

/* storage bytes of `count` elements of the dtype with this tag, as the library counts them */
CAMLprim value caml_nx_hip_dtype_bytes(value vtag, value vcount) {
  load_library();
  return Val_long((long)L.dtype_bytes(Int_val(vtag), (int64_t)Long_val(vcount)));
}
CAMLprim value caml_nx_hip_bytes(value vdev) { return Val_long((long)Dev_val(vdev)->bytes); }

/* from_host: the bigarray may be mutated or dropped as soon as this returns */
CAMLprim value caml_nx_hip_from_host(value vdev, value vba) {
  CAMLparam2(vdev, vba);
  dev_block *d = Dev_val(vdev);
  check(d->box->ctx, L.memcpy_h2d(d->box->ctx, d->ptr, Caml_ba_data_val(vba), d->bytes));
  CAMLreturn(Val_unit);
}

/* to_host: the whole backing storage; waits for the stream with the runtime
   lock released (the bigarray's data is malloc'd, so it does not move) */
CAMLprim value caml_nx_hip_to_host(value vba, value vdev) {
  CAMLparam2(vba, vdev);
  dev_block *d = Dev_val(vdev);
  void *dst = Caml_ba_data_val(vba);
  nxh_context *ctx = d->box->ctx;
  void *src = d->ptr;
  size_t n = d->bytes;
  caml_enter_blocking_section();
  int rc = L.memcpy_d2h(ctx, dst, src, n);
  caml_leave_blocking_section();
  check(ctx, rc);
  CAMLreturn(Val_unit);
}

/* ── operand extraction (nx_c.h:420-434) ─────────────────────────────────── */
static nxh_context *extract(value v, nxh_tensor *t) {
  value vs = Field(v, 1), vst = Field(v, 2);
  int nd = (int)Wosize_val(vs);
  if (nd > NXH_MAX_NDIM) caml_failwith("ndim exceeds NX_C_MAX_NDIM");
  if ((int)Wosize_val(vst) != nd) caml_failwith("shape and strides rank disagree");
  dev_block *d = Dev_val(Field(v, 0));
  t->data = d->ptr;
  t->ndim = nd;
  t->offset = Long_val(Field(v, 3));
  t->dtype = (int32_t)Long_val(Field(v, 4));
  for (int i = 0; i < nd; i++) {
    t->shape[i] = Long_val(Field(vs, i));
    t->strides[i] = Long_val(Field(vst, i));
  }
  return d->box->ctx;
}

#define UNARY_STUB(name, OP)                                              \
  CAMLprim value caml_nx_hip_##name(value vout, value vx) {               \
    CAMLparam2(vout, vx);                                                 \
    nxh_tensor o, x;                                                      \
    nxh_context *c = extract(vout, &o);                                   \
    extract(vx, &x);                                                      \
    check(c, L.unary(c, OP, &o, &x));                                     \
    CAMLreturn(Val_unit);                                                 \
  }
#define BINARY_STUB(name, OP)                                             \
  CAMLprim value caml_nx_hip_##name(value vout, value vx, value vy) {     \
    CAMLparam3(vout, vx, vy);                                             \
    nxh_tensor o, x, y;                                                   \
    nxh_context *c = extract(vout, &o);                                   \
    extract(vx, &x);                                                      \
    extract(vy, &y);                                                      \
    check(c, L.binary(c, OP, &o, &x, &y));                                \
    CAMLreturn(Val_unit);                                                 \
  }
#define COMPARE_STUB(name, OP)                                            \
  CAMLprim value caml_nx_hip_##name(value vout, value vx, value vy) {     \
    CAMLparam3(vout, vx, vy);                                             \
    nxh_tensor o, x, y;                                                   \
    nxh_context *c = extract(vout, &o);                                   \
    extract(vx, &x);                                                      \
    extract(vy, &y);                                                      \
    check(c, L.compare(c, OP, &o, &x, &y));                               \
    CAMLreturn(Val_unit);                                                 \
  }
UNARY_STUB(neg, NXH_NEG) UNARY_STUB(recip, NXH_RECIP) UNARY_STUB(abs, NXH_ABS)
UNARY_STUB(sign, NXH_SIGN) UNARY_STUB(sqrt, NXH_SQRT) UNARY_STUB(exp, NXH_EXP)
UNARY_STUB(log, NXH_LOG) UNARY_STUB(sin, NXH_SIN) UNARY_STUB(cos, NXH_COS)
UNARY_STUB(tan, NXH_TAN) UNARY_STUB(asin, NXH_ASIN) UNARY_STUB(acos, NXH_ACOS)
UNARY_STUB(atan, NXH_ATAN) UNARY_STUB(sinh, NXH_SINH) UNARY_STUB(cosh, NXH_COSH)
UNARY_STUB(tanh, NXH_TANH) UNARY_STUB(trunc, NXH_TRUNC) UNARY_STUB(ceil, NXH_CEIL)
UNARY_STUB(floor, NXH_FLOOR) UNARY_STUB(round, NXH_ROUND) UNARY_STUB(erf, NXH_ERF)
BINARY_STUB(add, NXH_ADD) BINARY_STUB(sub, NXH_SUB) BINARY_STUB(mul, NXH_MUL)
BINARY_STUB(idiv, NXH_IDIV) BINARY_STUB(fdiv, NXH_FDIV) BINARY_STUB(mod, NXH_MOD)
BINARY_STUB(pow, NXH_POW) BINARY_STUB(atan2, NXH_ATAN2) BINARY_STUB(max, NXH_MAX)
BINARY_STUB(min, NXH_MIN) BINARY_STUB(xor, NXH_XOR) BINARY_STUB(or, NXH_OR)
BINARY_STUB(and, NXH_AND)
COMPARE_STUB(cmpeq, NXH_CMPEQ) COMPARE_STUB(cmpne, NXH_CMPNE)
COMPARE_STUB(cmplt, NXH_CMPLT) COMPARE_STUB(cmple, NXH_CMPLE)

CAMLprim value caml_nx_hip_where(value vout, value vc, value va, value vb) {
  CAMLparam4(vout, vc, va, vb);
  nxh_tensor o, c, a, b;
  nxh_context *ctx = extract(vout, &o);
  extract(vc, &c);
  extract(va, &a);
  extract(vb, &b);
  check(ctx, L.where(ctx, &o, &c, &a, &b));
  CAMLreturn(Val_unit);
}
CAMLprim value caml_nx_hip_cast(value vout, value vx) {
  CAMLparam2(vout, vx);
  nxh_tensor o, x;
  nxh_context *c = extract(vout, &o);
  extract(vx, &x);
  check(c, L.cast(c, &o, &x));
  CAMLreturn(Val_unit);
}
CAMLprim value caml_nx_hip_copy(value vout, value vx) {
  CAMLparam2(vout, vx);
  nxh_tensor o, x;
  nxh_context *c = extract(vout, &o);
  extract(vx, &x);
  check(c, L.copy(c, &o, &x));
  CAMLreturn(Val_unit);
}
/* full: the value arrives as a one-element bigarray already encoded by
   Nx_buffer (so bf16/f16/fp8 use the buffer layer's converters) */
CAMLprim value caml_nx_hip_fill(value vout, value vba) {
  CAMLparam2(vout, vba);
  nxh_tensor o;
  nxh_context *c = extract(vout, &o);
  check(c, L.fill(c, &o, Caml_ba_data_val(vba)));
  CAMLreturn(Val_unit);
}
CAMLprim value caml_nx_hip_reduce(value vop, value vout, value vx, value vaxes) {
  CAMLparam4(vop, vout, vx, vaxes);
  nxh_tensor o, x;
  nxh_context *c = extract(vout, &o);
  extract(vx, &x);
  int n = (int)Wosize_val(vaxes);
  int32_t axes[NXH_MAX_NDIM];
  if (n > NXH_MAX_NDIM) caml_failwith("ndim exceeds NX_C_MAX_NDIM");
  for (int i = 0; i < n; i++) axes[i] = (int32_t)Long_val(Field(vaxes, i));
  check(c, L.reduce(c, Int_val(vop), &o, &x, axes, n));
  CAMLreturn(Val_unit);
}
CAMLprim value caml_nx_hip_argreduce(value vmin, value vout, value vx, value vaxis) {
  CAMLparam4(vmin, vout, vx, vaxis);
  nxh_tensor o, x;
  nxh_context *c = extract(vout, &o);
  extract(vx, &x);
  check(c, L.argreduce(c, Bool_val(vmin), &o, &x, Int_val(vaxis)));
  CAMLreturn(Val_unit);
}
CAMLprim value caml_nx_hip_matmul(value vout, value va, value vb) {
  CAMLparam3(vout, va, vb);
  nxh_tensor o, a, b;
  nxh_context *c = extract(vout, &o);
  extract(va, &a);
  extract(vb, &b);
  check(c, L.matmul(c, &o, &a, &b));
  CAMLreturn(Val_unit);
}
CAMLprim value caml_nx_hip_gather(value vout, value vdata, value vidx, value vaxis) {
  CAMLparam4(vout, vdata, vidx, vaxis);
  nxh_tensor o, d, i;
  nxh_context *c = extract(vout, &o);
  extract(vdata, &d);
  extract(vidx, &i);
  /* waits for the stream to report an out-of-range index from this call */
  caml_enter_blocking_section();
  int rc = L.gather(c, &o, &d, &i, Int_val(vaxis));
  caml_leave_blocking_section();
  check(c, rc);
  CAMLreturn(Val_unit);
}
CAMLprim value caml_nx_hip_scatter(value vout, value vidx, value vupd, value vaxis, value vmode) {
  CAMLparam5(vout, vidx, vupd, vaxis, vmode);
  nxh_tensor o, i, u;
  nxh_context *c = extract(vout, &o);
  extract(vidx, &i);
  extract(vupd, &u);
  /* waits for the stream to report an out-of-range index from this call */
  caml_enter_blocking_section();
  int rc = L.scatter(c, &o, &i, &u, Int_val(vaxis), Int_val(vmode));
  caml_leave_blocking_section();
  check(c, rc);
  CAMLreturn(Val_unit);
}
/* the fill value arrives as a 1-element host Nx_buffer, like caml_nx_hip_fill */
CAMLprim value caml_nx_hip_pad(value vout, value vx, value vfill, value vbefore) {
  CAMLparam4(vout, vx, vfill, vbefore);
  nxh_tensor o, x;
  nxh_context *c = extract(vout, &o);
  extract(vx, &x);
  int n = (int)Wosize_val(vbefore);
  int64_t before[NXH_MAX_NDIM];
  if (n > NXH_MAX_NDIM) caml_failwith("ndim exceeds NX_C_MAX_NDIM");
  for (int d = 0; d < n; d++) before[d] = Long_val(Field(vbefore, d));
  if (n != o.ndim) caml_invalid_argument("pad: shape mismatch");
  check(c, L.pad(c, &o, &x, Caml_ba_data_val(vfill), before));
  CAMLreturn(Val_unit);
}
CAMLprim value caml_nx_hip_cat(value vout, value vinputs, value vaxis) {
  CAMLparam3(vout, vinputs, vaxis);
  nxh_tensor o;
  nxh_context *c = extract(vout, &o);
  int n = (int)Wosize_val(vinputs);
  nxh_tensor *members = (nxh_tensor *)caml_stat_alloc(sizeof(nxh_tensor) * (size_t)(n > 0 ? n : 1));
  const nxh_tensor **ptrs = (const nxh_tensor **)caml_stat_alloc(sizeof(nxh_tensor *) * (size_t)(n > 0 ? n : 1));
  for (int m = 0; m < n; m++) {
    extract(Field(vinputs, m), &members[m]);
    ptrs[m] = &members[m];
  }
  int rc = L.cat(c, &o, ptrs, n, Int_val(vaxis));
  caml_stat_free(ptrs);
  caml_stat_free(members);
  check(c, rc);
  CAMLreturn(Val_unit);
}
CAMLprim value caml_nx_hip_scan(value vop, value vout, value vx, value vaxis) {
  CAMLparam4(vop, vout, vx, vaxis);
  nxh_tensor o, x;
  nxh_context *c = extract(vout, &o);
  extract(vx, &x);
  check(c, L.scan(c, Int_val(vop), &o, &x, Int_val(vaxis)));
  CAMLreturn(Val_unit);
}
CAMLprim value caml_nx_hip_threefry(value vout, value vkey, value vctr) {
  CAMLparam3(vout, vkey, vctr);
  nxh_tensor o, k, t;
  nxh_context *c = extract(vout, &o);
  extract(vkey, &k);
  extract(vctr, &t);
  check(c, L.threefry(c, &o, &k, &t));
  CAMLreturn(Val_unit);
}

/* sort / argsort: same shape as caml_nx_c_sort / caml_nx_c_argsort (nx_c_sort.c:472-514) */
CAMLprim value caml_nx_hip_sort(value vout, value vx, value vaxis, value vdesc) {
  CAMLparam4(vout, vx, vaxis, vdesc);
  nxh_tensor o, x;
  nxh_context *c = extract(vout, &o);
  extract(vx, &x);
  check(c, L.sort(c, &o, &x, Int_val(vaxis), Bool_val(vdesc)));
  CAMLreturn(Val_unit);
}
CAMLprim value caml_nx_hip_argsort(value vout, value vx, value vaxis, value vdesc) {
  CAMLparam4(vout, vx, vaxis, vdesc);
  nxh_tensor o, x;
  nxh_context *c = extract(vout, &o);
  extract(vx, &x);
  check(c, L.argsort(c, &o, &x, Int_val(vaxis), Bool_val(vdesc)));
  CAMLreturn(Val_unit);
}

/* int array -> int64_t[], at most `cap` entries; returns the length */
static int long_array(value v, int64_t *dst, int cap) {
  int n = (int)Wosize_val(v);
  if (n > cap) caml_failwith("ndim exceeds NX_C_MAX_NDIM");
  for (int i = 0; i < n; i++) dst[i] = Long_val(Field(v, i));
  return n;
}
/* windows: arguments as caml_nx_c_unfold / caml_nx_c_fold (nx_c_move.c:789-870),
   padding already flattened to [before0; after0; ...] by the OCaml side */
CAMLprim value caml_nx_hip_unfold(value vout, value vx, value vkernel, value vstride, value vdilation,
                                  value vpadding) {
  CAMLparam5(vout, vx, vkernel, vstride, vdilation);
  CAMLxparam1(vpadding);
  nxh_tensor o, x;
  nxh_context *c = extract(vout, &o);
  extract(vx, &x);
  int64_t kernel[NXH_MAX_NDIM], stride[NXH_MAX_NDIM], dilation[NXH_MAX_NDIM], padding[2 * NXH_MAX_NDIM];
  int k = long_array(vkernel, kernel, NXH_MAX_NDIM);
  if (long_array(vstride, stride, NXH_MAX_NDIM) != k || long_array(vdilation, dilation, NXH_MAX_NDIM) != k ||
      long_array(vpadding, padding, 2 * NXH_MAX_NDIM) != 2 * k)
    caml_invalid_argument("unfold: shape mismatch");
  check(c, L.unfold(c, &o, &x, k, kernel, stride, dilation, padding));
  CAMLreturn(Val_unit);
}
CAMLprim value caml_nx_hip_unfold_bc(value *argv, int argn) {
  (void)argn;
  return caml_nx_hip_unfold(argv[0], argv[1], argv[2], argv[3], argv[4], argv[5]);
}
CAMLprim value caml_nx_hip_fold(value vout, value vx, value vosize, value vkernel, value vstride,
                                value vdilation, value vpadding) {
  CAMLparam5(vout, vx, vosize, vkernel, vstride);
  CAMLxparam2(vdilation, vpadding);
  nxh_tensor o, x;
  nxh_context *c = extract(vout, &o);
  extract(vx, &x);
  int64_t osize[NXH_MAX_NDIM], kernel[NXH_MAX_NDIM], stride[NXH_MAX_NDIM], dilation[NXH_MAX_NDIM],
      padding[2 * NXH_MAX_NDIM];
  int k = long_array(vkernel, kernel, NXH_MAX_NDIM);
  if (long_array(vosize, osize, NXH_MAX_NDIM) != k || long_array(vstride, stride, NXH_MAX_NDIM) != k ||
      long_array(vdilation, dilation, NXH_MAX_NDIM) != k || long_array(vpadding, padding, 2 * NXH_MAX_NDIM) != 2 * k)
    caml_invalid_argument("fold: shape mismatch");
  check(c, L.fold(c, &o, &x, k, osize, kernel, stride, dilation, padding));
  CAMLreturn(Val_unit);
}
CAMLprim value caml_nx_hip_fold_bc(value *argv, int argn) {
  (void)argn;
  return caml_nx_hip_fold(argv[0], argv[1], argv[2], argv[3], argv[4], argv[5], argv[6]);
}

/* ── Fourier transforms: arguments as caml_nx_c_fft / _ifft / _rfft / _irfft
   (nx_c_fft.c:1159-1230); axes is an OCaml int array, s the optional sizes
   (empty = inferred), of which only the last entry is read ─────────────── */
static int axes_array(value v, int32_t *dst) {
  int n = (int)Wosize_val(v);
  if (n > NXH_MAX_NDIM) caml_failwith("ndim exceeds NX_C_MAX_NDIM");
  for (int i = 0; i < n; i++) dst[i] = (int32_t)Long_val(Field(v, i));
  return n;
}
static value fft_common(value vout, value vx, value vaxes, int inverse) {
  CAMLparam3(vout, vx, vaxes);
  nxh_tensor o, x;
  nxh_context *c = extract(vout, &o);
  extract(vx, &x);
  int32_t axes[NXH_MAX_NDIM];
  int n = axes_array(vaxes, axes);
  check(c, L.fft(c, &o, &x, axes, n, inverse));
  CAMLreturn(Val_unit);
}
CAMLprim value caml_nx_hip_fft(value vout, value vx, value vaxes) { return fft_common(vout, vx, vaxes, 0); }
CAMLprim value caml_nx_hip_ifft(value vout, value vx, value vaxes) { return fft_common(vout, vx, vaxes, 1); }
CAMLprim value caml_nx_hip_rfft(value vout, value vx, value vaxes) {
  CAMLparam3(vout, vx, vaxes);
  nxh_tensor o, x;
  nxh_context *c = extract(vout, &o);
  extract(vx, &x);
  int32_t axes[NXH_MAX_NDIM];
  int n = axes_array(vaxes, axes);
  check(c, L.rfft(c, &o, &x, axes, n));
  CAMLreturn(Val_unit);
}
CAMLprim value caml_nx_hip_irfft(value vout, value vx, value vaxes, value vs) {
  CAMLparam4(vout, vx, vaxes, vs);
  nxh_tensor o, x;
  nxh_context *c = extract(vout, &o);
  extract(vx, &x);
  int32_t axes[NXH_MAX_NDIM];
  int n = axes_array(vaxes, axes);
  int ns = (int)Wosize_val(vs);
  int64_t s_last = ns > 0 ? (int64_t)Long_val(Field(vs, ns - 1)) : 0;
  check(c, L.irfft(c, &o, &x, axes, n, s_last));
  CAMLreturn(Val_unit);
}

/* ── linear algebra: arguments as the reference's stubs (nx_c_tri.c:564-600,
   nx_c_qr.c, nx_c_eigh.c:1765-, nx_c_svd.c, nx_c_eig.c:1324-). These calls wait
   for the stream (a numeric failure belongs to the call), so the runtime lock is
   released around them ───────────────────────────────────────────────────── */
#define BLOCKING(call)                \
  do {                                \
    caml_release_runtime_system();    \
    int rc__ = (call);                \
    caml_acquire_runtime_system();    \
    check(c, rc__);                   \
  } while (0)

CAMLprim value caml_nx_hip_cholesky(value vout, value vx, value vupper) {
  CAMLparam3(vout, vx, vupper);
  nxh_tensor o, x;
  nxh_context *c = extract(vout, &o);
  extract(vx, &x);
  int upper = Bool_val(vupper);
  BLOCKING(L.cholesky(c, &o, &x, upper));
  CAMLreturn(Val_unit);
}
CAMLprim value caml_nx_hip_triangular_solve(value vout, value va, value vb, value vflags) {
  CAMLparam4(vout, va, vb, vflags);
  nxh_tensor o, a, b;
  nxh_context *c = extract(vout, &o);
  extract(va, &a);
  extract(vb, &b);
  int flags = Int_val(vflags);
  BLOCKING(L.triangular_solve(c, &o, &a, &b, flags));
  CAMLreturn(Val_unit);
}
CAMLprim value caml_nx_hip_qr(value vq, value vr, value vx, value vreduced) {
  CAMLparam4(vq, vr, vx, vreduced);
  nxh_tensor q, r, x;
  nxh_context *c = extract(vq, &q);
  extract(vr, &r);
  extract(vx, &x);
  int reduced = Bool_val(vreduced);
  BLOCKING(L.qr(c, &q, &r, &x, reduced));
  CAMLreturn(Val_unit);
}
/* vectors = false: the eigenvector slot holds the input again and is not read
   (nx_backend.ml:566-571, 679-689) */
CAMLprim value caml_nx_hip_eigh(value vw, value vv, value vx, value vvectors) {
  CAMLparam4(vw, vv, vx, vvectors);
  nxh_tensor w, v, x;
  nxh_context *c = extract(vw, &w);
  extract(vv, &v);
  extract(vx, &x);
  int vectors = Bool_val(vvectors);
  BLOCKING(L.eigh(c, &w, vectors ? &v : NULL, &x));
  CAMLreturn(Val_unit);
}
CAMLprim value caml_nx_hip_svd(value vu, value vs, value vvt, value vx) {
  CAMLparam4(vu, vs, vvt, vx);
  nxh_tensor u, s, vt, x;
  nxh_context *c = extract(vu, &u);
  extract(vs, &s);
  extract(vvt, &vt);
  extract(vx, &x);
  BLOCKING(L.svd(c, &u, &s, &vt, &x));
  CAMLreturn(Val_unit);
}
CAMLprim value caml_nx_hip_eig(value vw, value vv, value vx, value vvectors) {
  CAMLparam4(vw, vv, vx, vvectors);
  nxh_tensor w, v, x;
  nxh_context *c = extract(vw, &w);
  extract(vv, &v);
  extract(vx, &x);
  int vectors = Bool_val(vvectors);
  BLOCKING(L.eig(c, &w, vectors ? &v : NULL, &x));
  CAMLreturn(Val_unit);
}

/* ── what the reference backend has no stub for ─────────────────────────────
   Context services, the call that allocates nothing, the fused entry points,
   deferred evaluation and recorded sequences. The frontend reaches the fused
   kernels without any of the five fused stubs: with set_deferred on, the
   primitive stubs above record, and the library replaces the runs it recognises.
   The fused stubs are for callers that name the operation themselves. */

CAMLprim value caml_nx_hip_synchronize(value vctx) {
  CAMLparam1(vctx);
  nxh_context *c = Ctx_val(vctx);
  BLOCKING(L.synchronize(c));
  CAMLreturn(Val_unit);
}
CAMLprim value caml_nx_hip_trim(value vctx) {
  CAMLparam1(vctx);
  nxh_context *c = Ctx_val(vctx);
  BLOCKING(L.trim(c));
  CAMLreturn(Val_unit);
}
/* (device ordinal, device name, compute units) */
CAMLprim value caml_nx_hip_device_info(value vctx) {
  CAMLparam1(vctx);
  CAMLlocal2(v, vname);
  int device = 0, units = 0;
  char name[256];
  check(Ctx_val(vctx), L.device_info(Ctx_val(vctx), &device, name, sizeof name, &units));
  vname = caml_copy_string(name);
  v = caml_alloc_tuple(3);
  Store_field(v, 0, Val_int(device));
  Store_field(v, 1, vname);
  Store_field(v, 2, Val_int(units));
  CAMLreturn(v);
}
/* [| in_use; cached; reserved; driver_allocs |] */
CAMLprim value caml_nx_hip_memory_stats(value vctx) {
  CAMLparam1(vctx);
  CAMLlocal1(v);
  uint64_t s[4] = {0, 0, 0, 0};
  check(Ctx_val(vctx), L.memory_stats(Ctx_val(vctx), &s[0], &s[1], &s[2], &s[3]));
  v = caml_alloc_tuple(4);
  for (int i = 0; i < 4; i++) Store_field(v, i, Val_long((long)s[i]));
  CAMLreturn(v);
}
CAMLprim value caml_nx_hip_last_path(value vctx) {
  CAMLparam1(vctx);
  const char *p = L.last_path(Ctx_val(vctx));
  CAMLreturn(caml_copy_string(p ? p : ""));
}
CAMLprim value caml_nx_hip_timer_start(value vctx) {
  CAMLparam1(vctx);
  check(Ctx_val(vctx), L.timer_start(Ctx_val(vctx)));
  CAMLreturn(Val_unit);
}
CAMLprim value caml_nx_hip_timer_stop(value vctx) {
  CAMLparam1(vctx);
  nxh_context *c = Ctx_val(vctx);
  float ms = 0.0f;
  BLOCKING(L.timer_stop(c, &ms));
  CAMLreturn(caml_copy_double((double)ms));
}

CAMLprim value caml_nx_hip_reduce_noalloc(value vop, value vout, value vx, value vaxes) {
  CAMLparam4(vop, vout, vx, vaxes);
  nxh_tensor o, x;
  nxh_context *c = extract(vout, &o);
  extract(vx, &x);
  int32_t axes[NXH_MAX_NDIM];
  int n = axes_array(vaxes, axes);
  check(c, L.reduce_noalloc(c, Int_val(vop), &o, &x, axes, n));
  CAMLreturn(Val_unit);
}

/* an OCaml `'a t option` as a descriptor pointer or NULL; a `buffer option`
   (a one-element host Nx_buffer holding an encoded scalar) as its bytes or NULL */
static const nxh_tensor *optional(value v, nxh_tensor *slot) {
  if (!Is_block(v)) return NULL;
  extract(Field(v, 0), slot);
  return slot;
}
static const void *optional_bytes(value v) { return Is_block(v) ? Caml_ba_data_val(Field(v, 0)) : NULL; }

CAMLprim value caml_nx_hip_softmax_rows(value vout, value vx, value vscale, value vmask, value vfill) {
  CAMLparam5(vout, vx, vscale, vmask, vfill);
  nxh_tensor o, x, m;
  nxh_context *c = extract(vout, &o);
  extract(vx, &x);
  check(c, L.softmax_rows(c, &o, &x, optional_bytes(vscale), optional(vmask, &m), optional_bytes(vfill)));
  CAMLreturn(Val_unit);
}
CAMLprim value caml_nx_hip_layer_norm_rows(value vout, value vx, value vgamma, value vbeta, value veps) {
  CAMLparam5(vout, vx, vgamma, vbeta, veps);
  nxh_tensor o, x, g, b;
  nxh_context *c = extract(vout, &o);
  extract(vx, &x);
  check(c, L.layer_norm_rows(c, &o, &x, optional(vgamma, &g), optional(vbeta, &b), Double_val(veps)));
  CAMLreturn(Val_unit);
}
/* constants: a four-element host Nx_buffer of x's dtype (c0..c3 of fn.ml:31-38) */
CAMLprim value caml_nx_hip_gelu_tanh(value vout, value vx, value vconstants) {
  CAMLparam3(vout, vx, vconstants);
  nxh_tensor o, x;
  nxh_context *c = extract(vout, &o);
  extract(vx, &x);
  check(c, L.gelu_tanh(c, &o, &x, Caml_ba_data_val(vconstants)));
  CAMLreturn(Val_unit);
}
/* scale, fill: one-element float32 host buffers */
CAMLprim value caml_nx_hip_attention(value vout, value vq, value vk, value vv, value vscale, value vmask,
                                     value vfill, value vcausal) {
  CAMLparam5(vout, vq, vk, vv, vscale);
  CAMLxparam3(vmask, vfill, vcausal);
  nxh_tensor o, q, k, v, m;
  nxh_context *c = extract(vout, &o);
  extract(vq, &q);
  extract(vk, &k);
  extract(vv, &v);
  check(c, L.attention(c, &o, &q, &k, &v, optional_bytes(vscale), optional(vmask, &m), optional_bytes(vfill),
                       Bool_val(vcausal)));
  CAMLreturn(Val_unit);
}
CAMLprim value caml_nx_hip_attention_bc(value *argv, int argn) {
  (void)argn;
  return caml_nx_hip_attention(argv[0], argv[1], argv[2], argv[3], argv[4], argv[5], argv[6], argv[7]);
}
CAMLprim value caml_nx_hip_linear(value vout, value vx, value vw, value vbias, value vresidual) {
  CAMLparam5(vout, vx, vw, vbias, vresidual);
  nxh_tensor o, x, w, b, r;
  nxh_context *c = extract(vout, &o);
  extract(vx, &x);
  extract(vw, &w);
  check(c, L.linear(c, &o, &x, &w, optional(vbias, &b), optional(vresidual, &r)));
  CAMLreturn(Val_unit);
}

/* constants: as for caml_nx_hip_gelu_tanh */
CAMLprim value caml_nx_hip_linear_gelu_tanh(value vout, value vx, value vw, value vbias, value vconstants) {
  CAMLparam5(vout, vx, vw, vbias, vconstants);
  nxh_tensor o, x, w, b;
  nxh_context *c = extract(vout, &o);
  extract(vx, &x);
  extract(vw, &w);
  check(c, L.linear_gelu_tanh(c, &o, &x, &w, optional(vbias, &b), Caml_ba_data_val(vconstants)));
  CAMLreturn(Val_unit);
}

CAMLprim value caml_nx_hip_set_deferred(value vctx, value von) {
  CAMLparam2(vctx, von);
  check(Ctx_val(vctx), L.set_deferred(Ctx_val(vctx), Bool_val(von)));
  CAMLreturn(Val_unit);
}
/* the counters of nxhip.h, in its order */
CAMLprim value caml_nx_hip_deferred_stats(value vctx) {
  CAMLparam1(vctx);
  CAMLlocal1(v);
  uint64_t s[NXH_DEFER_STAT_COUNT];
  check(Ctx_val(vctx), L.deferred_stats(Ctx_val(vctx), s, NXH_DEFER_STAT_COUNT));
  v = caml_alloc_tuple(NXH_DEFER_STAT_COUNT);
  for (int i = 0; i < NXH_DEFER_STAT_COUNT; i++) Store_field(v, i, Val_long((long)s[i]));
  CAMLreturn(v);
}

/* bit 0: streaming loads, bit 1: streaming stores of blocks that are not touched again while cached */
CAMLprim value caml_nx_hip_set_cache_policy(value vctx, value vmode) {
  CAMLparam2(vctx, vmode);
  check(Ctx_val(vctx), L.set_cache_policy(Ctx_val(vctx), Int_val(vmode)));
  CAMLreturn(Val_unit);
}
/* (calls whose inputs streamed, calls whose result streamed) */
CAMLprim value caml_nx_hip_cache_policy_stats(value vctx) {
  CAMLparam1(vctx);
  CAMLlocal1(v);
  uint64_t in = 0, out = 0;
  check(Ctx_val(vctx), L.cache_policy_stats(Ctx_val(vctx), &in, &out));
  v = caml_alloc_tuple(2);
  Store_field(v, 0, Val_long((long)in));
  Store_field(v, 1, Val_long((long)out));
  CAMLreturn(v);
}

CAMLprim value caml_nx_hip_capture_begin(value vctx) {
  CAMLparam1(vctx);
  check(Ctx_val(vctx), L.capture_begin(Ctx_val(vctx)));
  CAMLreturn(Val_unit);
}
CAMLprim value caml_nx_hip_capture_end(value vctx) {
  CAMLparam1(vctx);
  CAMLlocal1(v);
  nxh_graph *g = NULL;
  check(Ctx_val(vctx), L.capture_end(Ctx_val(vctx), &g));
  v = caml_alloc_custom(&graph_ops, sizeof(graph_block), 0, 1);
  Graph_val(v)->box = box_retain(Box_val(vctx));
  Graph_val(v)->graph = g;
  CAMLreturn(v);
}
CAMLprim value caml_nx_hip_graph_launch(value vgraph) {
  CAMLparam1(vgraph);
  graph_block *g = Graph_val(vgraph);
  if (!g->graph) caml_invalid_argument("graph_launch: the graph was destroyed");
  check(g->box->ctx, L.graph_launch(g->box->ctx, g->graph));
  CAMLreturn(Val_unit);
}
/* releases the recorded launches and the storage they pinned now rather than at collection */
CAMLprim value caml_nx_hip_graph_destroy(value vgraph) {
  CAMLparam1(vgraph);
  graph_block *g = Graph_val(vgraph);
  if (g->graph) {
    nxh_graph *graph = g->graph;
    g->graph = NULL;
    check(g->box->ctx, L.graph_destroy(g->box->ctx, graph));
  }
  CAMLreturn(Val_unit);
}
