/* nx_host.h: the part of the Nx frontend that Kaun's GPT-2 needs, lowered to
   backend primitives exactly as packages/nx/lib/core/frontend.ml lowers it, in
   plain C over the libnxhip C ABI. One library call per primitive, a fresh
   output block per result, a free when the last reference goes: what the OCaml
   binding does, at the cost of a compiled host (no interpreter between calls).

   A value is a view (nxh_tensor) plus the block behind it. Blocks are counted
   by hand: every function below gives back what it allocated for its own
   intermediates as soon as they have been used, like a frontend whose handles
   die at scope exit; with nxhost_late_frees set they are given back only by
   nxhost_collect(), like handles that wait for a garbage collector. */

#ifndef NX_HOST_H
#define NX_HOST_H

#include <dlfcn.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "nxhip.h"

#define NXHOST_SYMBOLS(X)                                                                  \
  X(context_create) X(context_destroy) X(last_error) X(alloc) X(free) X(memcpy_h2d)        \
  X(memcpy_d2h) X(synchronize) X(fill) X(unary) X(binary) X(compare) X(where) X(cast)      \
  X(reduce) X(matmul) X(copy) X(gather) X(capture_begin) X(capture_end) X(graph_launch)    \
  X(graph_destroy) X(set_deferred) X(deferred_stats) X(timer_start) X(timer_stop)          \
  X(memory_stats) X(device_info)
static struct {
#define X(n) __typeof__(nxh_##n) *n;
  NXHOST_SYMBOLS(X)
#undef X
} L;

static nxh_context *ctx;

static void nxhost_open(const char *path) {
  void *h = dlopen(path, RTLD_NOW | RTLD_LOCAL);
  if (!h) {
    fprintf(stderr, "dlopen: %s\n", dlerror());
    exit(2);
  }
#define X(n)                                      \
  L.n = (__typeof__(L.n))dlsym(h, "nxh_" #n);     \
  if (!L.n) {                                     \
    fprintf(stderr, "missing nxh_" #n "\n");      \
    exit(2);                                      \
  }
  NXHOST_SYMBOLS(X)
#undef X
  if (L.context_create(&ctx) != NXH_OK) {
    fprintf(stderr, "create_context: %s\n", L.last_error(NULL));
    exit(2);
  }
}

static void must(int rc, const char *what) {
  if (rc != NXH_OK) {
    fprintf(stderr, "%s: status %d: %s\n", what, rc, L.last_error(ctx));
    exit(2);
  }
}

/* ── values ─────────────────────────────────────────────────────────────── */
typedef struct {
  nxh_tensor t;
  void *block;
} val;

static int nxhost_late_frees;
static void **nxhost_pending;
static size_t nxhost_n_pending, nxhost_cap_pending;

static size_t elem_size(int dtype) {
  switch (dtype) {
    case NXH_F64: case NXH_I64: case NXH_U64: case NXH_C32: return 8;
    case NXH_F32: case NXH_I32: case NXH_U32: return 4;
    case NXH_F16: case NXH_BF16: case NXH_I16: case NXH_U16: return 2;
    default: return 1;
  }
}
static int64_t numel(const nxh_tensor *t) {
  int64_t n = 1;
  for (int d = 0; d < t->ndim; d++) n *= t->shape[d];
  return n;
}
static nxh_tensor contiguous_desc(void *data, int dtype, int ndim, const int64_t *shape) {
  nxh_tensor t;
  memset(&t, 0, sizeof t);
  t.data = data, t.dtype = dtype, t.ndim = ndim;
  int64_t stride = 1;
  for (int d = ndim - 1; d >= 0; d--) t.shape[d] = shape[d], t.strides[d] = stride, stride *= shape[d];
  return t;
}
static val fresh(int dtype, int ndim, const int64_t *shape) {
  val v;
  size_t n = 1;
  for (int d = 0; d < ndim; d++) n *= (size_t)shape[d];
  must(L.alloc(ctx, n * elem_size(dtype), &v.block), "buffer");
  v.t = contiguous_desc(v.block, dtype, ndim, shape);
  return v;
}
static void drop(val v) {
  if (!nxhost_late_frees) {
    must(L.free(ctx, v.block), "free");
    return;
  }
  if (nxhost_n_pending == nxhost_cap_pending) {
    nxhost_cap_pending = nxhost_cap_pending ? 2 * nxhost_cap_pending : 4096;
    nxhost_pending = (void **)realloc(nxhost_pending, nxhost_cap_pending * sizeof(void *));
  }
  nxhost_pending[nxhost_n_pending++] = v.block;
}
/* the collector runs: every handle dropped since the last run is finalised */
static void nxhost_collect(void) {
  for (size_t i = 0; i < nxhost_n_pending; i++) must(L.free(ctx, nxhost_pending[i]), "free");
  nxhost_n_pending = 0;
}
static val from_host(const void *host, int dtype, int ndim, const int64_t *shape) {
  val v = fresh(dtype, ndim, shape);
  must(L.memcpy_h2d(ctx, v.block, host, (size_t)numel(&v.t) * elem_size(dtype)), "from_host");
  return v;
}

/* ── views (view.ml) ────────────────────────────────────────────────────── */
/* expand: leading extents are added, an extent of 1 is repeated with stride 0 */
static nxh_tensor expand(nxh_tensor t, int ndim, const int64_t *shape) {
  nxh_tensor r = t;
  const int pad = ndim - t.ndim;
  r.ndim = ndim;
  for (int d = 0; d < ndim; d++) {
    const int64_t have = d < pad ? 1 : t.shape[d - pad];
    r.strides[d] = (d < pad || (have == 1 && shape[d] != 1)) ? 0 : t.strides[d - pad];
    r.shape[d] = shape[d];
  }
  return r;
}
/* reshape of a C-contiguous view */
static nxh_tensor reshape(nxh_tensor t, int ndim, const int64_t *shape) {
  return contiguous_desc(t.data, t.dtype, ndim, shape);
}
static nxh_tensor keep_last(nxh_tensor t) { /* [.., R] -> [.., R, 1] */
  t.shape[t.ndim] = 1, t.strides[t.ndim] = 1, t.ndim++;
  return t;
}
static nxh_tensor swapaxes(nxh_tensor t, int a, int b) {
  int64_t s = t.shape[a], st = t.strides[a];
  t.shape[a] = t.shape[b], t.strides[a] = t.strides[b];
  t.shape[b] = s, t.strides[b] = st;
  return t;
}

/* ── scalars in a dtype's storage format (the buffer layer's converters) ─── */
static uint16_t bf16_of(float f) { /* round to nearest even; finite or infinite inputs */
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
  return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}
static void encode_scalar(int dtype, double value, void *element) {
  if (dtype == NXH_F32) {
    float f = (float)value;
    memcpy(element, &f, 4);
  } else if (dtype == NXH_BF16) {
    uint16_t h = bf16_of((float)value);
    memcpy(element, &h, 2);
  } else if (dtype == NXH_F64) {
    memcpy(element, &value, 8);
  } else {
    fprintf(stderr, "encode_scalar: dtype %d\n", dtype);
    exit(2);
  }
}

/* ── primitives: allocate the result, one library call ──────────────────── */
static val scalar(int dtype, double value) { /* frontend.ml:360: full ctx dt [||] value */
  unsigned char element[8];
  encode_scalar(dtype, value, element);
  val v = fresh(dtype, 0, NULL);
  must(L.fill(ctx, &v.t, element), "full");
  return v;
}
static val un(int op, nxh_tensor x) {
  val o = fresh(x.dtype, x.ndim, x.shape);
  must(L.unary(ctx, op, &o.t, &x), "unary");
  return o;
}
static val bin(int op, nxh_tensor x, nxh_tensor y) { /* operands already broadcast to one shape */
  val o = fresh(x.dtype, x.ndim, x.shape);
  must(L.binary(ctx, op, &o.t, &x, &y), "binary");
  return o;
}
static val cast_to(int dtype, nxh_tensor x) {
  val o = fresh(dtype, x.ndim, x.shape);
  must(L.cast(ctx, &o.t, &x), "cast");
  return o;
}
static val fold_last(int op, nxh_tensor x) {
  int32_t axis = x.ndim - 1;
  val o = fresh(x.dtype, x.ndim - 1, x.shape);
  must(L.reduce(ctx, op, &o.t, &x, &axis, 1), "reduce");
  return o;
}
static val matmul(nxh_tensor a, nxh_tensor b) { /* frontend.ml:2346-2352, equal ranks or a rank-2 b */
  int64_t shape[NXH_MAX_NDIM];
  memcpy(shape, a.shape, sizeof shape);
  shape[a.ndim - 1] = b.shape[b.ndim - 1];
  /* A long row that is no whole number of 128-byte lines (GPT-2's 50257 logits per token): the
     block's row pitch is rounded up to whole lines and the result is the [.., n] view of it, as
     the Python mirror's matmul does. The reference allocates C-contiguous (nx_backend.ml:485-500). */
  const int64_t n = shape[a.ndim - 1], line = 128 / (int64_t)elem_size(a.dtype);
  if (n >= 4096 && n % line) {
    shape[a.ndim - 1] = (n + line - 1) / line * line;
    val o = fresh(a.dtype, a.ndim, shape);
    o.t.shape[a.ndim - 1] = n;
    must(L.matmul(ctx, &o.t, &a, &b), "matmul");
    return o;
  }
  val o = fresh(a.dtype, a.ndim, shape);
  must(L.matmul(ctx, &o.t, &a, &b), "matmul");
  return o;
}
static val contiguous(nxh_tensor x) {
  val o = fresh(x.dtype, x.ndim, x.shape);
  must(L.copy(ctx, &o.t, &x), "contiguous");
  return o;
}

/* ── frontend.ml lowerings ──────────────────────────────────────────────── */
static val op_scalar(int op, nxh_tensor x, double s) { /* add_s / mul_s: x op (scalar broadcast) */
  val c = scalar(x.dtype, s);
  val o = bin(op, x, expand(c.t, x.ndim, x.shape));
  drop(c);
  return o;
}
/* frontend.ml:4242-4252 with scale = 1 */
static val softmax(nxh_tensor x) {
  val mx = fold_last(NXH_RMAX, x);
  val d = bin(NXH_SUB, x, expand(keep_last(mx.t), x.ndim, x.shape));
  drop(mx);
  val e = un(NXH_EXP, d.t);
  drop(d);
  val s = fold_last(NXH_SUM, e.t);
  val out = bin(NXH_FDIV, e.t, expand(keep_last(s.t), x.ndim, x.shape));
  drop(e);
  drop(s);
  return out;
}
/* frontend.ml:698-707 over the last axis, keepdims */
static val mean_last(nxh_tensor x) {
  val s = fold_last(NXH_SUM, x);
  val count = scalar(x.dtype, (double)x.shape[x.ndim - 1]);
  nxh_tensor sk = keep_last(s.t);
  val m = bin(NXH_FDIV, sk, expand(count.t, sk.ndim, sk.shape));
  drop(s);
  drop(count);
  return m;
}
/* frontend.ml:1410-1435 take along axis 0 of a [rows, width] table with `n` flat indices */
static val take_rows(nxh_tensor table, nxh_tensor flat_indices) {
  const int64_t n = flat_indices.shape[0], shape[2] = {n, table.shape[1]};
  nxh_tensor idx = expand(keep_last(flat_indices), 2, shape);
  val o = fresh(table.dtype, 2, shape);
  must(L.gather(ctx, &o.t, &table, &idx, 0), "gather");
  return o;
}

#endif /* NX_HOST_H */
