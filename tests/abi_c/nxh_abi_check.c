/* nxh_abi_check.c: the C ABI of libnxhip used from plain C, the way the OCaml
   stubs of the binding use it: dlopen, "output first" descriptors, status codes
   and nxh_last_error. No Python, no torch. Every result is compared with the
   same arithmetic done on the host in C (integer cases exactly, float cases that
   are exact by construction). With nxh_set_deferred on, the primitive sequences
   the frontend lowers softmax, layer norm and attention to are issued one call at
   a time, as a binding that knows no fused entry point would issue them, and the
   fused kernels are seen to have run (nxh_last_path, nxh_deferred_stats) with the
   results of the fused entry points, bit for bit, and of the eager sequence to
   rounding. Prints one line per check; exit status 0 = all ok.

   Usage: nxh_abi_check /path/to/libnxhip.so */

#include <dlfcn.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "nxhip.h"

#define SYMBOLS(X)                                                                       \
  X(context_create) X(context_destroy) X(last_error) X(alloc) X(free) X(memcpy_h2d)      \
  X(memcpy_d2h) X(synchronize) X(fill) X(unary) X(binary) X(compare) X(where) X(cast)   \
  X(reduce) X(argreduce) X(matmul) X(copy) X(gather) X(sort) X(fft) X(cholesky)         \
  X(capture_begin) X(capture_end) X(graph_launch) X(graph_destroy) X(softmax_rows)      \
  X(layer_norm_rows) X(attention) X(set_deferred) X(deferred_stats) X(last_path)
static struct {
#define X(n) __typeof__(nxh_##n) *n;
  SYMBOLS(X)
#undef X
} L;

static nxh_context *ctx;
static int failures;

static void expect(int ok, const char *what) {
  printf("%s %s\n", ok ? "ok  " : "FAIL", what);
  if (!ok) failures++;
}

static void must(int rc, const char *what) {
  if (rc != NXH_OK) {
    printf("FAIL %s: status %d: %s\n", what, rc, L.last_error(ctx));
    exit(2);
  }
}

/* contiguous descriptor over device memory */
static nxh_tensor desc(void *data, int dtype, int ndim, const int64_t *shape) {
  nxh_tensor t;
  memset(&t, 0, sizeof t);
  t.data = data;
  t.dtype = dtype;
  t.ndim = ndim;
  int64_t stride = 1;
  for (int d = ndim - 1; d >= 0; d--) {
    t.shape[d] = shape[d];
    t.strides[d] = stride;
    stride *= shape[d];
  }
  return t;
}

static void *upload(const void *host, size_t bytes) {
  void *p = NULL;
  must(L.alloc(ctx, bytes, &p), "alloc");
  must(L.memcpy_h2d(ctx, p, host, bytes), "from_host");
  return p;
}

/* ── the frontend's sequences, one primitive per call ─────────────────────── */

/* A value as the frontend holds it: a view and the block that backs it. */
typedef struct {
  nxh_tensor t;
  void *block;
} val;

static size_t elem_size(int dtype) { return dtype == NXH_F32 || dtype == NXH_I32 ? 4 : dtype == NXH_BOOL ? 1 : 2; }

static val fresh(int dtype, int ndim, const int64_t *shape) {
  size_t n = 1;
  for (int d = 0; d < ndim; d++) n *= (size_t)shape[d];
  val v;
  must(L.alloc(ctx, n * elem_size(dtype), &v.block), "alloc");
  v.t = desc(v.block, dtype, ndim, shape);
  return v;
}
static void drop(val v) { must(L.free(ctx, v.block), "free"); }

/* view.ml expand: leading extents are added, an extent of 1 is repeated with stride 0 */
static nxh_tensor expand(nxh_tensor t, int ndim, const int64_t *shape) {
  nxh_tensor r = t;
  int pad = ndim - t.ndim;
  r.ndim = ndim;
  for (int d = 0; d < ndim; d++) {
    int64_t have = d < pad ? 1 : t.shape[d - pad];
    r.strides[d] = (d < pad || (have == 1 && shape[d] != 1)) ? 0 : t.strides[d - pad];
    r.shape[d] = shape[d];
  }
  return r;
}
/* reshape [.., R] -> [.., R, 1] of a contiguous view (the keepdims form of a reduction) */
static nxh_tensor keep_last(nxh_tensor t) {
  t.shape[t.ndim] = 1;
  t.strides[t.ndim] = 1;
  t.ndim++;
  return t;
}
static val scalar(int dtype, const void *element) {
  val v = fresh(dtype, 0, NULL);
  must(L.fill(ctx, &v.t, element), "full");
  return v;
}
static val un(int op, nxh_tensor x) {
  val o = fresh(x.dtype, x.ndim, x.shape);
  must(L.unary(ctx, op, &o.t, &x), "unary");
  return o;
}
static val bin(int op, nxh_tensor x, nxh_tensor y) {
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
static val product(nxh_tensor a, nxh_tensor b) {
  int64_t shape[NXH_MAX_NDIM];
  memcpy(shape, a.shape, sizeof shape);
  shape[a.ndim - 1] = b.shape[b.ndim - 1];
  val o = fresh(a.dtype, a.ndim, shape);
  must(L.matmul(ctx, &o.t, &a, &b), "matmul");
  return o;
}

/* frontend.ml:4242-4252 with scale = 1 */
static val softmax_sequence(nxh_tensor x) {
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

/* frontend.ml:698-707 mean over the last axis, keepdims */
static val mean_last(nxh_tensor x) {
  float n = (float)x.shape[x.ndim - 1];
  val s = fold_last(NXH_SUM, x);
  val count = scalar(NXH_F32, &n);
  nxh_tensor sk = keep_last(s.t);
  val m = bin(NXH_FDIV, sk, expand(count.t, sk.ndim, sk.shape));
  drop(s);
  drop(count);
  return m;
}

/* kaun/lib/layer_norm.ml:43-68 for float32 */
static val layer_norm_sequence(nxh_tensor x, nxh_tensor gamma, nxh_tensor beta, float eps) {
  val mu = mean_last(x);
  val xc = bin(NXH_SUB, x, expand(mu.t, x.ndim, x.shape));
  drop(mu);
  val sq = bin(NXH_MUL, xc.t, xc.t);
  val var = mean_last(sq.t);
  drop(sq);
  val e = scalar(NXH_F32, &eps);
  val ve = bin(NXH_ADD, var.t, expand(e.t, var.t.ndim, var.t.shape));
  drop(var);
  drop(e);
  val rt = un(NXH_SQRT, ve.t);
  drop(ve);
  val nrm = bin(NXH_FDIV, xc.t, expand(rt.t, x.ndim, x.shape));
  drop(xc);
  drop(rt);
  val g = bin(NXH_MUL, nrm.t, expand(gamma, x.ndim, x.shape));
  drop(nrm);
  val out = bin(NXH_ADD, g.t, expand(beta, x.ndim, x.shape));
  drop(g);
  return out;
}

/* kaun/lib/attention.ml:67-110 for bfloat16 q, k, v of [B, H, S, D] under the causal mask
   of attention.ml:218-265 (less_equal of two views of one arange) */
static val attention_sequence(nxh_tensor q, nxh_tensor k, nxh_tensor v) {
  int64_t S = q.shape[2], D = q.shape[3];
  val qf = cast_to(NXH_F32, q), kf = cast_to(NXH_F32, k);
  nxh_tensor kt = kf.t; /* swapaxes of the last two */
  kt.shape[2] = D, kt.shape[3] = S, kt.strides[2] = 1, kt.strides[3] = D;
  val sc = product(qf.t, kt);
  drop(qf);
  drop(kf);
  float scale = 1.0f / sqrtf((float)D), ninf = -INFINITY;
  val c = scalar(NXH_F32, &scale);
  val scaled = bin(NXH_MUL, sc.t, expand(c.t, 4, sc.t.shape));
  drop(sc);
  drop(c);
  int32_t *range = malloc(sizeof(int32_t) * (size_t)S);
  for (int64_t i = 0; i < S; i++) range[i] = (int32_t)i;
  val idx;
  idx.block = upload(range, sizeof(int32_t) * (size_t)S);
  free(range);
  int64_t s1[1] = {S}, sq[2] = {S, S};
  idx.t = desc(idx.block, NXH_I32, 1, s1);
  nxh_tensor row = idx.t, col = keep_last(idx.t); /* [1, S] and [S, 1] */
  row.ndim = 2, row.shape[0] = 1, row.shape[1] = S, row.strides[0] = S, row.strides[1] = 1;
  nxh_tensor xrow = expand(row, 2, sq), xcol = expand(col, 2, sq);
  val mask = fresh(NXH_BOOL, 2, sq);
  must(L.compare(ctx, NXH_CMPLE, &mask.t, &xrow, &xcol), "less_equal");
  drop(idx);
  val fill = scalar(NXH_F32, &ninf);
  val w = fresh(NXH_F32, 4, scaled.t.shape);
  nxh_tensor xmask = expand(mask.t, 4, scaled.t.shape), xfill = expand(fill.t, 4, scaled.t.shape);
  must(L.where(ctx, &w.t, &xmask, &scaled.t, &xfill), "where");
  drop(scaled);
  drop(fill);
  drop(mask);
  val p = softmax_sequence(w.t);
  drop(w);
  val pb = cast_to(NXH_BF16, p.t);
  drop(p);
  val out = product(pb.t, v);
  drop(pb);
  return out;
}

static uint16_t bf16_of(float f) { /* round to nearest even; no NaN in these inputs */
  uint32_t u;
  memcpy(&u, &f, 4);
  return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}
static float bf16_value(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static float noise(uint32_t i) { /* in [-2, 2) */
  i = (i ^ 61u) ^ (i >> 16), i *= 9u, i ^= i >> 4, i *= 0x27d4eb2du, i ^= i >> 15;
  return (float)(i >> 8) / 4194304.0f - 2.0f;
}
static void counters(uint64_t *s) { must(L.deferred_stats(ctx, s, NXH_DEFER_STAT_COUNT), "deferred_stats"); }

static void deferred_sequences(void) {
  enum { R = 48, C = 200, N = R * C };
  static float x[N], gamma[C], beta[C], eager[N], fused[N], direct[N];
  for (int i = 0; i < N; i++) x[i] = 3.0f * noise(i);
  for (int j = 0; j < C; j++) gamma[j] = 1.0f + 0.1f * noise(100000 + j), beta[j] = 0.1f * noise(200000 + j);
  int64_t sh[2] = {R, C}, shc[1] = {C};
  val vx = {desc(upload(x, sizeof x), NXH_F32, 2, sh), NULL}, vg = {desc(upload(gamma, sizeof gamma), NXH_F32, 1, shc), NULL},
      vb = {desc(upload(beta, sizeof beta), NXH_F32, 1, shc), NULL};
  vx.block = vx.t.data, vg.block = vg.t.data, vb.block = vb.t.data;
  uint64_t s0[NXH_DEFER_STAT_COUNT], s1[NXH_DEFER_STAT_COUNT];

  /* softmax: eager, recorded, and the fused entry point called by name */
  val r = softmax_sequence(vx.t);
  must(L.memcpy_d2h(ctx, eager, r.block, sizeof eager), "to_host");
  drop(r);
  counters(s0);
  must(L.set_deferred(ctx, 1), "set_deferred");
  r = softmax_sequence(vx.t);
  must(L.memcpy_d2h(ctx, fused, r.block, sizeof fused), "to_host"); /* the read executes the record */
  expect(strcmp(L.last_path(ctx), "softmax_rows") == 0, "deferred: the five softmax primitives ran as softmax_rows");
  drop(r);
  counters(s1);
  expect(s1[NXH_DEFER_SOFTMAX] - s0[NXH_DEFER_SOFTMAX] == 1 && s1[NXH_DEFER_RECORDED] - s0[NXH_DEFER_RECORDED] == 5 &&
             s1[NXH_DEFER_ISSUED] == s0[NXH_DEFER_ISSUED] && s1[NXH_DEFER_FALLBACKS] == s0[NXH_DEFER_FALLBACKS],
         "deferred: softmax counters (5 recorded, 0 issued as recorded, 1 fused)");
  must(L.set_deferred(ctx, 0), "set_deferred");
  r = fresh(NXH_F32, 2, sh);
  must(L.softmax_rows(ctx, &r.t, &vx.t, NULL, NULL, NULL), "softmax_rows");
  must(L.memcpy_d2h(ctx, direct, r.block, sizeof direct), "to_host");
  drop(r);
  expect(memcmp(fused, direct, sizeof fused) == 0, "deferred: softmax equals nxh_softmax_rows bit for bit");
  int ok = 1;
  for (int i = 0; i < R; i++) {
    double m = -INFINITY, z = 0, rowsum = 0;
    for (int j = 0; j < C; j++) m = fmax(m, x[i * C + j]);
    for (int j = 0; j < C; j++) z += exp((double)x[i * C + j] - m);
    for (int j = 0; j < C; j++) {
      double want = exp((double)x[i * C + j] - m) / z;
      ok &= fabs(fused[i * C + j] - want) <= 2e-6 * want + 1e-12 && fabs(eager[i * C + j] - want) <= 2e-6 * want + 1e-12;
      rowsum += fused[i * C + j];
    }
    ok &= fabs(rowsum - 1.0) < 1e-5;
  }
  expect(ok, "deferred: softmax, fused and eager, against the host in double");

  /* layer norm */
  r = layer_norm_sequence(vx.t, vg.t, vb.t, 1e-5f);
  must(L.memcpy_d2h(ctx, eager, r.block, sizeof eager), "to_host");
  drop(r);
  counters(s0);
  must(L.set_deferred(ctx, 1), "set_deferred");
  r = layer_norm_sequence(vx.t, vg.t, vb.t, 1e-5f);
  must(L.synchronize(ctx), "synchronize"); /* executes the record as well */
  expect(strcmp(L.last_path(ctx), "layer_norm_rows") == 0, "deferred: the layer-norm primitives ran as layer_norm_rows");
  must(L.memcpy_d2h(ctx, fused, r.block, sizeof fused), "to_host");
  drop(r);
  counters(s1);
  expect(s1[NXH_DEFER_LAYER_NORM] - s0[NXH_DEFER_LAYER_NORM] == 1 && s1[NXH_DEFER_RECORDED] - s0[NXH_DEFER_RECORDED] == 14 &&
             s1[NXH_DEFER_ISSUED] == s0[NXH_DEFER_ISSUED] && s1[NXH_DEFER_FALLBACKS] == s0[NXH_DEFER_FALLBACKS],
         "deferred: layer-norm counters (14 recorded, 0 issued as recorded, 1 fused)");
  must(L.set_deferred(ctx, 0), "set_deferred");
  r = fresh(NXH_F32, 2, sh);
  must(L.layer_norm_rows(ctx, &r.t, &vx.t, &vg.t, &vb.t, (double)1e-5f), "layer_norm_rows");
  must(L.memcpy_d2h(ctx, direct, r.block, sizeof direct), "to_host");
  drop(r);
  expect(memcmp(fused, direct, sizeof fused) == 0, "deferred: layer norm equals nxh_layer_norm_rows bit for bit");
  ok = 1;
  for (int i = 0; i < R; i++) {
    double mu = 0, var = 0;
    for (int j = 0; j < C; j++) mu += x[i * C + j];
    mu /= C;
    for (int j = 0; j < C; j++) var += (x[i * C + j] - mu) * (x[i * C + j] - mu);
    var /= C;
    for (int j = 0; j < C; j++) {
      double want = (x[i * C + j] - mu) / sqrt(var + (double)1e-5f) * gamma[j] + beta[j];
      ok &= fabs(fused[i * C + j] - want) <= 4e-6 * (1 + fabs(want)) && fabs(eager[i * C + j] - want) <= 4e-6 * (1 + fabs(want));
    }
  }
  expect(ok, "deferred: layer norm, fused and eager, against the host in double");

  /* an intermediate the caller keeps: the run is fused all the same, the kept result is written
     when it is read, and holds the eager value */
  counters(s0);
  must(L.set_deferred(ctx, 1), "set_deferred");
  val mx = fold_last(NXH_RMAX, vx.t);
  val d = bin(NXH_SUB, vx.t, expand(keep_last(mx.t), 2, sh));
  val e = un(NXH_EXP, d.t);
  val s = fold_last(NXH_SUM, e.t);
  r = bin(NXH_FDIV, e.t, expand(keep_last(s.t), 2, sh));
  drop(mx), drop(d), drop(s);
  must(L.memcpy_d2h(ctx, fused, r.block, sizeof fused), "to_host");
  counters(s1);
  ok = s1[NXH_DEFER_SOFTMAX] - s0[NXH_DEFER_SOFTMAX] == 1 && s1[NXH_DEFER_ISSUED] == s0[NXH_DEFER_ISSUED] &&
       s1[NXH_DEFER_POSTPONED] - s0[NXH_DEFER_POSTPONED] == 4 && s1[NXH_DEFER_MATERIALISED] == s0[NXH_DEFER_MATERIALISED];
  expect(ok, "deferred: a held intermediate does not stop the fusion (4 entries postponed)");
  must(L.memcpy_d2h(ctx, direct, e.block, sizeof direct), "to_host");
  counters(s1);
  ok = s1[NXH_DEFER_MATERIALISED] - s0[NXH_DEFER_MATERIALISED] == 4;
  drop(r), drop(e);
  must(L.set_deferred(ctx, 0), "set_deferred");
  for (int i = 0; i < R && ok; i++) {
    float m = -INFINITY;
    for (int j = 0; j < C; j++) m = fmaxf(m, x[i * C + j]);
    for (int j = 0; j < C; j++) ok &= fabs(direct[i * C + j] - exp((double)(x[i * C + j] - m))) <= 2e-6;
  }
  expect(ok, "deferred: the held intermediate is written when it is read and holds the eager value");
  /* handles given back only after the read, as a collector's finalisers would: fused, nothing ever written */
  counters(s0);
  must(L.set_deferred(ctx, 1), "set_deferred");
  mx = fold_last(NXH_RMAX, vx.t);
  d = bin(NXH_SUB, vx.t, expand(keep_last(mx.t), 2, sh));
  e = un(NXH_EXP, d.t);
  s = fold_last(NXH_SUM, e.t);
  r = bin(NXH_FDIV, e.t, expand(keep_last(s.t), 2, sh));
  must(L.memcpy_d2h(ctx, direct, r.block, sizeof direct), "to_host");
  expect(strcmp(L.last_path(ctx), "softmax_rows") == 0, "deferred: late frees: the five primitives ran as softmax_rows");
  drop(mx), drop(d), drop(s), drop(e), drop(r);
  must(L.synchronize(ctx), "synchronize");
  counters(s1);
  must(L.set_deferred(ctx, 0), "set_deferred");
  expect(s1[NXH_DEFER_SOFTMAX] - s0[NXH_DEFER_SOFTMAX] == 1 && s1[NXH_DEFER_ISSUED] == s0[NXH_DEFER_ISSUED] &&
             s1[NXH_DEFER_MATERIALISED] == s0[NXH_DEFER_MATERIALISED] && memcmp(direct, fused, sizeof fused) == 0,
         "deferred: late frees: same bits, nothing issued as recorded");

  /* attention, bfloat16 [2, 3, 96, 64], causal */
  enum { B = 2, H = 3, S = 96, D = 64, NA = B * H * S * D };
  static uint16_t q[NA], k[NA], v[NA], ae[NA], af[NA], ad[NA];
  for (int i = 0; i < NA; i++) q[i] = bf16_of(noise(300000 + i)), k[i] = bf16_of(noise(700000 + i)), v[i] = bf16_of(noise(1100000 + i));
  int64_t sa[4] = {B, H, S, D};
  nxh_tensor tq = desc(upload(q, sizeof q), NXH_BF16, 4, sa), tk = desc(upload(k, sizeof k), NXH_BF16, 4, sa),
             tv = desc(upload(v, sizeof v), NXH_BF16, 4, sa);
  r = attention_sequence(tq, tk, tv);
  must(L.memcpy_d2h(ctx, ae, r.block, sizeof ae), "to_host");
  drop(r);
  counters(s0);
  must(L.set_deferred(ctx, 1), "set_deferred");
  r = attention_sequence(tq, tk, tv);
  must(L.memcpy_d2h(ctx, af, r.block, sizeof af), "to_host");
  expect(strcmp(L.last_path(ctx), "attention_fused") == 0, "deferred: the attention primitives ran as attention_fused");
  drop(r);
  counters(s1);
  expect(s1[NXH_DEFER_ATTENTION] - s0[NXH_DEFER_ATTENTION] == 1 && s1[NXH_DEFER_ISSUED] == s0[NXH_DEFER_ISSUED] &&
             s1[NXH_DEFER_SOFTMAX] == s0[NXH_DEFER_SOFTMAX] && s1[NXH_DEFER_FALLBACKS] == s0[NXH_DEFER_FALLBACKS],
         "deferred: attention counters (nothing issued as recorded: the causal mask is never computed)");
  must(L.set_deferred(ctx, 0), "set_deferred");
  r = fresh(NXH_BF16, 4, sa);
  float scale = 1.0f / sqrtf((float)D), ninf = -INFINITY;
  must(L.attention(ctx, &r.t, &tq, &tk, &tv, &scale, NULL, &ninf, 1), "attention");
  must(L.memcpy_d2h(ctx, ad, r.block, sizeof ad), "to_host");
  drop(r);
  expect(memcmp(af, ad, sizeof af) == 0, "deferred: attention equals nxh_attention bit for bit");
  ok = 1;
  static double p[S];
  for (int bh = 0; bh < B * H; bh++)
    for (int i = 0; i < S; i += 5) { /* every fifth query row, in double from the bf16 operands */
      const uint16_t *qr = q + ((size_t)bh * S + i) * D;
      double m = -INFINITY, z = 0;
      for (int j = 0; j <= i; j++) {
        double dot = 0;
        for (int t = 0; t < D; t++) dot += (double)bf16_value(qr[t]) * bf16_value(k[((size_t)bh * S + j) * D + t]);
        p[j] = dot * scale, m = fmax(m, p[j]);
      }
      for (int j = 0; j <= i; j++) p[j] = exp(p[j] - m), z += p[j];
      for (int t = 0; t < D; t++) {
        double want = 0;
        for (int j = 0; j <= i; j++) want += p[j] / z * bf16_value(v[((size_t)bh * S + j) * D + t]);
        size_t at = ((size_t)bh * S + i) * D + t;
        double tol = 0.02 + 0.02 * fabs(want); /* probabilities and the output are rounded to bfloat16 (2^-8 relative each) */
        ok &= fabs(bf16_value(af[at]) - want) <= tol && fabs(bf16_value(ae[at]) - want) <= tol;
      }
    }
  expect(ok, "deferred: attention, fused and eager, against the host in double");
  must(L.free(ctx, tq.data), "free"), must(L.free(ctx, tk.data), "free"), must(L.free(ctx, tv.data), "free");
  drop(vx), drop(vg), drop(vb);
}

int main(int argc, char **argv) {
  if (argc < 2) {
    fprintf(stderr, "usage: %s libnxhip.so\n", argv[0]);
    return 2;
  }
  void *h = dlopen(argv[1], RTLD_NOW | RTLD_LOCAL);
  if (!h) {
    fprintf(stderr, "dlopen: %s\n", dlerror());
    return 2;
  }
#define X(n)                                      \
  L.n = (__typeof__(L.n))dlsym(h, "nxh_" #n);     \
  if (!L.n) {                                     \
    fprintf(stderr, "missing nxh_" #n "\n");      \
    return 2;                                     \
  }
  SYMBOLS(X)
#undef X
  if (L.context_create(&ctx) != NXH_OK) {
    fprintf(stderr, "create_context: %s\n", L.last_error(NULL));
    return 2;
  }

  enum { R = 37, C = 53, N = R * C };
  static int32_t a[N], b[C], got[N], want[N];
  for (int i = 0; i < N; i++) a[i] = (int32_t)((i * 2654435761u) >> 7) - (1 << 23);
  for (int j = 0; j < C; j++) b[j] = 1000 * j - 7;
  int64_t sh2[2] = {R, C}, shT[2] = {C, R};
  void *da = upload(a, sizeof a), *db = upload(b, sizeof b), *dout = NULL;
  must(L.alloc(ctx, sizeof a, &dout), "alloc");

  /* int32 add of a transposed view and a broadcast row: out[j][i] = a[i][j] + b[j] (wraps) */
  nxh_tensor ta = desc(da, NXH_I32, 2, shT), tb = desc(db, NXH_I32, 2, shT), to = desc(dout, NXH_I32, 2, shT);
  ta.strides[0] = 1, ta.strides[1] = C;   /* permute (1, 0) of the [R, C] array */
  tb.strides[0] = 1, tb.strides[1] = 0;   /* b[j] expanded along the second dim */
  must(L.binary(ctx, NXH_ADD, &to, &ta, &tb), "add");
  must(L.memcpy_d2h(ctx, got, dout, sizeof got), "to_host");
  for (int j = 0; j < C; j++)
    for (int i = 0; i < R; i++) want[j * R + i] = (int32_t)((uint32_t)a[i * C + j] + (uint32_t)b[j]);
  expect(memcmp(got, want, sizeof got) == 0, "int32 add over a permuted and a broadcast view");

  /* sum over axis 1 of the [R, C] array, int64 accumulate, wrap on store */
  static int32_t rs[R], rw[R];
  void *drs = NULL;
  must(L.alloc(ctx, sizeof rs, &drs), "alloc");
  int64_t sh1[1] = {R};
  nxh_tensor tin = desc(da, NXH_I32, 2, sh2), trs = desc(drs, NXH_I32, 1, sh1);
  int32_t axis1 = 1;
  must(L.reduce(ctx, NXH_SUM, &trs, &tin, &axis1, 1), "reduce_sum");
  must(L.memcpy_d2h(ctx, rs, drs, sizeof rs), "to_host");
  for (int i = 0; i < R; i++) {
    int64_t s = 0;
    for (int j = 0; j < C; j++) s += a[i * C + j];
    rw[i] = (int32_t)(uint32_t)(uint64_t)s;
  }
  expect(memcmp(rs, rw, sizeof rs) == 0, "int32 sum along axis 1");

  /* argmax along axis 0: first maximum wins */
  static int32_t am[C], aw[C];
  void *dam = NULL;
  must(L.alloc(ctx, sizeof am, &dam), "alloc");
  int64_t shc[1] = {C};
  nxh_tensor tam = desc(dam, NXH_I32, 1, shc);
  must(L.argreduce(ctx, 0, &tam, &tin, 0), "argmax");
  must(L.memcpy_d2h(ctx, am, dam, sizeof am), "to_host");
  for (int j = 0; j < C; j++) {
    int best = 0;
    for (int i = 1; i < R; i++)
      if (a[i * C + j] > a[best * C + j]) best = i;
    aw[j] = best;
  }
  expect(memcmp(am, aw, sizeof am) == 0, "argmax along axis 0");

  /* f32 matmul of small integers (exact in any summation order) */
  enum { M = 48, K = 64, NN = 40 };
  static float fa[M * K], fb[K * NN], fc[M * NN], fw[M * NN];
  for (int i = 0; i < M * K; i++) fa[i] = (float)((i * 7) % 11 - 5);
  for (int i = 0; i < K * NN; i++) fb[i] = (float)((i * 5) % 13 - 6);
  void *dfa = upload(fa, sizeof fa), *dfb = upload(fb, sizeof fb), *dfc = NULL;
  must(L.alloc(ctx, sizeof fc, &dfc), "alloc");
  int64_t sa[2] = {M, K}, sb[2] = {K, NN}, sc[2] = {M, NN};
  nxh_tensor tfa = desc(dfa, NXH_F32, 2, sa), tfb = desc(dfb, NXH_F32, 2, sb), tfc = desc(dfc, NXH_F32, 2, sc);
  must(L.matmul(ctx, &tfc, &tfa, &tfb), "matmul");
  must(L.memcpy_d2h(ctx, fc, dfc, sizeof fc), "to_host");
  for (int i = 0; i < M; i++)
    for (int j = 0; j < NN; j++) {
      float s = 0;
      for (int k = 0; k < K; k++) s += fa[i * K + k] * fb[k * NN + j];
      fw[i * NN + j] = s;
    }
  expect(memcmp(fc, fw, sizeof fc) == 0, "f32 matmul on small integers");

  /* gather with an index out of bounds: Failure from this call, context usable afterwards */
  static int32_t idx[C];
  for (int j = 0; j < C; j++) idx[j] = j % R;
  idx[5] = R; /* one past the end */
  void *didx = upload(idx, sizeof idx), *dg = NULL;
  must(L.alloc(ctx, sizeof idx, &dg), "alloc");
  int64_t sg[2] = {1, C};
  nxh_tensor tidx = desc(didx, NXH_I32, 2, sg), tg = desc(dg, NXH_I32, 2, sg);
  int rc = L.gather(ctx, &tg, &tin, &tidx, 0);
  expect(rc == NXH_FAILURE && strstr(L.last_error(ctx), "gather") != NULL, "gather reports an index out of bounds");
  idx[5] = -1; /* wraps once to the last row */
  must(L.memcpy_h2d(ctx, didx, idx, sizeof idx), "from_host");
  must(L.gather(ctx, &tg, &tin, &tidx, 0), "gather");
  static int32_t gg[C];
  must(L.memcpy_d2h(ctx, gg, dg, sizeof gg), "to_host");
  int gok = 1;
  for (int j = 0; j < C; j++) gok &= gg[j] == a[(j == 5 ? R - 1 : j % R) * C + j];
  expect(gok, "gather with a negative index");

  /* a precondition violation is Invalid_argument */
  nxh_tensor bad = tfb;
  bad.shape[0] = K + 1;
  expect(L.matmul(ctx, &tfc, &tfa, &bad) == NXH_INVALID_ARGUMENT, "matmul shape mismatch is Invalid_argument");

  /* a recorded sequence: add then reduce, replayed after the input changed */
  nxh_graph *graph = NULL;
  must(L.binary(ctx, NXH_ADD, &to, &ta, &tb), "warm add");
  must(L.synchronize(ctx), "synchronize");
  must(L.capture_begin(ctx), "capture_begin");
  must(L.binary(ctx, NXH_ADD, &to, &ta, &tb), "recorded add");
  must(L.capture_end(ctx, &graph), "capture_end");
  for (int j = 0; j < C; j++) b[j] = -3 * j;
  must(L.memcpy_h2d(ctx, db, b, sizeof b), "from_host");
  must(L.graph_launch(ctx, graph), "graph_launch");
  must(L.memcpy_d2h(ctx, got, dout, sizeof got), "to_host");
  for (int j = 0; j < C; j++)
    for (int i = 0; i < R; i++) want[j * R + i] = (int32_t)((uint32_t)a[i * C + j] + (uint32_t)b[j]);
  expect(memcmp(got, want, sizeof got) == 0, "graph replay reads the rewritten input");
  must(L.graph_destroy(ctx, graph), "graph_destroy");

  /* fft of a delta is all ones; cholesky of a non-positive-definite matrix fails with the reference's text */
  static double z[16], zo[16];
  memset(z, 0, sizeof z);
  z[0] = 1.0;
  void *dz = upload(z, sizeof z), *dzo = NULL;
  must(L.alloc(ctx, sizeof zo, &dzo), "alloc");
  int64_t s8[1] = {8};
  nxh_tensor tz = desc(dz, NXH_C64, 1, s8), tzo = desc(dzo, NXH_C64, 1, s8);
  int32_t ax0 = 0;
  must(L.fft(ctx, &tzo, &tz, &ax0, 1, 0), "fft");
  must(L.memcpy_d2h(ctx, zo, dzo, sizeof zo), "to_host");
  int fok = 1;
  for (int k = 0; k < 8; k++) fok &= zo[2 * k] == 1.0 && zo[2 * k + 1] == 0.0;
  expect(fok, "fft of a unit impulse");
  static double spd[4] = {1.0, 2.0, 2.0, 1.0}; /* eigenvalues 3 and -1 */
  void *dm = upload(spd, sizeof spd), *dl = NULL;
  must(L.alloc(ctx, sizeof spd, &dl), "alloc");
  int64_t s22[2] = {2, 2};
  nxh_tensor tm = desc(dm, NXH_F64, 2, s22), tl = desc(dl, NXH_F64, 2, s22);
  rc = L.cholesky(ctx, &tl, &tm, 0);
  expect(rc == NXH_FAILURE && strstr(L.last_error(ctx), "matrix is not positive definite") != NULL,
         "cholesky of an indefinite matrix fails with the reference's message");

  deferred_sequences();

  void *blocks[] = {da, db, dout, drs, dam, dfa, dfb, dfc, didx, dg, dz, dzo, dm, dl};
  for (size_t i = 0; i < sizeof blocks / sizeof *blocks; i++) must(L.free(ctx, blocks[i]), "free");
  L.context_destroy(ctx);
  printf("%s\n", failures ? "FAILED" : "all ok");
  return failures ? 1 : 0;
}
