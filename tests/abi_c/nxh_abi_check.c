/* nxh_abi_check.c: the C ABI of libnxhip used from plain C, the way the OCaml
   stubs of the binding use it: dlopen, "output first" descriptors, status codes
   and nxh_last_error. No Python, no torch. Every result is compared with the
   same arithmetic done on the host in C (integer cases exactly, float cases that
   are exact by construction). Prints one line per check; exit status 0 = all ok.

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
  X(capture_begin) X(capture_end) X(graph_launch) X(graph_destroy)
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

  void *blocks[] = {da, db, dout, drs, dam, dfa, dfb, dfc, didx, dg, dz, dzo, dm, dl};
  for (size_t i = 0; i < sizeof blocks / sizeof *blocks; i++) must(L.free(ctx, blocks[i]), "free");
  L.context_destroy(ctx);
  printf("%s\n", failures ? "FAILED" : "all ok");
  return failures ? 1 : 0;
}
