/* kaun_gpt2_host.c: Kaun's GPT-2 forward (packages/kaun/examples/04-gpt2/gpt2.ml:165-200
   over packages/kaun/lib/{embedding,linear,layer_norm,attention,fn}.ml) issued from a
   compiled host through the libnxhip C ABI, one library call per backend primitive, the
   way the OCaml binding issues it. No Python, no torch.

   It answers one question: what does a forward cost through the boundary, host included?
   Four ways of running the same call sequence are timed (wall clock from the first call to
   the return of the synchronisation, per forward):
     eager      every primitive runs as it is called;
     deferred   nxh_set_deferred: the library records and fuses, handles freed at scope exit;
     late       the same with every free held back until the forward has been read
                (handles that wait for a garbage collector);
     replay     the deferred forward recorded into a graph once and replayed
                (no host work per forward: the GPU's own time).

   Usage:
     kaun_gpt2_host LIB [--vocab V --positions P --embd D --layers L --heads H --inner I]
                        [--batch B --seq S] [--dtype bf16|f32] [--iters N]
                        [--time eager,deferred,late,replay]
                        [--params FILE --ids FILE --logits FILE [--logits-bytes N] --mode eager|deferred|late]
   Without --params the weights are seeded noise of standard deviation 0.02 generated here;
   with it, FILE holds every leaf's storage bytes in the order of `leaves` below, --ids the
   int32 token ids, and the logits of one forward in --mode (their first --logits-bytes bytes,
   when given) are written to --logits (this is
   how the test compares this host with the Python mirror, bit for bit).
   Prints one JSON line. */

#include <time.h>

#include "nx_host.h"

typedef struct { val w, b; } linear_p;
typedef struct { val gamma, beta; } norm_p;
typedef struct { norm_p ln1; linear_p q, k, v, out; norm_p ln2; linear_p fc, proj; } block_p;
typedef struct { val wte, wpe; block_p *blocks; norm_p ln_f; } params;
typedef struct { int64_t vocab, positions, embd, layers, heads, inner, batch, seq; int dtype; double eps; } config;

static config cfg = {50257, 1024, 768, 12, 12, 3072, 8, 1024, NXH_BF16, 1e-5};

static double now_ms(void) {
  struct timespec ts;
  clock_gettime(CLOCK_MONOTONIC, &ts);
  return ts.tv_sec * 1e3 + ts.tv_nsec * 1e-6;
}

/* ── the layers ─────────────────────────────────────────────────────────── */

/* linear.ml:50-52 */
static val linear(const linear_p *p, nxh_tensor x) {
  val y = matmul(x, p->w.t);
  val o = bin(NXH_ADD, y.t, expand(p->b.t, y.t.ndim, y.t.shape));
  drop(y);
  return o;
}

/* layer_norm.ml:43-68: the statistics in a float32 island for 16-bit floats */
static val normalize(nxh_tensor x, double eps) {
  val mu = mean_last(x);
  val xc = bin(NXH_SUB, x, expand(mu.t, x.ndim, x.shape));
  drop(mu);
  val sq = bin(NXH_MUL, xc.t, xc.t);
  val var = mean_last(sq.t);
  drop(sq);
  val ve = op_scalar(NXH_ADD, var.t, eps);
  drop(var);
  val rt = un(NXH_SQRT, ve.t);
  drop(ve);
  val o = bin(NXH_FDIV, xc.t, expand(rt.t, x.ndim, x.shape));
  drop(xc);
  drop(rt);
  return o;
}
static val layer_norm(const norm_p *p, nxh_tensor x) {
  val n;
  if (x.dtype == NXH_BF16 || x.dtype == NXH_F16) {
    val xf = cast_to(NXH_F32, x);
    val nf = normalize(xf.t, cfg.eps);
    drop(xf);
    n = cast_to(x.dtype, nf.t);
    drop(nf);
  } else {
    n = normalize(x, cfg.eps);
  }
  val g = bin(NXH_MUL, n.t, expand(p->gamma.t, x.ndim, x.shape));
  drop(n);
  val o = bin(NXH_ADD, g.t, expand(p->beta.t, x.ndim, x.shape));
  drop(g);
  return o;
}

/* fn.ml:31-38 */
static val gelu_approx(nxh_tensor x) {
  val x2 = bin(NXH_MUL, x, x);
  val x3 = bin(NXH_MUL, x, x2.t);
  drop(x2);
  val a = op_scalar(NXH_MUL, x3.t, 0.044715);
  drop(x3);
  val b = bin(NXH_ADD, x, a.t);
  drop(a);
  val inner = op_scalar(NXH_MUL, b.t, 0.7978845608028654);
  drop(b);
  val th = un(NXH_TANH, inner.t);
  drop(inner);
  val t1 = op_scalar(NXH_ADD, th.t, 1.0);
  drop(th);
  val xt = bin(NXH_MUL, x, t1.t);
  drop(t1);
  val o = op_scalar(NXH_MUL, xt.t, 0.5);
  drop(xt);
  return o;
}

/* attention.ml:67-110 */
static val weights(nxh_tensor q, nxh_tensor k, const nxh_tensor *mask) {
  const int r = k.ndim;
  val scores = matmul(q, swapaxes(k, r - 2, r - 1));
  val scaled = op_scalar(NXH_MUL, scores.t, 1.0 / sqrt((double)q.shape[r - 1]));
  drop(scores);
  if (mask) {
    val fill = scalar(scaled.t.dtype, -INFINITY);
    val w = fresh(scaled.t.dtype, r, scaled.t.shape);
    nxh_tensor xm = expand(*mask, r, scaled.t.shape), xf = expand(fill.t, r, scaled.t.shape);
    must(L.where(ctx, &w.t, &xm, &scaled.t, &xf), "where");
    drop(scaled);
    drop(fill);
    scaled = w;
  }
  val p = softmax(scaled.t);
  drop(scaled);
  return p;
}
static val scaled_dot_product_attention(nxh_tensor q, nxh_tensor k, nxh_tensor v, const nxh_tensor *mask) {
  val probs;
  if (q.dtype == NXH_BF16 || q.dtype == NXH_F16) {
    val qf = cast_to(NXH_F32, q), kf = cast_to(NXH_F32, k);
    val pf = weights(qf.t, kf.t, mask);
    drop(qf);
    drop(kf);
    probs = cast_to(q.dtype, pf.t);
    drop(pf);
  } else {
    probs = weights(q, k, mask);
  }
  val o = matmul(probs.t, v);
  drop(probs);
  return o;
}

/* attention.ml:218-265, causal; x: [batch, seq, embd] */
static val attention(const block_p *b, nxh_tensor x) {
  const int64_t B = x.shape[0], S = x.shape[1], D = x.shape[2], H = cfg.heads, hd = D / H;
  const int64_t split_shape[4] = {B, S, H, hd};
  val q = linear(&b->q, x), k = linear(&b->k, x), v = linear(&b->v, x);
  nxh_tensor qh = swapaxes(reshape(q.t, 4, split_shape), 1, 2), kh = swapaxes(reshape(k.t, 4, split_shape), 1, 2),
             vh = swapaxes(reshape(v.t, 4, split_shape), 1, 2);
  /* the mask: less_equal of two views of one arange (values made on the host, frontend.ml:1246-1290) */
  int32_t *range = (int32_t *)malloc(sizeof(int32_t) * (size_t)S);
  for (int64_t i = 0; i < S; i++) range[i] = (int32_t)i;
  const int64_t s1[1] = {S}, row_shape[2] = {1, S}, sq[2] = {S, S};
  val idx = from_host(range, NXH_I32, 1, s1);
  free(range);
  nxh_tensor row = expand(reshape(idx.t, 2, row_shape), 2, sq), col = expand(keep_last(idx.t), 2, sq);
  val mask = fresh(NXH_BOOL, 2, sq);
  must(L.compare(ctx, NXH_CMPLE, &mask.t, &row, &col), "less_equal");
  drop(idx);
  val a = scaled_dot_product_attention(qh, kh, vh, &mask.t);
  drop(mask);
  drop(q);
  drop(k);
  drop(v);
  val merged = contiguous(swapaxes(a.t, 1, 2));
  drop(a);
  val o = linear(&b->out, reshape(merged.t, 3, x.shape));
  drop(merged);
  return o;
}

/* gpt2.ml:165-176 */
static val block(const block_p *b, val x) {
  val n1 = layer_norm(&b->ln1, x.t);
  val a = attention(b, n1.t);
  drop(n1);
  val x1 = bin(NXH_ADD, x.t, a.t);
  drop(a);
  drop(x);
  val n2 = layer_norm(&b->ln2, x1.t);
  val f = linear(&b->fc, n2.t);
  drop(n2);
  val g = gelu_approx(f.t);
  drop(f);
  val p = linear(&b->proj, g.t);
  drop(g);
  val x2 = bin(NXH_ADD, x1.t, p.t);
  drop(p);
  drop(x1);
  return x2;
}

/* embedding.ml:31-36 */
static val embedding(nxh_tensor table, nxh_tensor indices) {
  const int64_t n[1] = {numel(&indices)};
  return take_rows(table, reshape(indices, 1, n));
}

/* gpt2.ml:178-200; ids: [batch, seq] int32 */
static val logits(const params *p, nxh_tensor ids) {
  const int64_t B = ids.shape[0], S = ids.shape[1], D = cfg.embd;
  int32_t *range = (int32_t *)malloc(sizeof(int32_t) * (size_t)S);
  for (int64_t i = 0; i < S; i++) range[i] = (int32_t)i;
  const int64_t s1[1] = {S}, tok_shape[3] = {B, S, D}, pos_shape[3] = {1, S, D};
  val pos = from_host(range, NXH_I32, 1, s1);
  free(range);
  val te = embedding(p->wte.t, ids), pe = embedding(p->wpe.t, pos.t);
  drop(pos);
  val x = bin(NXH_ADD, reshape(te.t, 3, tok_shape), expand(reshape(pe.t, 3, pos_shape), 3, tok_shape));
  drop(te);
  drop(pe);
  for (int64_t l = 0; l < cfg.layers; l++) x = block(&p->blocks[l], x);
  val h = layer_norm(&p->ln_f, x.t);
  drop(x);
  val out = matmul(h.t, swapaxes(p->wte.t, 0, 1)); /* tied head: h @ wte^T, a strided operand */
  drop(h);
  return out;
}

/* ── parameters ─────────────────────────────────────────────────────────── */
static uint32_t mix(uint32_t i) {
  i = (i ^ 61u) ^ (i >> 16), i *= 9u, i ^= i >> 4, i *= 0x27d4eb2du, i ^= i >> 15;
  return i;
}
static FILE *param_file;
static uint32_t leaf_seed = 1;
/* one leaf: read from the file, or noise of standard deviation 0.02 (sum of two uniforms), or a constant */
static val leaf(int ndim, const int64_t *shape, int constant, double value) {
  int64_t n = 1;
  for (int d = 0; d < ndim; d++) n *= shape[d];
  const size_t es = elem_size(cfg.dtype);
  unsigned char *host = (unsigned char *)malloc((size_t)n * es);
  if (param_file) {
    if (fread(host, es, (size_t)n, param_file) != (size_t)n) {
      fprintf(stderr, "params: file too short\n");
      exit(2);
    }
  } else {
    const uint32_t seed = leaf_seed++ * 0x9e3779b9u;
    for (int64_t i = 0; i < n; i++) {
      double v = value;
      if (!constant) {
        const uint32_t a = mix(seed + (uint32_t)i), b = mix(a ^ 0x85ebca6bu);
        v = ((a >> 8) + (double)(b >> 8) - 16777216.0) / 16777216.0 * 0.02 * 2.449489742783178; /* triangular, sd 0.02 */
      }
      encode_scalar(cfg.dtype, v, host + (size_t)i * es);
    }
  }
  val t = from_host(host, cfg.dtype, ndim, shape);
  free(host);
  return t;
}
static linear_p linear_leaf(int64_t in, int64_t out) {
  const int64_t ws[2] = {in, out}, bs[1] = {out};
  linear_p p;
  p.w = leaf(2, ws, 0, 0), p.b = leaf(1, bs, 0, 0);
  return p;
}
static norm_p norm_leaf(void) {
  const int64_t s[1] = {cfg.embd};
  norm_p p;
  p.gamma = leaf(1, s, 1, 1.0), p.beta = leaf(1, s, 1, 0.0);
  return p;
}
static params leaves(void) {
  params p;
  const int64_t d = cfg.embd, te[2] = {cfg.vocab, d}, pe[2] = {cfg.positions, d};
  p.wte = leaf(2, te, 0, 0), p.wpe = leaf(2, pe, 0, 0);
  p.blocks = (block_p *)calloc((size_t)cfg.layers, sizeof(block_p));
  for (int64_t l = 0; l < cfg.layers; l++) {
    block_p *b = &p.blocks[l];
    b->ln1 = norm_leaf();
    b->q = linear_leaf(d, d), b->k = linear_leaf(d, d), b->v = linear_leaf(d, d), b->out = linear_leaf(d, d);
    b->ln2 = norm_leaf();
    b->fc = linear_leaf(d, cfg.inner), b->proj = linear_leaf(cfg.inner, d);
  }
  p.ln_f = norm_leaf();
  return p;
}

/* ── timing ─────────────────────────────────────────────────────────────── */
typedef struct { double wall_ms, gpu_ms; } timing;

/* `iters` forwards, each read back to nothing but synchronised: wall per forward */
static timing time_forwards(const params *p, nxh_tensor ids, int deferred, int late, int iters) {
  must(L.set_deferred(ctx, deferred), "set_deferred");
  nxhost_late_frees = late;
  timing t = {0, 0};
  for (int i = -2; i < iters; i++) { /* two warm-ups: allocator and kernel caches */
    must(L.synchronize(ctx), "synchronize");
    const double t0 = now_ms();
    must(L.timer_start(ctx), "timer_start");
    val out = logits(p, ids);
    float gpu = 0;
    must(L.timer_stop(ctx, &gpu), "timer_stop"); /* executes the record, waits for the stream */
    const double t1 = now_ms();
    drop(out);
    nxhost_collect();
    if (i >= 0) t.wall_ms += (t1 - t0) / iters, t.gpu_ms += gpu / iters;
  }
  nxhost_late_frees = 0;
  must(L.set_deferred(ctx, 0), "set_deferred");
  return t;
}

static timing time_replays(const params *p, nxh_tensor ids, int iters) {
  must(L.set_deferred(ctx, 1), "set_deferred");
  nxh_graph *graph = NULL;
  uint64_t s0[NXH_DEFER_STAT_COUNT], s1[NXH_DEFER_STAT_COUNT];
  /* once outside a capture first: what the library makes on first use (tables, workspaces)
     cannot be made while a capture is open */
  val warm = logits(p, ids);
  must(L.synchronize(ctx), "synchronize");
  drop(warm);
  must(L.deferred_stats(ctx, s0, NXH_DEFER_STAT_COUNT), "deferred_stats");
  must(L.capture_begin(ctx), "capture_begin");
  val out = logits(p, ids);
  must(L.capture_end(ctx, &graph), "capture_end");
  must(L.deferred_stats(ctx, s1, NXH_DEFER_STAT_COUNT), "deferred_stats");
  if (getenv("NXHOST_VERBOSE")) {
    fprintf(stderr, "captured:");
    for (int i = 0; i < NXH_DEFER_STAT_COUNT; i++) fprintf(stderr, " %llu", (unsigned long long)(s1[i] - s0[i]));
    fprintf(stderr, "\n");
  }
  timing t = {0, 0};
  for (int i = -2; i < iters; i++) {
    must(L.synchronize(ctx), "synchronize");
    const double t0 = now_ms();
    must(L.timer_start(ctx), "timer_start");
    must(L.graph_launch(ctx, graph), "graph_launch");
    float gpu = 0;
    must(L.timer_stop(ctx, &gpu), "timer_stop");
    const double t1 = now_ms();
    if (i >= 0) t.wall_ms += (t1 - t0) / iters, t.gpu_ms += gpu / iters;
  }
  must(L.graph_destroy(ctx, graph), "graph_destroy");
  drop(out);
  must(L.set_deferred(ctx, 0), "set_deferred");
  return t;
}

int main(int argc, char **argv) {
  if (argc < 2) {
    fprintf(stderr, "usage: %s libnxhip.so [options]\n", argv[0]);
    return 2;
  }
  const char *params_path = NULL, *ids_path = NULL, *logits_path = NULL, *mode = "deferred", *which = "eager,deferred,late,replay";
  size_t logits_bytes = 0; /* 0: all of them; else only this many leading bytes go to the file */
  int iters = 5;
  for (int i = 2; i + 1 < argc; i += 2) {
    const char *k = argv[i], *v = argv[i + 1];
    if (!strcmp(k, "--vocab")) cfg.vocab = atoll(v);
    else if (!strcmp(k, "--positions")) cfg.positions = atoll(v);
    else if (!strcmp(k, "--embd")) cfg.embd = atoll(v);
    else if (!strcmp(k, "--layers")) cfg.layers = atoll(v);
    else if (!strcmp(k, "--heads")) cfg.heads = atoll(v);
    else if (!strcmp(k, "--inner")) cfg.inner = atoll(v);
    else if (!strcmp(k, "--batch")) cfg.batch = atoll(v);
    else if (!strcmp(k, "--seq")) cfg.seq = atoll(v);
    else if (!strcmp(k, "--iters")) iters = atoi(v);
    else if (!strcmp(k, "--dtype")) cfg.dtype = !strcmp(v, "f32") ? NXH_F32 : NXH_BF16;
    else if (!strcmp(k, "--params")) params_path = v;
    else if (!strcmp(k, "--ids")) ids_path = v;
    else if (!strcmp(k, "--logits")) logits_path = v;
    else if (!strcmp(k, "--logits-bytes")) logits_bytes = (size_t)atoll(v);
    else if (!strcmp(k, "--mode")) mode = v;
    else if (!strcmp(k, "--time")) which = v;
    else {
      fprintf(stderr, "unknown option %s\n", k);
      return 2;
    }
  }
  if (cfg.seq > cfg.positions || cfg.embd % cfg.heads) {
    fprintf(stderr, "Gpt2.logits: seq exceeds n_positions, or heads do not divide the width\n");
    return 2;
  }
  nxhost_open(argv[1]);
  if (params_path && !(param_file = fopen(params_path, "rb"))) {
    perror(params_path);
    return 2;
  }
  params p = leaves();
  const int64_t n_ids = cfg.batch * cfg.seq, ids_shape[2] = {cfg.batch, cfg.seq};
  int32_t *host_ids = (int32_t *)malloc(sizeof(int32_t) * (size_t)n_ids);
  if (ids_path) {
    FILE *f = fopen(ids_path, "rb");
    if (!f || fread(host_ids, 4, (size_t)n_ids, f) != (size_t)n_ids) {
      fprintf(stderr, "ids: cannot read %s\n", ids_path);
      return 2;
    }
    fclose(f);
  } else {
    for (int64_t i = 0; i < n_ids; i++) host_ids[i] = (int32_t)(mix(0xabcdu + (uint32_t)i) % (uint32_t)cfg.vocab);
  }
  val ids = from_host(host_ids, NXH_I32, 2, ids_shape);
  free(host_ids);

  if (logits_path) { /* one forward in --mode, its logits to the file */
    const int deferred = strcmp(mode, "eager") != 0;
    must(L.set_deferred(ctx, deferred), "set_deferred");
    nxhost_late_frees = !strcmp(mode, "late");
    uint64_t s0[NXH_DEFER_STAT_COUNT], s1[NXH_DEFER_STAT_COUNT];
    must(L.deferred_stats(ctx, s0, NXH_DEFER_STAT_COUNT), "deferred_stats");
    val out = logits(&p, ids.t);
    const size_t bytes = (size_t)numel(&out.t) * elem_size(cfg.dtype);
    void *host = malloc(bytes);
    /* the head's result is a view of a block with padded rows (matmul in nx_host.h): gathered first */
    const int nd = out.t.ndim, pitched = out.t.strides[nd - 2] != out.t.shape[nd - 1];
    val dense = pitched ? contiguous(out.t) : out;
    must(L.memcpy_d2h(ctx, host, dense.block, bytes), "to_host");
    if (pitched) drop(dense);
    must(L.deferred_stats(ctx, s1, NXH_DEFER_STAT_COUNT), "deferred_stats");
    drop(out);
    nxhost_collect();
    nxhost_late_frees = 0;
    must(L.set_deferred(ctx, 0), "set_deferred");
    uint64_t s2[NXH_DEFER_STAT_COUNT];
    must(L.deferred_stats(ctx, s2, NXH_DEFER_STAT_COUNT), "deferred_stats");
    FILE *f = fopen(logits_path, "wb");
    const size_t written = logits_bytes && logits_bytes < bytes ? logits_bytes : bytes;
    if (!f || fwrite(host, 1, written, f) != written) {
      fprintf(stderr, "logits: cannot write %s\n", logits_path);
      return 2;
    }
    fclose(f);
    free(host);
    printf("{\"mode\": \"%s\", \"recorded\": %llu, \"issued\": %llu, \"fallbacks\": %llu, \"softmax_rows\": %llu, "
           "\"layer_norm_rows\": %llu, \"gelu_tanh\": %llu, \"attention\": %llu, \"linear\": %llu, \"linear_gelu\": %llu, \"postponed\": %llu, "
           "\"materialised\": %llu}\n",
           mode, (unsigned long long)(s1[NXH_DEFER_RECORDED] - s0[NXH_DEFER_RECORDED]),
           (unsigned long long)(s1[NXH_DEFER_ISSUED] - s0[NXH_DEFER_ISSUED]),
           (unsigned long long)(s1[NXH_DEFER_FALLBACKS] - s0[NXH_DEFER_FALLBACKS]),
           (unsigned long long)(s1[NXH_DEFER_SOFTMAX] - s0[NXH_DEFER_SOFTMAX]),
           (unsigned long long)(s1[NXH_DEFER_LAYER_NORM] - s0[NXH_DEFER_LAYER_NORM]),
           (unsigned long long)(s1[NXH_DEFER_GELU] - s0[NXH_DEFER_GELU]),
           (unsigned long long)(s1[NXH_DEFER_ATTENTION] - s0[NXH_DEFER_ATTENTION]),
           (unsigned long long)(s1[NXH_DEFER_LINEAR] - s0[NXH_DEFER_LINEAR]),
           (unsigned long long)(s1[NXH_DEFER_LINEAR_GELU] - s0[NXH_DEFER_LINEAR_GELU]),
           (unsigned long long)(s1[NXH_DEFER_POSTPONED] - s0[NXH_DEFER_POSTPONED]),
           (unsigned long long)(s2[NXH_DEFER_MATERIALISED] - s0[NXH_DEFER_MATERIALISED]));
    L.context_destroy(ctx);
    return 0;
  }

  const timing none = {0, 0};
  const timing eager = strstr(which, "eager") ? time_forwards(&p, ids.t, 0, 0, iters) : none;
  const timing deferred = strstr(which, "deferred") ? time_forwards(&p, ids.t, 1, 0, iters) : none;
  const timing late = strstr(which, "late") ? time_forwards(&p, ids.t, 1, 1, iters) : none;
  const timing replay = strstr(which, "replay") ? time_replays(&p, ids.t, iters) : none;
  const double tokens = (double)(cfg.batch * cfg.seq);
  printf("{\"host\": \"c\", \"dtype\": \"%s\", \"batch\": %lld, \"seq\": %lld, \"layers\": %lld, \"embd\": %lld, \"iters\": %d, "
         "\"eager_wall_ms\": %.3f, \"eager_gpu_ms\": %.3f, \"deferred_wall_ms\": %.3f, \"deferred_gpu_ms\": %.3f, "
         "\"late_free_wall_ms\": %.3f, \"late_free_gpu_ms\": %.3f, \"replay_wall_ms\": %.3f, \"replay_gpu_ms\": %.3f, "
         "\"deferred_wall_over_replay_gpu\": %.3f, \"deferred_tokens_per_s\": %.0f}\n",
         cfg.dtype == NXH_F32 ? "f32" : "bf16", (long long)cfg.batch, (long long)cfg.seq, (long long)cfg.layers,
         (long long)cfg.embd, iters, eager.wall_ms, eager.gpu_ms, deferred.wall_ms, deferred.gpu_ms, late.wall_ms, late.gpu_ms,
         replay.wall_ms, replay.gpu_ms, replay.gpu_ms > 0 ? deferred.wall_ms / replay.gpu_ms : 0.0,
         deferred.wall_ms > 0 ? tokens / (deferred.wall_ms * 1e-3) : 0.0);
  L.context_destroy(ctx);
  return 0;
}
