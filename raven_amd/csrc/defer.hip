// defer.hip — the deferred-evaluation window below the C ABI.
//
// The frontend lowers softmax to five primitives (frontend.ml:4242-4252), Kaun's
// layer norm to fourteen (layer_norm.ml:43-68), its tanh GELU to nine
// (fn.ml:31-38), the attention core to seven (attention.ml:67-110) and a linear
// layer with its residual to three (linear.ml:50-52, gpt2.ml:165-176); an eager
// backend pays a pass over memory, an allocation and a launch for each. With
// nxh_set_deferred(ctx, 1) the primitive entry points (unary, binary, compare,
// where, cast, reduce, matmul, one-element fill) only RECORD their call. The
// record is executed, in issue order, as soon as anything else is asked of the
// context (any other entry point, a host read, a synchronisation), at a recorded copy
// once it holds 48 entries, or when it reaches 2048 entries. At that moment a run of entries that spells one of the
// five sequences is replaced by the fused call (nxh_softmax_rows,
// nxh_layer_norm_rows, nxh_gelu_tanh, nxh_attention, nxh_linear), provided that
// every recorded reader of its intermediate results is inside the run. An
// intermediate whose storage was given back with nxh_free while recorded is never
// written. One whose handle is still held is POSTPONED: its entry (and the rest
// of the run, with the blocks it reads kept from reuse) stays behind, unexecuted,
// and is issued as recorded the moment anything reads that block (an operand of a
// later call, a host read) or writes a block the run reads; when nxh_free arrives
// first, it is dropped. So a host whose handles die late (a garbage collector's
// finalisers) gets the same fused kernels as one that frees at once. Everything
// else is issued as recorded: what a caller can observe is the eager result, with
// two differences: an error of a recorded primitive surfaces from the call that
// executes it, and a fused float result may differ from the op-by-op one by the
// order in which a row's sum is added.
//
// Any binding gets this by switching the mode on: the caller keeps allocating
// outputs (nxh_alloc) and freeing dead handles (nxh_free) exactly as before. A
// free that arrives while recorded or postponed entries still use the block is
// held back until they have run or been dropped, so the allocator never hands out
// memory they will touch. While a graph is being captured nothing is postponed
// (a later materialisation would fall outside the graph): there an intermediate
// that is still held blocks the fusion and is written as recorded.

#include <array>
#include <memory>
#include <unordered_map>

#include "nxh_common.hpp"

namespace {

enum { D_UNARY = NXH_D_UNARY, D_BINARY = NXH_D_BINARY, D_COMPARE = NXH_D_COMPARE, D_WHERE = NXH_D_WHERE, D_CAST = NXH_D_CAST,
       D_REDUCE = NXH_D_REDUCE, D_MATMUL = NXH_D_MATMUL, D_FULL = NXH_D_FULL, D_COPY = NXH_D_COPY, D_UPLOAD = NXH_D_UPLOAD };
constexpr size_t LIMIT = 2048;
// A recorded copy (the frontend's `contiguous`) ends whatever run led up to it; once the record holds
// this many entries it is executed there, so that the device works while the host records on.
constexpr size_t COPY_FLUSH = 48;
constexpr size_t UPLOAD_LIMIT = 65536;  // bytes of a host upload that may wait in the record
constexpr int64_t MAX_ROW = (int64_t)1 << 24;  // the longest row the fused row kernels take

struct DEntry {
  int kind = 0, op = 0, nin = 0, n_axes = 0;
  nxh_tensor out{}, in[3] = {};
  DEntry *prod[3] = {nullptr, nullptr, nullptr};  // recorded producer of each input, if any
  DEntry *upl[3] = {nullptr, nullptr, nullptr};   // or the recorded upload that fills it (an operand like any stored tensor)
  int32_t axes[NXH_MAX_NDIM] = {};
  unsigned char value[16] = {};  // D_FULL: the element
  std::vector<unsigned char> payload;  // D_UPLOAD: the host bytes
  bool alive = true;             // the output block has not been freed
  bool done = false;             // issued, or inside a fused run that was issued
  bool skipped = false;          // done without having been written (a causal mask that every reader took as a flag)
  DEntry *fused_into = nullptr;
  std::vector<DEntry *> readers;
  int64_t causal = 0;  // n: the result is the n x n mask [i][j] = (j <= i)
  size_t id = 0;
};

struct Known {  // what the window knows about the contents of a block
  int dtype = -1;
  unsigned char scalar[16] = {};  // one element, every element of the block equals it
  bool has_scalar = false;
  std::vector<int32_t> host_i32;  // a small upload, as int32
  int64_t causal = 0;
};

// The unexecuted rest of a fused run: interior entries, and the scalar fills and causal
// mask that only the run read, in issue order. `alive` counts members whose handle is held.
struct Postponed {
  std::vector<std::unique_ptr<DEntry>> members;
  int alive = 0;
};

struct Window {
  std::mutex mu;
  bool on = false;
  bool may_postpone = true;  // false while the executing flush is being captured
  std::vector<std::unique_ptr<DEntry>> entries;
  std::vector<std::unique_ptr<Postponed>> postponed;
  std::unordered_map<void *, Postponed *> postponed_out;  // block -> the run one of whose members writes it
  std::unordered_map<void *, DEntry *> producer;  // block -> its recorded writer
  std::unordered_map<void *, int> pinned;         // block -> recorded entries that read or write it
  std::vector<void *> held_frees;
  std::unordered_map<void *, Known> known;
  uint64_t stats[NXH_DEFER_STAT_COUNT] = {};
};

std::mutex g_windows_mu;
std::unordered_map<nxh_context *, std::unique_ptr<Window>> g_windows;
thread_local bool tls_in_flush = false;

Window *window_of(nxh_context *ctx, bool create) {
  std::lock_guard<std::mutex> g(g_windows_mu);
  auto it = g_windows.find(ctx);
  if (it != g_windows.end()) return it->second.get();
  if (!create) return nullptr;
  return (g_windows[ctx] = std::make_unique<Window>()).get();
}

// ── views ───────────────────────────────────────────────────────────────────
int64_t numel(const nxh_tensor &t) {
  int64_t n = 1;
  for (int i = 0; i < t.ndim; i++) n *= t.shape[i];
  return n;
}
bool same_shape(const nxh_tensor &a, const nxh_tensor &b) {
  if (a.ndim != b.ndim) return false;
  for (int i = 0; i < a.ndim; i++)
    if (a.shape[i] != b.shape[i]) return false;
  return true;
}
bool c_contiguous(const nxh_tensor &t) {
  int64_t acc = 1;
  for (int i = t.ndim - 1; i >= 0; i--) {
    if (t.shape[i] != 1 && t.strides[i] != acc) return false;
    acc *= t.shape[i];
  }
  return true;
}
// The whole result of `e`, as it was written: offset 0, its shape, C-contiguous.
bool identity_of(const nxh_tensor &v, const DEntry *e) {
  return v.offset == 0 && v.dtype == e->out.dtype && same_shape(v, e->out) && c_contiguous(v);
}
// A keepdims result [..., 1] expanded along the last axis to `shape`.
bool row_broadcast(const nxh_tensor &v, const nxh_tensor &shape) {
  if (!same_shape(v, shape) || v.offset != 0 || v.ndim == 0) return false;
  const int n = v.ndim;
  if (v.shape[n - 1] != 1 && v.strides[n - 1] != 0) return false;
  int64_t acc = 1;
  for (int i = n - 2; i >= 0; i--) {
    if (v.shape[i] != 1 && v.strides[i] != acc) return false;
    acc *= v.shape[i];
  }
  return true;
}
bool all_broadcast(const nxh_tensor &v) {
  if (v.offset != 0) return false;
  for (int i = 0; i < v.ndim; i++)
    if (v.shape[i] != 1 && v.strides[i] != 0) return false;
  return true;
}
// A rank-1 tensor of the row length broadcast over the outer dims.
bool vector_broadcast(const nxh_tensor &v, const nxh_tensor &shape) {
  if (!same_shape(v, shape) || v.ndim == 0) return false;
  const int n = v.ndim;
  if (v.shape[n - 1] != 1 && v.strides[n - 1] != 1) return false;
  for (int i = 0; i < n - 1; i++)
    if (v.shape[i] != 1 && v.strides[i] != 0) return false;
  return true;
}
bool same_view(const nxh_tensor &a, const nxh_tensor &b) {
  if (a.data != b.data || a.offset != b.offset || !same_shape(a, b)) return false;
  for (int i = 0; i < a.ndim; i++)
    if (a.shape[i] != 1 && a.strides[i] != b.strides[i]) return false;
  return true;
}
bool is_float_fused(int dt) { return dt == NXH_F16 || dt == NXH_BF16 || dt == NXH_F32 || dt == NXH_F64; }
bool is_island(int dt) { return dt == NXH_F16 || dt == NXH_BF16; }

// An input of an entry.
struct Opnd {
  const nxh_tensor *t = nullptr;
  DEntry *prod = nullptr;
  DEntry *upl = nullptr;
  explicit operator bool() const { return t != nullptr; }
};
Opnd in_of(DEntry *e, int k) { return Opnd{&e->in[k], e->prod[k], e->upl[k]}; }
bool same_operand(const Opnd &a, const Opnd &b) { return a.prod == b.prod && same_view(*a.t, *b.t); }

DEntry *producer_of(const Opnd &o, int kind, int op = -1, bool identity = true) {
  DEntry *e = o.prod;
  if (!e || e->kind != kind || (op >= 0 && e->op != op) || e->fused_into || e->done) return nullptr;
  if (o.t->dtype != e->out.dtype) return nullptr;  // a view that reinterprets the bytes is not that result
  if (identity && !identity_of(*o.t, e)) return nullptr;
  return e;
}
bool rows_ok(const Opnd &o, const nxh_tensor &shape) {
  if (shape.ndim == 0 || shape.ndim > 9 || shape.shape[shape.ndim - 1] > MAX_ROW) return false;
  if (!same_shape(*o.t, shape)) return false;
  return shape.shape[shape.ndim - 1] == 1 || o.t->strides[shape.ndim - 1] == 1;
}
// All recorded readers of the interior results are inside the run (and, where nothing may be
// postponed, no handle to one is left).
thread_local bool tls_may_postpone = true;
bool hidden(const std::vector<DEntry *> &interior, const DEntry *anchor) {
  for (DEntry *e : interior) {
    if (e->alive && !tls_may_postpone) return false;
    for (DEntry *r : e->readers) {
      bool inside = r == anchor;
      for (DEntry *i : interior) inside = inside || i == r;
      if (!inside) return false;
    }
  }
  return true;
}
// The one element every element of the operand equals, in `dtype`'s storage format.
const unsigned char *scalar_of(Window *w, const Opnd &o, int dtype) {
  if (o.t->dtype != dtype || !all_broadcast(*o.t)) return nullptr;
  if (o.prod) return o.prod->kind == D_FULL && !o.prod->done ? o.prod->value : nullptr;
  auto it = w->known.find(o.t->data);
  if (it == w->known.end() || !it->second.has_scalar || it->second.dtype != dtype) return nullptr;
  return it->second.scalar;
}
double scalar_as_double(const unsigned char *p, int dt) {
  if (dt == NXH_F32) {
    float f;
    memcpy(&f, p, 4);
    return f;
  }
  if (dt == NXH_F64) {
    double d;
    memcpy(&d, p, 8);
    return d;
  }
  uint16_t h;
  memcpy(&h, p, 2);
  if (dt == NXH_BF16) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
  }
  // f16
  const int s = h >> 15, e = (h >> 10) & 31, m = h & 1023;
  double v = e == 0 ? ldexp((double)m, -24) : e == 31 ? (m ? NAN : INFINITY) : ldexp(1.0 + m / 1024.0, e - 15);
  return s ? -v : v;
}

// ── plans ───────────────────────────────────────────────────────────────────
struct Plan {
  int stat = 0;
  std::vector<DEntry *> interior;
  bool causal_flag = false;
  bool has_out_view = false;  // ATTENTION: the result goes straight into a following transposing copy's output
  nxh_tensor out_view{};
  DEntry *linear_out = nullptr;  // LINEAR_GELU: the bias add whose result the GELU read
  // operands of the fused call
  Opnd x, a, b, c;
  unsigned char s0[16] = {}, s1[16] = {}, consts[64] = {};
  bool has_s0 = false, has_s1 = false;
  double eps = 0;
};

struct SoftmaxParts {
  std::vector<DEntry *> interior;
  Opnd x, mask;
  const unsigned char *scale = nullptr, *masked = nullptr;
  const nxh_tensor *shape = nullptr;
};

// The softmax run ending in `anchor` (the final division, or the cast behind it).
bool softmax_parts(Window *w, DEntry *anchor, SoftmaxParts *sp) {
  DEntry *d = anchor;
  if (anchor->kind == D_CAST) {
    d = producer_of(in_of(anchor, 0), D_BINARY, NXH_FDIV);
    if (!d || d->out.dtype != NXH_F32 || !is_island(anchor->out.dtype)) return false;
    sp->interior.push_back(d);
  }
  if (d->kind != D_BINARY || d->op != NXH_FDIV || !is_float_fused(d->out.dtype) || d->out.ndim == 0) return false;
  const nxh_tensor &shape = d->out;
  const int last = shape.ndim - 1;
  DEntry *ex = producer_of(in_of(d, 0), D_UNARY, NXH_EXP);
  DEntry *s = d->prod[1];
  if (!ex || !s || s->kind != D_REDUCE || s->op != NXH_SUM || s->n_axes != 1 || s->axes[0] != last || s->fused_into || s->done)
    return false;
  if (!row_broadcast(d->in[1], shape) || producer_of(in_of(s, 0), D_UNARY, NXH_EXP) != ex) return false;
  DEntry *sub = producer_of(in_of(ex, 0), D_BINARY, NXH_SUB);
  if (!sub) return false;
  DEntry *mx = sub->prod[1];
  if (!mx || mx->kind != D_REDUCE || mx->op != NXH_RMAX || mx->n_axes != 1 || mx->axes[0] != last || mx->fused_into ||
      mx->done || !row_broadcast(sub->in[1], shape) || !same_operand(in_of(mx, 0), in_of(sub, 0)))
    return false;
  sp->interior.insert(sp->interior.end(), {ex, s, sub, mx});
  Opnd x = in_of(sub, 0);
  // the mask and the scale in front (attention.ml:93-101), each only if it can be hidden too
  if (DEntry *wh = producer_of(x, D_WHERE)) {
    std::vector<DEntry *> with = sp->interior;
    with.push_back(wh);
    if (hidden(with, anchor)) {
      const unsigned char *fill = scalar_of(w, in_of(wh, 2), wh->out.dtype);
      const nxh_tensor &m = wh->in[0];
      if (fill && same_shape(m, shape) && (shape.shape[last] == 1 || m.strides[last] == 0 || m.strides[last] == 1)) {
        sp->interior.push_back(wh);
        sp->mask = in_of(wh, 0);
        sp->masked = fill;
        x = in_of(wh, 1);
      }
    }
  }
  if (DEntry *mul = producer_of(x, D_BINARY, NXH_MUL)) {
    std::vector<DEntry *> with = sp->interior;
    with.push_back(mul);
    if (hidden(with, anchor)) {
      if (const unsigned char *sc = scalar_of(w, in_of(mul, 1), mul->out.dtype)) {
        sp->interior.push_back(mul);
        sp->scale = sc;
        x = in_of(mul, 0);
      }
    }
  }
  if (!hidden(sp->interior, anchor)) return false;
  sp->x = x;
  sp->shape = &shape;
  return true;
}

int dtype_size(int dt) { return (int)nxh_elem_size(dt); }

bool match_softmax(Window *w, DEntry *anchor, Plan *p) {
  SoftmaxParts sp;
  if (!softmax_parts(w, anchor, &sp) || !rows_ok(sp.x, *sp.shape)) return false;
  p->stat = NXH_DEFER_SOFTMAX;
  p->interior = sp.interior;
  p->x = sp.x;
  p->a = sp.mask;
  const int es = dtype_size(sp.x.t->dtype);
  if (sp.scale) memcpy(p->s0, sp.scale, es), p->has_s0 = true;
  if (sp.masked) memcpy(p->s1, sp.masked, es), p->has_s1 = true;
  return true;
}

// kaun/lib/attention.ml:67-110 for 16-bit operands: cast q and k to float32, Q K^T,
// [scale], [mask], softmax, cast back, probs x V.
bool match_attention(Window *w, DEntry *anchor, Plan *p) {
  if (anchor->kind != D_MATMUL || !is_island(anchor->out.dtype) || anchor->out.ndim < 2) return false;
  const int dt = anchor->out.dtype;
  DEntry *probs = producer_of(in_of(anchor, 0), D_CAST);
  if (!probs || probs->out.dtype != dt) return false;
  SoftmaxParts sp;
  if (!softmax_parts(w, probs, &sp)) return false;
  DEntry *scores = producer_of(sp.x, D_MATMUL);
  if (!scores || scores->out.dtype != NXH_F32) return false;
  DEntry *cq = producer_of(in_of(scores, 0), D_CAST);
  DEntry *ck = scores->prod[1];
  if (!cq || !ck || ck->kind != D_CAST || ck->fused_into || ck->done || ck->out.ndim < 2) return false;
  // the second operand of the scores product is cast(k) with its last two axes swapped
  const nxh_tensor &kt = scores->in[1];
  const int r = ck->out.ndim;
  if (kt.ndim != r || kt.offset != 0) return false;
  {
    int64_t acc = 1, want[NXH_MAX_NDIM];
    for (int i = r - 1; i >= 0; i--) want[i] = acc, acc *= ck->out.shape[i];
    for (int i = 0; i < r; i++) {
      const int j = i == r - 1 ? r - 2 : i == r - 2 ? r - 1 : i;
      if (kt.shape[i] != ck->out.shape[j]) return false;
      if (kt.shape[i] != 1 && kt.strides[i] != want[j]) return false;
    }
  }
  Opnd q = in_of(cq, 0), k = in_of(ck, 0), v = in_of(anchor, 1);
  if (q.t->dtype != dt || k.t->dtype != dt || v.t->dtype != dt) return false;
  const nxh_tensor &qs = *q.t, &ks = *k.t, &vs = *v.t;
  if (qs.ndim != r || vs.ndim != r || ks.ndim != r || r > 6 || !same_shape(ks, vs) || !same_shape(anchor->out, qs)) return false;
  for (int i = 0; i < r - 2; i++)
    if (qs.shape[i] != ks.shape[i]) return false;
  const int64_t hd = qs.shape[r - 1];
  if (ks.shape[r - 1] != hd || (hd != 32 && hd != 64 && hd != 128)) return false;
  if (qs.strides[r - 1] != 1 || ks.strides[r - 1] != 1 || vs.strides[r - 1] != 1) return false;
  std::vector<DEntry *> interior = sp.interior;
  interior.insert(interior.end(), {probs, scores, cq, ck});
  if (!hidden(interior, anchor)) return false;
  bool causal = false;
  Opnd mask = sp.mask;
  if (mask) {
    const int64_t n = qs.shape[r - 2];
    int64_t tag = mask.prod ? mask.prod->causal : 0;
    if (!mask.prod) {
      auto it = w->known.find(mask.t->data);
      if (it != w->known.end()) tag = it->second.causal;
    }
    float fill;
    memcpy(&fill, sp.masked, 4);
    bool ok = tag == n && ks.shape[r - 2] == n && mask.t->offset == 0 && fill == -INFINITY &&
              (n == 1 || (mask.t->strides[r - 2] == n && mask.t->strides[r - 1] == 1));
    for (int i = 0; ok && i < r - 2; i++)
      if (mask.t->shape[i] != 1 && mask.t->strides[i] != 0) ok = false;
    if (ok) causal = true, mask = Opnd{};  // the kernel takes the mask as a flag
  }
  p->stat = NXH_DEFER_ATTENTION;
  p->interior = interior;
  p->x = q;
  p->a = k;
  p->b = v;
  p->c = mask;
  p->causal_flag = causal;
  if (sp.scale) memcpy(p->s0, sp.scale, 4), p->has_s0 = true;
  if (sp.masked) memcpy(p->s1, sp.masked, 4), p->has_s1 = true;
  return true;
}

// kaun/lib/linear.ml:50-52 and the residual add around it (gpt2.ml:165-176).
bool match_linear(Window *w, DEntry *anchor, Plan *p) {
  const int dt = anchor->out.dtype;
  if (anchor->kind != D_BINARY || anchor->op != NXH_ADD || (dt != NXH_F16 && dt != NXH_BF16 && dt != NXH_F32)) return false;
  const nxh_tensor &shape = anchor->out;
  if (shape.ndim < 2) return false;
  const int last = shape.ndim - 1;
  DEntry *mm = nullptr, *inner_add = nullptr;
  Opnd bias, residual;
  auto biased = [&](const Opnd &o, DEntry **add, DEntry **m, Opnd *b) {
    DEntry *e = producer_of(o, D_BINARY, NXH_ADD);
    if (!e) return false;
    DEntry *m0 = producer_of(in_of(e, 0), D_MATMUL);
    if (!m0 || e->prod[1] || !vector_broadcast(e->in[1], shape)) return false;
    *add = e, *m = m0, *b = in_of(e, 1);
    return true;
  };
  // residual + (matmul + bias), either operand order; then matmul + bias; then residual + matmul
  for (int side = 1; side >= 0 && !mm; side--) {
    DEntry *e, *m0;
    Opnd b;
    if (biased(in_of(anchor, side), &e, &m0, &b) && hidden({e, m0}, anchor) && same_shape(anchor->in[1 - side], shape)) {
      inner_add = e, mm = m0, bias = b, residual = in_of(anchor, 1 - side);
    }
  }
  if (!mm) {
    DEntry *m0 = producer_of(in_of(anchor, 0), D_MATMUL);
    if (m0 && !anchor->prod[1] && vector_broadcast(anchor->in[1], shape) && hidden({m0}, anchor)) mm = m0, bias = in_of(anchor, 1);
  }
  if (!mm) {
    for (int side = 1; side >= 0 && !mm; side--) {
      DEntry *m0 = producer_of(in_of(anchor, side), D_MATMUL);
      if (m0 && hidden({m0}, anchor) && same_shape(anchor->in[1 - side], shape)) mm = m0, residual = in_of(anchor, 1 - side);
    }
  }
  if (!mm || !same_shape(mm->out, shape)) return false;
  if (residual && shape.shape[last] > 1 && residual.t->strides[last] != 1) return false;
  p->stat = NXH_DEFER_LINEAR;
  p->interior.clear();
  if (inner_add) p->interior.push_back(inner_add);
  p->interior.push_back(mm);
  p->x = in_of(mm, 0);
  p->a = in_of(mm, 1);
  p->b = bias;
  p->c = residual;
  return true;
}

// anchor: add(mul(normalized, gamma), beta)   (layer_norm.ml:66-68)
bool match_layer_norm(Window *w, DEntry *anchor, Plan *p) {
  const int dt = anchor->out.dtype;
  if (anchor->kind != D_BINARY || anchor->op != NXH_ADD || !is_float_fused(dt) || anchor->out.ndim == 0) return false;
  const nxh_tensor &shape = anchor->out;
  const int last = shape.ndim - 1;
  DEntry *g = producer_of(in_of(anchor, 0), D_BINARY, NXH_MUL);
  if (!g || anchor->prod[1] || !vector_broadcast(anchor->in[1], shape)) return false;
  if (g->prod[1] || !vector_broadcast(g->in[1], shape)) return false;
  std::vector<DEntry *> interior{g};
  const bool island = is_island(dt);
  Opnd n_op = in_of(g, 0);
  int stat = dt;
  if (island) {
    DEntry *c_out = producer_of(n_op, D_CAST);
    if (!c_out) return false;
    interior.push_back(c_out);
    n_op = in_of(c_out, 0);
    stat = NXH_F32;
  }
  DEntry *nrm = producer_of(n_op, D_BINARY, NXH_FDIV);
  if (!nrm || nrm->out.dtype != stat) return false;
  DEntry *xc = producer_of(in_of(nrm, 0), D_BINARY, NXH_SUB);
  DEntry *rt = nrm->prod[1];
  if (!xc || !rt || rt->kind != D_UNARY || rt->op != NXH_SQRT || rt->fused_into || rt->done || !row_broadcast(nrm->in[1], shape))
    return false;
  // keep = shape[:-1] + (1,)
  auto is_keep = [&](const nxh_tensor &t) {
    if (t.ndim != shape.ndim || t.shape[last] != 1) return false;
    for (int i = 0; i < last; i++)
      if (t.shape[i] != shape.shape[i]) return false;
    return true;
  };
  DEntry *add = producer_of(in_of(rt, 0), D_BINARY, NXH_ADD);
  if (!add || !is_keep(add->out)) return false;
  const unsigned char *eps = scalar_of(w, in_of(add, 1), stat);
  DEntry *var = producer_of(in_of(add, 0), D_BINARY, NXH_FDIV);
  if (!eps || !var) return false;
  DEntry *s2 = var->prod[0];
  const unsigned char *cnt2 = scalar_of(w, in_of(var, 1), stat);
  if (!s2 || s2->kind != D_REDUCE || s2->op != NXH_SUM || s2->n_axes != 1 || s2->axes[0] != last || s2->fused_into || s2->done ||
      !cnt2)
    return false;
  // the reduce result [..] seen as keep [.., 1]: same elements in the same order
  auto keep_view_of = [&](const nxh_tensor &v, const DEntry *e) {
    return v.offset == 0 && is_keep(v) && c_contiguous(v) && numel(v) == numel(e->out);
  };
  if (!keep_view_of(var->in[0], s2)) return false;
  DEntry *sq = producer_of(in_of(s2, 0), D_BINARY, NXH_MUL);
  if (!sq || producer_of(in_of(sq, 0), D_BINARY, NXH_SUB) != xc || producer_of(in_of(sq, 1), D_BINARY, NXH_SUB) != xc) return false;
  DEntry *mu = xc->prod[1];
  if (!mu || mu->kind != D_BINARY || mu->op != NXH_FDIV || mu->fused_into || mu->done || !row_broadcast(xc->in[1], shape)) return false;
  DEntry *s1 = mu->prod[0];
  const unsigned char *cnt1 = scalar_of(w, in_of(mu, 1), stat);
  if (!s1 || s1->kind != D_REDUCE || s1->op != NXH_SUM || s1->n_axes != 1 || s1->axes[0] != last || s1->fused_into || s1->done ||
      !cnt1 || !keep_view_of(mu->in[0], s1) || !same_operand(in_of(s1, 0), in_of(xc, 0)))
    return false;
  const double count = (double)shape.shape[last];
  if (scalar_as_double(cnt1, stat) != count || scalar_as_double(cnt2, stat) != count || (double)(float)count != count) return false;
  interior.insert(interior.end(), {nrm, rt, add, var, s2, sq, xc, mu, s1});
  Opnd x = in_of(xc, 0);
  if (island) {
    DEntry *c_in = producer_of(x, D_CAST);
    if (!c_in || !same_shape(c_in->in[0], shape)) return false;
    interior.push_back(c_in);
    x = in_of(c_in, 0);
    if (x.t->dtype != dt) return false;
  }
  const double eps_value = scalar_as_double(eps, stat);
  if (!(eps_value >= 0) || !hidden(interior, anchor) || !rows_ok(x, shape)) return false;
  p->stat = NXH_DEFER_LAYER_NORM;
  p->interior = interior;
  p->x = x;
  p->a = in_of(g, 1);       // gamma
  p->b = in_of(anchor, 1);  // beta
  p->eps = eps_value;
  return true;
}

// fn.ml:31-38, outermost first
bool match_gelu(Window *w, DEntry *anchor, Plan *p) {
  const int d = anchor->out.dtype;
  if (anchor->kind != D_BINARY || anchor->op != NXH_MUL || !is_float_fused(d)) return false;
  const unsigned char *c3 = scalar_of(w, in_of(anchor, 1), d);
  DEntry *wv = producer_of(in_of(anchor, 0), D_BINARY, NXH_MUL);
  if (!c3 || !wv) return false;
  const Opnd x = in_of(wv, 0);
  DEntry *u = producer_of(in_of(wv, 1), D_BINARY, NXH_ADD);
  if (!u) return false;
  const unsigned char *c2 = scalar_of(w, in_of(u, 1), d);
  DEntry *th = producer_of(in_of(u, 0), D_UNARY, NXH_TANH);
  if (!c2 || !th) return false;
  DEntry *inner = producer_of(in_of(th, 0), D_BINARY, NXH_MUL);
  if (!inner) return false;
  const unsigned char *c1 = scalar_of(w, in_of(inner, 1), d);
  DEntry *q = producer_of(in_of(inner, 0), D_BINARY, NXH_ADD);
  if (!c1 || !q || !same_operand(in_of(q, 0), x)) return false;
  DEntry *pp = producer_of(in_of(q, 1), D_BINARY, NXH_MUL);
  if (!pp) return false;
  const unsigned char *c0 = scalar_of(w, in_of(pp, 1), d);
  DEntry *x3 = producer_of(in_of(pp, 0), D_BINARY, NXH_MUL);
  if (!c0 || !x3 || !same_operand(in_of(x3, 0), x)) return false;
  DEntry *x2 = producer_of(in_of(x3, 1), D_BINARY, NXH_MUL);
  if (!x2 || !same_operand(in_of(x2, 0), x) || !same_operand(in_of(x2, 1), x)) return false;
  std::vector<DEntry *> interior{wv, u, th, inner, q, pp, x3, x2};
  if (!hidden(interior, anchor) || !c_contiguous(*x.t) || !same_shape(*x.t, anchor->out)) return false;
  const int es = dtype_size(d);
  memcpy(p->consts, c0, es);
  memcpy(p->consts + es, c1, es);
  memcpy(p->consts + 2 * es, c2, es);
  memcpy(p->consts + 3 * es, c3, es);
  p->stat = NXH_DEFER_GELU;
  p->interior = interior;
  p->x = x;
  // gelu (matmul x w + bias), the first half of the MLP (gpt2.ml:165-176): one GEMM whose
  // epilogue applies the GELU, when nothing else reads the linear layer's result
  if (is_island(d) && x.t->offset == 0) {
    DEntry *add = producer_of(x, D_BINARY, NXH_ADD);
    DEntry *mm = add ? producer_of(in_of(add, 0), D_MATMUL) : nullptr;
    if (mm && !add->prod[1] && add->out.ndim >= 2 && vector_broadcast(add->in[1], add->out) && same_shape(mm->out, add->out)) {
      std::vector<DEntry *> with = interior;
      with.push_back(add);
      with.push_back(mm);
      if (hidden(with, anchor)) {
        p->stat = NXH_DEFER_LINEAR_GELU;
        p->interior = with;
        p->linear_out = add;
        p->x = in_of(mm, 0);
        p->a = in_of(mm, 1);
        p->b = in_of(add, 1);
      }
    }
  }
  return true;
}

bool match(Window *w, DEntry *e, Plan *p) {
  if (e->kind == D_MATMUL) return match_attention(w, e, p);
  if (e->kind == D_CAST) return match_softmax(w, e, p);
  if (e->kind == D_BINARY) {
    if (e->op == NXH_ADD) return match_linear(w, e, p) || (*p = Plan{}, match_layer_norm(w, e, p));
    if (e->op == NXH_MUL) return match_gelu(w, e, p);
    if (e->op == NXH_FDIV) return match_softmax(w, e, p);
  }
  return false;
}

// ── issuing ─────────────────────────────────────────────────────────────────
int issue(nxh_context *ctx, DEntry *e);

int issue_inputs(nxh_context *ctx, DEntry *e) {
  // a scalar that something outside a fused run still reads is filled now
  for (int k = 0; k < e->nin; k++)
    if (e->prod[k] && !e->prod[k]->done && e->prod[k]->kind == D_FULL)
      if (int rc = issue(ctx, e->prod[k])) return rc;
  // and an upload that nobody holds any more happens now
  for (int k = 0; k < e->nin; k++)
    if (e->upl[k] && !e->upl[k]->done)
      if (int rc = issue(ctx, e->upl[k])) return rc;
  return NXH_OK;
}

int issue(nxh_context *ctx, DEntry *e) {
  if (e->done) return NXH_OK;
  if (int rc = issue_inputs(ctx, e)) return rc;
  e->done = true;
  switch (e->kind) {
    case D_UNARY: return nxh_unary(ctx, e->op, &e->out, &e->in[0]);
    case D_BINARY: return nxh_binary(ctx, e->op, &e->out, &e->in[0], &e->in[1]);
    case D_COMPARE: return nxh_compare(ctx, e->op, &e->out, &e->in[0], &e->in[1]);
    case D_WHERE: return nxh_where(ctx, &e->out, &e->in[0], &e->in[1], &e->in[2]);
    case D_CAST: return nxh_cast(ctx, &e->out, &e->in[0]);
    case D_REDUCE: return nxh_reduce(ctx, e->op, &e->out, &e->in[0], e->axes, e->n_axes);
    case D_MATMUL: return nxh_matmul(ctx, &e->out, &e->in[0], &e->in[1]);
    case D_COPY: return nxh_copy(ctx, &e->out, &e->in[0]);
    case D_UPLOAD: return nxh_memcpy_h2d(ctx, e->out.data, e->payload.data(), e->payload.size());
    default: return nxh_fill(ctx, &e->out, e->value);
  }
}

// The rank-1 parameter behind a vector broadcast over `shape`: its last axis.
nxh_tensor vector_of(const nxh_tensor &v) {
  nxh_tensor t = v;
  const int last = v.ndim - 1;
  t.ndim = 1;
  t.shape[0] = v.shape[last];
  t.strides[0] = v.shape[last] > 1 ? v.strides[last] : 1;
  return t;
}

int run_plan(nxh_context *ctx, DEntry *anchor, const Plan &p) {
  // inputs of the fused call that are recorded scalars never reach it as tensors; the
  // tensors it reads are results of entries issued before the run or existing storage
  for (const Opnd *o : {&p.x, &p.a, &p.b, &p.c}) {
    if (*o && o->prod && !o->prod->done && o->prod->kind == D_FULL)
      if (int rc = issue(ctx, o->prod)) return rc;
    if (*o && o->upl && !o->upl->done)
      if (int rc = issue(ctx, o->upl)) return rc;
  }
  switch (p.stat) {
    case NXH_DEFER_SOFTMAX:
      return nxh_softmax_rows(ctx, &anchor->out, p.x.t, p.has_s0 ? p.s0 : nullptr, p.a ? p.a.t : nullptr, p.has_s1 ? p.s1 : nullptr);
    case NXH_DEFER_ATTENTION:
      return nxh_attention(ctx, p.has_out_view ? &p.out_view : &anchor->out, p.x.t, p.a.t, p.b.t, p.has_s0 ? p.s0 : nullptr, p.c ? p.c.t : nullptr,
                           p.has_s1 ? p.s1 : nullptr, p.causal_flag ? 1 : 0);
    case NXH_DEFER_LINEAR: {
      nxh_tensor bias;
      if (p.b) bias = vector_of(*p.b.t);
      return nxh_linear(ctx, &anchor->out, p.x.t, p.a.t, p.b ? &bias : nullptr, p.c ? p.c.t : nullptr);
    }
    case NXH_DEFER_LAYER_NORM: {
      nxh_tensor gamma = vector_of(*p.a.t), beta = vector_of(*p.b.t);
      return nxh_layer_norm_rows(ctx, &anchor->out, p.x.t, &gamma, &beta, p.eps);
    }
    case NXH_DEFER_LINEAR_GELU: {
      nxh_tensor bias = vector_of(*p.b.t);
      const int rc = nxh_linear_gelu_tanh(ctx, &anchor->out, p.x.t, p.a.t, &bias, p.consts);
      if (rc != NXH_FAILURE) return rc;
      // the epilogue does not take this shape: the fused linear into the block the bias add
      // was given (held back while the record uses it), then the GELU from there
      if (const int r2 = nxh_linear(ctx, &p.linear_out->out, p.x.t, p.a.t, &bias, nullptr)) return r2;
      return nxh_gelu_tanh(ctx, &anchor->out, &p.linear_out->out, p.consts);
    }
    default: return nxh_gelu_tanh(ctx, &anchor->out, p.x.t, p.consts);
  }
}

void unpin(Window *w, void *block) {
  auto it = w->pinned.find(block);
  if (it != w->pinned.end() && --it->second <= 0) w->pinned.erase(it);
}
void unpin_entry(Window *w, const DEntry *e) {
  unpin(w, e->out.data);
  for (int i = 0; i < e->nin; i++) unpin(w, e->in[i].data);
}
// What the window now knows about a result that was written and is still held.
void remember(Window *w, const DEntry *e) {
  if (!e->alive || (e->kind != D_FULL && !e->causal)) return;
  Known &k = w->known[e->out.data];
  k = Known{};
  k.dtype = e->out.dtype;
  if (e->kind == D_FULL) memcpy(k.scalar, e->value, 16), k.has_scalar = true;
  k.causal = e->causal;
}
// Frees that were held back for blocks nothing recorded or postponed uses any more.
void release_held(nxh_context *ctx, Window *w) {
  std::vector<void *> frees;
  frees.swap(w->held_frees);
  for (void *p : frees) {
    if (w->pinned.count(p)) {
      w->held_frees.push_back(p);
      continue;
    }
    w->known.erase(p);
    std::lock_guard<std::mutex> g(ctx->mu);
    nxh_free_locked(ctx, p);
  }
}

// Ends a postponed run: with `write`, its members are issued as recorded first (somebody is
// about to look); without, they are forgotten (every handle is gone).
int retire(nxh_context *ctx, Window *w, Postponed *run, bool write) {
  int rc = NXH_OK;
  const bool outer = tls_in_flush;
  tls_in_flush = true;
  for (auto &m : run->members) {
    if (write && !rc && !m->done) {
      rc = issue(ctx, m.get());
      w->stats[NXH_DEFER_ISSUED]++;
      w->stats[NXH_DEFER_MATERIALISED]++;
      if (!rc) remember(w, m.get());
    }
    w->postponed_out.erase(m->out.data);
    unpin_entry(w, m.get());
  }
  tls_in_flush = outer;
  for (size_t i = 0; i < w->postponed.size(); i++)
    if (w->postponed[i].get() == run) {
      w->postponed.erase(w->postponed.begin() + (long)i);
      break;
    }
  release_held(ctx, w);
  return rc;
}
int retire_all(nxh_context *ctx, Window *w, bool write) {
  int rc = NXH_OK;
  while (!w->postponed.empty()) {
    const int r = retire(ctx, w, w->postponed.front().get(), write);
    if (!rc) rc = r;
  }
  return rc;
}
// Before `block` is read: the postponed run that would have written it runs now. A scalar fill
// or a causal mask that rode along with a run depends on nothing in it and is written alone.
int settle_read(nxh_context *ctx, Window *w, const void *block) {
  if (w->postponed.empty()) return NXH_OK;
  auto it = w->postponed_out.find(const_cast<void *>(block));
  if (it == w->postponed_out.end()) return NXH_OK;
  for (auto &m : it->second->members) {
    if (m->out.data != block || (m->kind != D_FULL && m->kind != D_UPLOAD && !(m->kind == D_COMPARE && m->causal))) continue;
    if (m->done) return NXH_OK;
    const bool outer = tls_in_flush;
    tls_in_flush = true;
    int rc = NXH_OK;
    // a causal mask is computed from uploads that may be waiting beside it
    if (m->kind == D_COMPARE)
      for (auto &u : it->second->members)
        if (!rc && u->kind == D_UPLOAD && !u->done && (u->out.data == m->in[0].data || u->out.data == m->in[1].data)) {
          rc = issue(ctx, u.get());
          w->stats[NXH_DEFER_ISSUED]++;
          w->stats[NXH_DEFER_MATERIALISED]++;
        }
    if (!rc) rc = issue(ctx, m.get());
    tls_in_flush = outer;
    w->stats[NXH_DEFER_ISSUED]++;
    w->stats[NXH_DEFER_MATERIALISED]++;
    if (!rc) remember(w, m.get());
    return rc;
  }
  return retire(ctx, w, it->second, true);
}
// Before `block` is written by anything but the record: a postponed run may read it, or write it later.
int settle_write(nxh_context *ctx, Window *w, const void *block) {
  if (w->postponed.empty() || !w->pinned.count(const_cast<void *>(block))) return NXH_OK;
  return retire_all(ctx, w, true);
}

// Executes the record. Called with w->mu held.
int flush_locked(nxh_context *ctx, Window *w) {
  if (w->entries.empty()) return NXH_OK;
  std::vector<std::unique_ptr<DEntry>> entries;
  entries.swap(w->entries);
  w->producer.clear();
  w->stats[NXH_DEFER_FLUSHES]++;
  {
    std::lock_guard<std::mutex> g(ctx->mu);
    w->may_postpone = ctx->capture == nullptr;
  }
  tls_may_postpone = w->may_postpone;
  std::unordered_map<DEntry *, Plan> plans;
  for (size_t i = entries.size(); i-- > 0;) {
    DEntry *e = entries[i].get();
    if (e->fused_into || plans.count(e)) continue;
    Plan p;
    if (match(w, e, &p)) {
      for (DEntry *inner : p.interior) inner->fused_into = e;
      plans.emplace(e, std::move(p));
    }
  }
  // attention.ml:218-265 merges the heads by `contiguous (swapaxes ...)` of the attention result:
  // when that copy is the result's only reader, the kernel writes through the copy's output with
  // the permuted strides, and the copy becomes the run's last entry.
  {
    std::vector<std::pair<DEntry *, DEntry *>> moves;  // (attention anchor, copy)
    for (auto &pl : plans) {
      DEntry *e = pl.first;
      if (pl.second.stat != NXH_DEFER_ATTENTION || e->readers.size() != 1) continue;
      DEntry *r = e->readers[0];
      if (r->kind != D_COPY || r->prod[0] != e || r->fused_into || plans.count(r) || (e->alive && !w->may_postpone)) continue;
      const nxh_tensor &v = r->in[0], &o = e->out, &ro = r->out;
      const int nd = o.ndim;
      if (v.ndim != nd || ro.ndim != nd || v.offset != 0 || ro.dtype != o.dtype || !same_shape(v, ro) || !c_contiguous(ro) ||
          ro.offset != 0)
        continue;
      // v is a permutation of the result's axes: axis j of v is axis perm[j] of the result
      int64_t cs[NXH_MAX_NDIM], acc = 1;
      for (int i = nd - 1; i >= 0; i--) cs[i] = acc, acc *= o.shape[i];
      int perm[NXH_MAX_NDIM];
      bool used[NXH_MAX_NDIM] = {}, ok = true;
      for (int j = 0; j < nd && ok; j++) {
        int hit = -1;
        for (int i = 0; i < nd && hit < 0; i++)
          if (!used[i] && o.shape[i] == v.shape[j] && (o.shape[i] == 1 || cs[i] == v.strides[j])) hit = i;
        if (hit < 0) ok = false;
        else used[hit] = true, perm[j] = hit;
      }
      if (!ok || perm[nd - 1] != nd - 1) continue;  // rows stay contiguous
      nxh_tensor view = o;                           // the result's shape, laid over the copy's output
      view.data = ro.data;
      view.offset = 0;
      for (int j = 0; j < nd; j++) view.strides[perm[j]] = ro.strides[j];
      pl.second.has_out_view = true;
      pl.second.out_view = view;
      moves.push_back({e, r});
    }
    for (auto &mv : moves) {
      Plan p = std::move(plans.at(mv.first));
      plans.erase(mv.first);
      p.interior.push_back(mv.first);
      for (DEntry *inner : p.interior) inner->fused_into = mv.second;
      plans.emplace(mv.second, std::move(p));
    }
  }
  // A scalar fill, or a causal mask taken as a flag, that only one fused run reads belongs to that
  // run: it is written only if the run is (when it is declined, or postponed and looked at later).
  std::unordered_map<DEntry *, DEntry *> home;  // entry -> the anchor of its run
  for (auto &up : entries) {
    DEntry *e = up.get();
    if ((e->kind != D_FULL && !(e->kind == D_COMPARE && e->causal)) || e->readers.empty()) continue;
    if (e->alive && !w->may_postpone) continue;
    DEntry *anchor = nullptr;
    bool single = true;
    for (DEntry *r : e->readers) {
      DEntry *a = r->fused_into ? r->fused_into : (plans.count(r) ? r : nullptr);
      single = single && a && (!anchor || anchor == a);
      anchor = a;
    }
    if (!single) continue;
    const Plan &pl = plans.at(anchor);
    if (e->kind == D_COMPARE && !(pl.stat == NXH_DEFER_ATTENTION && pl.causal_flag)) continue;
    home[e] = anchor;
  }
  // an upload that only such entries read (the aranges of a causal mask) goes with them
  for (size_t i = entries.size(); i-- > 0;) {
    DEntry *e = entries[i].get();
    if (e->kind != D_UPLOAD || e->readers.empty() || (e->alive && !w->may_postpone)) continue;
    DEntry *anchor = nullptr;
    bool single = true;
    for (DEntry *r : e->readers) {
      auto h = home.find(r);
      single = single && h != home.end() && (!anchor || anchor == h->second);
      if (h != home.end()) anchor = h->second;
    }
    if (single && anchor) home[e] = anchor;
  }
  auto members_of = [&](DEntry *anchor) {
    std::vector<DEntry *> run = plans.at(anchor).interior;
    for (auto &h : home)
      if (h.second == anchor) run.push_back(h.first);
    std::sort(run.begin(), run.end(), [](DEntry *a, DEntry *b) { return a->id < b->id; });
    return run;
  };
  // Linear layers (bias, no residual) that read one x through equal views, with weights, biases
  // and outputs of one shape and layout, run as ONE launch at the place of the last of them:
  // the q / k / v projections of attention.ml:218-265. Nothing recorded before that place
  // may read an earlier member's result.
  std::unordered_map<DEntry *, std::vector<DEntry *>> group_at;  // last member -> all members, in order
  std::unordered_map<DEntry *, DEntry *> grouped;                 // member -> last member
  {
    auto same_layout = [](const nxh_tensor &a, const nxh_tensor &b) {
      if (a.dtype != b.dtype || a.offset != b.offset || !same_shape(a, b)) return false;
      for (int i = 0; i < a.ndim; i++)
        if (a.shape[i] != 1 && a.strides[i] != b.strides[i]) return false;
      return true;
    };
    std::vector<std::vector<DEntry *>> open;
    for (auto &up : entries) {
      DEntry *e = up.get();
      auto it = plans.find(e);
      if (it == plans.end() || it->second.stat != NXH_DEFER_LINEAR || !it->second.b || it->second.c) continue;
      const Plan &pe = it->second;
      bool placed = false;
      for (auto &g : open) {
        const Plan &p0 = plans.at(g.front());
        if (g.size() >= 3 || !same_operand(pe.x, p0.x) || !same_layout(*pe.a.t, *p0.a.t) || !same_layout(*pe.b.t, *p0.b.t) ||
            !same_layout(e->out, g.front()->out))
          continue;
        bool safe = true;
        for (DEntry *m : g) {
          for (DEntry *r : m->readers) safe = safe && r->id > e->id;
          // a member whose own run holds entries of another run's operands stays alone
          for (DEntry *inner : plans.at(m).interior)
            for (DEntry *r : inner->readers) safe = safe && (r->fused_into == m || r == m);
        }
        if (!safe) continue;
        g.push_back(e);
        placed = true;
        break;
      }
      if (!placed) open.push_back({e});
    }
    for (auto &g : open)
      if (g.size() >= 2) {
        for (DEntry *m : g) grouped[m] = g.back();
        group_at[g.back()] = g;
      }
  }
  std::vector<DEntry *> fused;  // anchors whose fused call ran
  int rc = NXH_OK;
  tls_in_flush = true;
  // One fused run at its anchor: the fused call, or (declined) the run as recorded.
  auto run_anchor = [&](DEntry *e) {
    Plan &pl = plans.at(e);
    e->done = true;
    rc = run_plan(ctx, e, pl);
    if (rc == NXH_FAILURE) {
      // the fused form was declined: the run as recorded, in its own order
      w->stats[NXH_DEFER_FALLBACKS]++;
      rc = NXH_OK;
      for (DEntry *inner : members_of(e)) {
        inner->fused_into = nullptr;
        home.erase(inner);
        if (!rc) rc = issue(ctx, inner), w->stats[NXH_DEFER_ISSUED]++;
      }
      e->done = false;
      if (!rc) rc = issue(ctx, e), w->stats[NXH_DEFER_ISSUED]++;
    } else if (!rc) {
      w->stats[pl.stat]++;
      fused.push_back(e);
    }
  };
  for (auto &up : entries) {
    DEntry *e = up.get();
    if (rc) break;
    if (e->fused_into || e->done || home.count(e)) continue;
    if (e->kind == D_COMPARE && e->causal && !e->alive && !e->readers.empty()) {
      // a causal mask nobody holds any more, whose readers (several runs) all took it as a flag
      bool flagged = true;
      for (DEntry *r : e->readers) {
        auto it = r->fused_into ? plans.find(r->fused_into) : plans.end();
        flagged = flagged && it != plans.end() && it->second.stat == NXH_DEFER_ATTENTION && it->second.causal_flag;
      }
      if (flagged) {
        e->done = e->skipped = true;
        continue;
      }
    }
    if (e->kind == D_FULL || e->kind == D_UPLOAD) {
      // filled / sent only if a handle is left (or, in issue(), when a reader outside a fused run is issued)
      if (e->alive) rc = issue(ctx, e);
      continue;
    }
    auto it = plans.find(e);
    if (it == plans.end()) {
      rc = issue(ctx, e);
      w->stats[NXH_DEFER_ISSUED]++;
      continue;
    }
    auto gr = grouped.find(e);
    if (gr == grouped.end()) {
      run_anchor(e);
      continue;
    }
    if (gr->second != e) continue;  // runs with the last member of its group
    const std::vector<DEntry *> &members = group_at.at(e);
    const nxh_tensor *outs[3], *ws[3], *biases[3];
    nxh_tensor bias_v[3];
    for (size_t i = 0; i < members.size(); i++) {
      const Plan &pm = plans.at(members[i]);
      outs[i] = &members[i]->out;
      ws[i] = pm.a.t;
      bias_v[i] = vector_of(*pm.b.t);
      biases[i] = &bias_v[i];
    }
    const int grc = nxh_linear_group(ctx, (int)members.size(), outs, plans.at(members[0]).x.t, ws, biases);
    if (grc == NXH_OK) {
      for (DEntry *m : members) {
        m->done = true;
        w->stats[NXH_DEFER_LINEAR]++;
        fused.push_back(m);
      }
      w->stats[NXH_DEFER_GROUPED] += members.size();
    } else if (grc == NXH_FAILURE) {
      for (DEntry *m : members)
        if (!rc) run_anchor(m);  // one by one, each with its own fallback
    } else {
      rc = grc;
    }
  }
  tls_in_flush = false;
  // The members of a fused run that somebody still holds stay behind with the rest of their run.
  std::unordered_map<DEntry *, Postponed *> kept;
  if (!rc && w->may_postpone)
    for (DEntry *anchor : fused) {
      std::vector<DEntry *> run = members_of(anchor);
      int alive = 0;
      for (DEntry *m : run) alive += m->alive ? 1 : 0;
      if (!alive) continue;
      auto pr = std::make_unique<Postponed>();
      pr->alive = alive;
      for (DEntry *m : run) kept[m] = pr.get();
      w->postponed.push_back(std::move(pr));
    }
  // A scalar fill, an upload or a flagged causal mask that several runs read rides along with
  // none of them and, with its handle gone, was not written above. A member that stays behind
  // would read that block when it is issued as recorded later: it is written now, while the
  // entry that says how still exists (the block is pinned by the member, so it is still there).
  if (!kept.empty()) {
    tls_in_flush = true;
    for (auto &up : entries) {
      DEntry *e = up.get();
      if (!kept.count(e)) continue;
      for (int i = 0; i < 3 && !rc; i++)
        for (DEntry *src : {e->prod[i], e->upl[i]}) {
          if (!src || kept.count(src) || (src->done && !src->skipped) || rc) continue;
          if (src->kind != D_FULL && src->kind != D_UPLOAD && !(src->kind == D_COMPARE && src->causal)) continue;
          src->done = src->skipped = false;
          rc = issue(ctx, src);
          w->stats[NXH_DEFER_ISSUED]++;
        }
    }
    tls_in_flush = false;
  }
  for (auto &up : entries) {
    DEntry *e = up.get();
    auto k = kept.find(e);
    if (k == kept.end()) {
      if (e->done && !rc) remember(w, e);
      unpin_entry(w, e);
      continue;
    }
    // cut loose from entries that are about to go away; its operands' blocks stay pinned
    for (int i = 0; i < 3; i++) e->prod[i] = e->upl[i] = nullptr;
    e->readers.clear();
    e->fused_into = nullptr;
    w->postponed_out[e->out.data] = k->second;
    w->stats[NXH_DEFER_POSTPONED]++;
    k->second->members.push_back(std::move(up));  // `entries` is in issue order, so the run is too
  }
  release_held(ctx, w);
  return rc;
}

// n if `compare op x y` is the n x n causal mask of attention.ml:236-243: cmple of arange(n)
// along the columns against arange(n) down the rows, so that element [i][j] is (j <= i).
int64_t causal_length(Window *w, int op, const nxh_tensor *x, const nxh_tensor *y, DEntry *const *prod) {
  if (op != NXH_CMPLE || x->ndim != 2 || x->shape[0] != x->shape[1] || x->dtype != NXH_I32 || prod[0] || prod[1]) return 0;
  const int64_t n = x->shape[0];
  auto kx = w->known.find(x->data), ky = w->known.find(y->data);
  if (kx == w->known.end() || ky == w->known.end()) return 0;
  const auto &hx = kx->second.host_i32, &hy = ky->second.host_i32;
  if ((int64_t)hx.size() != n || (int64_t)hy.size() != n) return 0;
  if (x->offset != 0 || y->offset != 0) return 0;
  if (n > 1 && (x->strides[0] != 0 || x->strides[1] != 1 || y->strides[0] != 1 || y->strides[1] != 0)) return 0;
  for (int64_t i = 0; i < n; i++)
    if (hx[i] != i || hy[i] != i) return 0;
  return n;
}

}  // namespace

// ── what the entry points call ──────────────────────────────────────────────

bool nxh_defer_active(nxh_context *ctx) {
  if (!ctx || tls_in_flush) return false;
  Window *w = window_of(ctx, false);
  return w && w->on;
}

int nxh_defer_flush(nxh_context *ctx) {
  if (tls_in_flush) return NXH_OK;
  Window *w = window_of(ctx, false);
  if (!w) return NXH_OK;
  std::lock_guard<std::mutex> g(w->mu);
  return flush_locked(ctx, w);
}

// Before an entry point that is not recorded and does not say what it reads: the record runs
// first, everything postponed is written, and whatever the window knew about the blocks this
// call writes is forgotten.
int nxh_defer_barrier(nxh_context *ctx, const nxh_tensor *out0, const nxh_tensor *out1, const nxh_tensor *out2) {
  if (!ctx || tls_in_flush) return NXH_OK;
  Window *w = window_of(ctx, false);
  if (!w) return NXH_OK;
  std::lock_guard<std::mutex> g(w->mu);
  int rc = flush_locked(ctx, w);
  if (!rc) rc = retire_all(ctx, w, true);
  for (const nxh_tensor *t : {out0, out1, out2})
    if (t) w->known.erase(t->data);
  return rc;
}

// The same for an entry point that names its operands: the first n_out are written, the
// others read. Only the postponed runs those blocks belong to are written.
int nxh_defer_touch(nxh_context *ctx, const nxh_tensor *const *tensors, int n, int n_out) {
  if (!ctx || tls_in_flush) return NXH_OK;
  Window *w = window_of(ctx, false);
  if (!w) return NXH_OK;
  std::lock_guard<std::mutex> g(w->mu);
  int rc = flush_locked(ctx, w);
  for (int i = 0; i < n; i++) {
    const nxh_tensor *t = tensors[i];
    if (!t) continue;
    if (i < n_out) {
      if (!rc) rc = settle_write(ctx, w, t->data);
      w->known.erase(t->data);
    } else if (!rc) {
      rc = settle_read(ctx, w, t->data);
    }
  }
  return rc;
}

// An entry point that touches no tensor (a synchronisation, a timer): the record runs, what is
// postponed stays so.
int nxh_defer_quiet(nxh_context *ctx) {
  if (!ctx || tls_in_flush) return NXH_OK;
  Window *w = window_of(ctx, false);
  if (!w) return NXH_OK;
  std::lock_guard<std::mutex> g(w->mu);
  return flush_locked(ctx, w);
}

// A host read of device bytes at `src` (any address inside a block).
int nxh_defer_host_read(nxh_context *ctx, const void *src) {
  if (!ctx || tls_in_flush) return NXH_OK;
  Window *w = window_of(ctx, false);
  if (!w) return NXH_OK;
  std::lock_guard<std::mutex> g(w->mu);
  int rc = flush_locked(ctx, w);
  if (rc || w->postponed.empty()) return rc;
  const void *block = nullptr;
  {
    std::lock_guard<std::mutex> a(ctx->mu);
    for (auto &po : w->postponed_out) {
      auto live = ctx->live.find(po.first);
      const char *base = (const char *)po.first;
      if (live != ctx->live.end() && (const char *)src >= base && (const char *)src < base + std::max<size_t>(live->second, 1)) block = po.first;
    }
  }
  return block ? settle_read(ctx, w, block) : NXH_OK;
}

// Records one primitive. Returns NXH_OK when recorded, -1 when the call has to run now (the
// record has been executed first), or a failure of that execution.
int nxh_defer_record(nxh_context *ctx, int kind, int op, const nxh_tensor *out, const nxh_tensor *const *ins, int nin,
                     const int32_t *axes, int n_axes, const void *value) {
  Window *w = window_of(ctx, false);
  if (!w) return -1;
  std::lock_guard<std::mutex> g(w->mu);
  bool ok = out && out->ndim >= 0 && out->ndim <= NXH_MAX_NDIM && n_axes <= NXH_MAX_NDIM;
  for (int k = 0; ok && k < nin; k++) ok = ins[k] && ins[k]->ndim >= 0 && ins[k]->ndim <= NXH_MAX_NDIM;
  // an operand that a postponed run would have written is written now, ahead of the record
  // (nothing recorded writes what that run reads: recorded outputs are fresh blocks)
  for (int k = 0; ok && k < nin; k++)
    if (int rc = settle_read(ctx, w, ins[k]->data)) return rc;
  // The output must be a whole block of this context that no recorded entry touches yet:
  // results are fresh allocations (backend_intf.ml:61-67); anything else runs now.
  bool capturing = false;
  if (ok) {
    std::lock_guard<std::mutex> a(ctx->mu);
    ok = ctx->live.count(out->data) != 0;
    capturing = ctx->capture != nullptr;
  }
  ok = ok && out->offset == 0 && c_contiguous(*out) && !w->pinned.count(out->data);
  if (ok && kind == D_FULL) ok = numel(*out) == 1 && !nxh_is_packed(out->dtype);
  if (!ok) {
    int rc = flush_locked(ctx, w);
    // the flush itself may have postponed the run that writes one of this call's operands
    for (int k = 0; !rc && k < nin; k++)
      if (ins[k]) rc = settle_read(ctx, w, ins[k]->data);
    if (out) {
      if (!rc) rc = settle_write(ctx, w, out->data);
      w->known.erase(out->data);
    }
    return rc ? rc : -1;
  }
  auto e = std::make_unique<DEntry>();
  e->kind = kind, e->op = op, e->nin = nin, e->out = *out, e->n_axes = n_axes;
  e->id = w->entries.size();
  for (int i = 0; i < n_axes; i++) e->axes[i] = axes[i];
  if (value) memcpy(e->value, value, (size_t)nxh_elem_size(out->dtype));
  for (int k = 0; k < nin; k++) {
    e->in[k] = *ins[k];
    auto it = w->producer.find(ins[k]->data);
    if (it != w->producer.end()) {
      (it->second->kind == D_UPLOAD ? e->upl[k] : e->prod[k]) = it->second;
      it->second->readers.push_back(e.get());
    }
    w->pinned[ins[k]->data]++;
  }
  w->pinned[out->data]++;
  if (kind == D_COMPARE) e->causal = causal_length(w, op, ins[0], ins[1], e->prod);
  w->known.erase(out->data);
  w->producer[out->data] = e.get();
  w->entries.push_back(std::move(e));
  w->stats[NXH_DEFER_RECORDED]++;
  // (while a graph is captured nothing executes anyway: the record stays whole)
  if (w->entries.size() >= LIMIT || (kind == D_COPY && !capturing && w->entries.size() >= COPY_FLUSH)) return flush_locked(ctx, w);
  return NXH_OK;
}

// nxh_free: true when the window took the free over (the block is used by the record, or by a
// postponed run that other handles keep).
bool nxh_defer_free(nxh_context *ctx, void *p) {
  if (tls_in_flush) return false;
  Window *w = window_of(ctx, false);
  if (!w) return false;
  std::lock_guard<std::mutex> g(w->mu);
  auto it = w->producer.find(p);
  if (it != w->producer.end()) it->second->alive = false;
  auto po = w->postponed_out.find(p);
  if (po != w->postponed_out.end()) {
    Postponed *run = po->second;
    for (auto &m : run->members)
      if (m->out.data == p && m->alive) m->alive = false, run->alive--;
    if (run->alive <= 0) retire(ctx, w, run, false);  // nobody can look any more
  }
  if (w->pinned.count(p)) {
    w->held_frees.push_back(p);
    return true;
  }
  w->known.erase(p);
  return false;
}

// nxh_memcpy_h2d. With the mode on, a small upload into a whole block that nothing recorded touches
// waits in the record with its bytes (*recorded = true: the caller copies nothing): the aranges
// behind a causal mask that is taken as a flag are then never sent at all. Otherwise the record
// runs first if it touches the block, and so does whatever is postponed. What a small upload
// holds is remembered either way (the aranges of a causal mask are recognised from it).
int nxh_defer_uploaded(nxh_context *ctx, void *dst, const void *src, size_t bytes, bool *recorded) {
  *recorded = false;
  if (tls_in_flush) return NXH_OK;
  Window *w = window_of(ctx, false);
  if (!w) return NXH_OK;
  std::lock_guard<std::mutex> g(w->mu);
  int rc = NXH_OK;
  // the ABI takes any device address: what the window knows is kept per block, so an upload
  // into the middle of one counts as a write of that block
  void *block = dst;
  {
    std::lock_guard<std::mutex> a(ctx->mu);
    auto it = ctx->live.upper_bound(dst);
    if (it != ctx->live.begin()) {
      --it;
      if ((const char *)dst < (const char *)it->first + std::max<size_t>(it->second, 1)) block = it->first;
    }
  }
  const bool pinned = w->pinned.count(block) != 0;
  if (pinned) {
    rc = flush_locked(ctx, w);
    if (!rc) rc = settle_write(ctx, w, block);
  }
  w->known.erase(block);
  if (rc || !w->on || bytes == 0 || bytes > UPLOAD_LIMIT || block != dst) return rc;
  if (bytes % 4 == 0) {
    Known &k = w->known[dst];
    k.dtype = NXH_I32;
    k.host_i32.resize(bytes / 4);
    memcpy(k.host_i32.data(), src, bytes);
  }
  bool whole = false;
  {
    std::lock_guard<std::mutex> a(ctx->mu);
    auto live = ctx->live.find(dst);
    whole = live != ctx->live.end() && live->second >= bytes;
  }
  if (!whole || w->pinned.count(dst)) return NXH_OK;
  auto e = std::make_unique<DEntry>();
  e->kind = D_UPLOAD;
  e->id = w->entries.size();
  e->out.data = dst;
  e->out.dtype = NXH_U8;
  e->out.ndim = 1;
  e->out.shape[0] = (int64_t)bytes;
  e->out.strides[0] = 1;
  e->payload.assign((const unsigned char *)src, (const unsigned char *)src + bytes);
  w->pinned[dst]++;
  w->producer[dst] = e.get();
  w->entries.push_back(std::move(e));
  w->stats[NXH_DEFER_RECORDED]++;
  *recorded = true;
  if (w->entries.size() >= LIMIT) return flush_locked(ctx, w);
  return NXH_OK;
}

void nxh_defer_context_gone(nxh_context *ctx) {
  std::lock_guard<std::mutex> g(g_windows_mu);
  g_windows.erase(ctx);
}

NXH_EXPORT int nxh_set_deferred(nxh_context *ctx, int on) {
  if (!ctx) return nxh_fail(NXH_INVALID_ARGUMENT, "set_deferred", "null context");
  Window *w = window_of(ctx, true);
  std::lock_guard<std::mutex> g(w->mu);
  int rc = flush_locked(ctx, w);
  w->on = on != 0;
  if (!w->on) {
    // with the mode off no call announces what it reads: nothing may stay unwritten
    const int r = retire_all(ctx, w, true);
    if (!rc) rc = r;
    w->known.clear();
  }
  return rc;
}

NXH_EXPORT int nxh_deferred_stats(nxh_context *ctx, uint64_t *stats, int count) {
  if (!ctx || !stats) return nxh_fail(NXH_INVALID_ARGUMENT, "deferred_stats", "null argument");
  Window *w = window_of(ctx, false);
  for (int i = 0; i < count; i++) stats[i] = 0;
  if (!w) return NXH_OK;
  std::lock_guard<std::mutex> g(w->mu);
  for (int i = 0; i < count && i < NXH_DEFER_STAT_COUNT; i++) stats[i] = w->stats[i];
  return NXH_OK;
}
