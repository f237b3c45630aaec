// attention.hip — scaled dot-product attention for 16-bit operands as ONE
// kernel that never writes the S x S score tensor.
//
// It stands for the sequence kaun/lib/attention.ml:67-110 issues for f16 / bf16
// inputs, primitive by primitive:
//   scores = matmul (cast f32 q) (transpose (cast f32 k))      -- f32
//   scores = scores * scale                                     -- f32
//   scores = where mask scores masked_value                     -- f32
//   probs  = cast dtype (softmax scores)                        -- frontend.ml:4242-4252
//   out    = matmul probs v                                     -- dtype, f32 accumulation
// with the same rounding points: products of 16-bit values are exact in the
// f32 accumulator of v_mfma_f32_32x32x16, the scale is one f32 multiply, each
// probability is exp(t - rowmax) / rowsum rounded to the 16-bit dtype BEFORE it
// meets v, and the output is rounded once from the f32 accumulator. What
// differs from the op-by-op result: the order of the f32 sums (scores, row sum,
// probs x v); the row sum is accumulated tile by tile against a running maximum;
// the exponential is this file's six-instruction form (within 2 ulp, the
// primitive's within 1) and the quotient one Newton step on e x (1 / rowsum),
// which is the correctly rounded quotient in all but rare cases. Both sit far
// below the 16-bit rounding that follows them.
//
// Layout of the work (the two-wave kernel; the default for a positive scale and a -inf fill is
// its four-wave variant further down, which also splits every key tile between two waves): a
// block of two wave64s owns one 64-query tile of one
// (batch, head), each wave 32 queries; the grid hands out the late tiles of all
// heads first, which under a causal mask are the long ones (pairing tile t with
// tile T-1-t in one block balanced the blocks but left three waves per two SIMDs:
// 0.118 ms against 0.094 ms at [8,12,1024,64]). Keys are visited 64 at a time through
// LDS (K as [key][d], V as [key][d] too and read back with the transposing LDS
// load, so no operand is ever transposed in memory). The wave computes the
// TRANSPOSED score tile S^T = K Q^T, so that a lane holds 16 scores of ONE
// query (accumulator column = lane % 32): row maxima and sums are 16 in-lane
// steps plus one exchange with lane ^ 32. Pass 1 walks the keys for the row
// maximum and sum; pass 2 walks them again, forms the rounded probabilities in
// registers, exchanges halves with lane ^ 32 to lay them out as the B operand
// of O^T = V^T P^T, and accumulates the output. Recomputing Q K^T is cheap
// next to the 2 x S x S x 4 bytes it saves. With `causal` the mask is generated from
// indices and key tiles above the diagonal are skipped.

#include "fold_common.hpp"
#include "softmax_math.hpp"
#include "gemm_tile.hpp"
#include "map_ops.hpp"

namespace {

using gemm_tile::f32x16;
using gemm_tile::lds_s16x4;
using gemm_tile::s16x4;
using gemm_tile::V16;

constexpr int ATT_MAXB = 4;   // outer (batch) dims
constexpr int KEYS = 64;      // per LDS tile

struct AttOperand {
  const char *base;
  int64_t outer[ATT_MAXB];  // strides of the outer dims, elements
  int64_t row;              // stride of the sequence dim
};
struct AttArgs {
  AttOperand q, k, v, out, mask;
  int64_t mask_col;  // stride of the mask along keys
  int nouter;
  uint32_t oshape[ATT_MAXB];
  int64_t batches;
  int sq, sk, qtiles;
  int causal, has_mask, has_scale;
  float scale, masked;
  // one-pass form with a positive scale and a -inf fill: the scores stay unscaled and the scale
  // goes into the exponent, e^(scale (s - m)) = 2^(s c - m c) with c = scale log2(e)
  int raw;
  float c2;
};

template <class EL>
__device__ __forceinline__ uint16_t narrow(float x) {
  return EL::BF16 ? f32_to_bf16(x) : f32_to_f16(x);
}
template <class EL>
__device__ __forceinline__ uint32_t narrow2(float lo, float hi) {
  if constexpr (EL::BF16) return f32x2_to_bf16x2(lo, hi);
  else return (uint32_t)f32_to_f16(lo) | ((uint32_t)f32_to_f16(hi) << 16);
}

__device__ __forceinline__ float xor32(float v) {
  return __builtin_bit_cast(float, __shfl_xor(__builtin_bit_cast(int, v), 32, 64));
}

template <class EL, int DHEAD, bool ONLINE>
__global__ __launch_bounds__(128) void attention_kernel(AttArgs a) {
  using S = uint16_t;
  using MX = Combine<NXH_RMAX, float, CAT_FLOAT>;
  constexpr int KSTEPS = DHEAD / 16;  // k-steps of Q K^T
  constexpr int OT = DHEAD / 32;      // 32-row tiles of O^T
  constexpr int PK = DHEAD + 8;       // pitch of K in LDS ([key][d], read along d)
  constexpr int PV = DHEAD + 16;      // pitch of V in LDS ([key][d], read transposed)
  constexpr int VPR = DHEAD / 8;      // 16-byte vectors per row
  __shared__ __attribute__((aligned(16))) S Ks[KEYS * PK];
  __shared__ __attribute__((aligned(16))) S Vs[KEYS * PV];

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, c32 = lane & 31, g = lane >> 5;
  const int64_t bid = blockIdx.x;
  // Late query tiles first, those of every (batch, head) before any earlier tile:
  // under a causal mask they meet the most keys, and the short tiles fill the end.
  const int tile = a.qtiles - 1 - (int)(bid / a.batches);
  int64_t batch = bid % a.batches;
  int64_t qo = 0, ko = 0, vo = 0, oo = 0, mo = 0;
  for (int d = a.nouter - 1; d >= 0; d--) {
    const int64_t c = batch % a.oshape[d];
    batch /= a.oshape[d];
    qo += c * a.q.outer[d];
    ko += c * a.k.outer[d];
    vo += c * a.v.outer[d];
    oo += c * a.out.outer[d];
    mo += c * a.mask.outer[d];
  }
  const S *Q = reinterpret_cast<const S *>(a.q.base) + qo;
  const S *K = reinterpret_cast<const S *>(a.k.base) + ko;
  const S *V = reinterpret_cast<const S *>(a.v.base) + vo;
  S *O = reinterpret_cast<S *>(const_cast<char *>(a.out.base)) + oo;
  const uint8_t *M = reinterpret_cast<const uint8_t *>(a.mask.base) + mo;

  const int qw = tile * 64 + wave * 32;        // first query of the wave
  const int qi = qw + c32;                     // this lane's query
  const int qrow = qi < a.sq ? qi : a.sq - 1;  // clamp: rows past the end are never stored
  // Q fragments: B operand of S^T = K Q^T, this lane's 8 d-values per k-step
  V16 qf[KSTEPS];
#pragma unroll
  for (int s = 0; s < KSTEPS; s++)
    qf[s] = *reinterpret_cast<const V16 *>(Q + (int64_t)qrow * a.q.row + s * 16 + g * 8);

  // keys this block needs: all, or up to its last query under a causal mask
  const int qend = (tile + 1) * 64;  // one past the tile's last query
  const int klimit = a.causal ? (qend < a.sk ? qend : a.sk) : a.sk;
  const int ktiles = (klimit + KEYS - 1) / KEYS;

  float m_run = MX::init(), l_run = 0.0f;
  f32x16 oacc[OT];
#pragma unroll
  for (int t = 0; t < OT; t++)
#pragma unroll
    for (int e = 0; e < 16; e++) oacc[t][e] = 0.0f;

  // One 32-key sub-tile of scores for this wave: t[e] is the masked, scaled
  // score of key j0 + (e/4)*8 + g*4 + e%4 against query qi. `inner` sub-tiles
  // lie wholly inside the keys every query of the wave may see: no mask, no
  // bounds to test.
  auto scores = [&](int j0, float (&t)[16], bool inner) {
    f32x16 acc;
#pragma unroll
    for (int e = 0; e < 16; e++) acc[e] = 0.0f;
    const S *kr = Ks + (j0 % KEYS + c32) * PK + g * 8;
#pragma unroll
    for (int s = 0; s < KSTEPS; s++) {
      const V16 kf = *reinterpret_cast<const V16 *>(kr + s * 16);
      gemm_tile::mfma_step<EL>(acc, kf, qf[s]);
    }
    const bool scaled = a.has_scale && !(ONLINE && a.raw);
    if (inner) {
#pragma unroll
      for (int e = 0; e < 16; e++) t[e] = scaled ? acc[e] * a.scale : acc[e];
      return;
    }
#pragma unroll
    for (int e = 0; e < 16; e++) {
      const int j = j0 + (e >> 2) * 8 + g * 4 + (e & 3);
      float x = acc[e];
      if (scaled) x = x * a.scale;
      bool keep = true;
      if (a.causal) keep = j <= qi;
      else if (a.has_mask) keep = M[(int64_t)qrow * a.mask.row + (int64_t)(j < a.sk ? j : a.sk - 1) * a.mask_col] != 0;
      x = keep ? x : a.masked;
      t[e] = j < a.sk ? x : -__builtin_inff();  // keys past the end do not exist
    }
  };

  // Global -> registers for one key tile (K, and V when the tile is for pass
  // 1), issued a tile ahead so that the loads fly during the previous tile's
  // arithmetic; registers -> LDS between the two barriers.
  constexpr int NV = KEYS * VPR / 128;
  V16 kpre[NV], vpre[NV];
  // this lane's vectors inside a key tile, as element offsets from the tile's first row (a whole
  // tile then costs no address arithmetic per load: one uniform base per operand and tile)
  uint32_t koff[NV], voff[NV];
  const bool short_offsets = (int64_t)KEYS * a.k.row < ((int64_t)1 << 31) && (int64_t)KEYS * a.v.row < ((int64_t)1 << 31) &&
                             a.k.row >= 0 && a.v.row >= 0;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const int v = threadIdx.x + i * 128;
    const int r = v / VPR, c = (v % VPR) * 8;
    koff[i] = (uint32_t)(r * a.k.row + c);
    voff[i] = (uint32_t)(r * a.v.row + c);
  }
  auto prefetch = [&](int pass, int kt) {
    if (short_offsets && (kt + 1) * KEYS <= a.sk) {  // uniform: every key of the tile exists
      const S *kb = K + (int64_t)kt * KEYS * a.k.row, *vb = V + (int64_t)kt * KEYS * a.v.row;
#pragma unroll
      for (int i = 0; i < NV; i++) {
        kpre[i] = *reinterpret_cast<const V16 *>(kb + koff[i]);
        if (pass == 1) vpre[i] = *reinterpret_cast<const V16 *>(vb + voff[i]);
      }
      return;
    }
#pragma unroll
    for (int i = 0; i < NV; i++) {
      const int v = threadIdx.x + i * 128;
      const int r = v / VPR, c = (v % VPR) * 8;
      int key = kt * KEYS + r;
      key = key < a.sk ? key : a.sk - 1;
      kpre[i] = *reinterpret_cast<const V16 *>(K + (int64_t)key * a.k.row + c);
      if (pass == 1) vpre[i] = *reinterpret_cast<const V16 *>(V + (int64_t)key * a.v.row + c);
    }
  };
  prefetch(ONLINE ? 1 : 0, 0);
  for (int pass = ONLINE ? 1 : 0; pass < 2; pass++) {
    float l_total = 0.0f, l_recip = 0.0f;
    if (!ONLINE && pass == 1) {
      l_total = l_run + xor32(l_run);
      l_recip = 1.0f / l_total;
    }
    for (int kt = 0; kt < ktiles; kt++) {
      __syncthreads();  // the previous tile has been consumed
#pragma unroll
      for (int i = 0; i < NV; i++) {
        const int v = threadIdx.x + i * 128;
        const int r = v / VPR, c = (v % VPR) * 8;
        *reinterpret_cast<V16 *>(Ks + r * PK + c) = kpre[i];
        if (pass == 1) *reinterpret_cast<V16 *>(Vs + r * PV + c) = vpre[i];
      }
      __syncthreads();
      if (kt + 1 < ktiles) prefetch(pass, kt + 1);
      else if (pass == 0) prefetch(1, 0);
      // B operand of O^T = V^T P^T for k-step ks of sub-tile `sub`: this lane's query, keys
      // ks*16 + g*8 + 0..7. The accumulator gave keys ks*16 + g*4 + 0..3 and
      // ks*16 + 8 + g*4 + 0..3: swap one half with lane ^ 32. Then the products with V^T.
      auto times_v = [&](int sub, const uint32_t (&pk)[8]) {
#pragma unroll
        for (int ks = 0; ks < 2; ks++) {
          const uint32_t a0 = pk[ks * 4 + 0], a1 = pk[ks * 4 + 1];  // keys g*4 + 0..3
          const uint32_t b0 = pk[ks * 4 + 2], b1 = pk[ks * 4 + 3];  // keys 8 + g*4 + 0..3
          const uint32_t s0 = g == 0 ? b0 : a0, s1 = g == 0 ? b1 : a1;
          const uint32_t r0 = (uint32_t)__shfl_xor((int)s0, 32, 64), r1 = (uint32_t)__shfl_xor((int)s1, 32, 64);
          const V16 pf = g == 0 ? V16{a0, a1, r0, r1} : V16{r0, r1, b0, b1};
#pragma unroll
          for (int ot = 0; ot < OT; ot++) {
            // A operand: V^T rows d = ot*32 + lane%32, keys as above, by transposing LDS reads
            const int kk = sub * 32 + ks * 16 + g * 8 + ((lane & 15) >> 2);
            const int rr = ot * 32 + ((lane >> 4) & 1) * 16 + (lane & 3) * 4;
            const S *src = Vs + kk * PV + rr;
            const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)src);
            const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(src + 4 * PV));
            typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
            const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
            gemm_tile::mfma_step<EL>(oacc[ot], V16{l2[0], l2[1], h2[0], h2[1]}, pf);
          }
        }
      };
      if constexpr (ONLINE) {
        if (a.raw) {
          // Both 32-key sub-tiles of the tile in one step: one maximum, one decision about the
          // reference and 32 independent exponentials per lane instead of two dependent rounds
          // of 16. The first sub-tile is visible whenever the tile is visited (its first key is
          // at or before the wave's first query and inside the keys); the second may lie wholly
          // above the diagonal or past the last key: then only the first is worked on.
          const int j0 = kt * KEYS;
          const bool two = !(j0 + 32 >= a.sk || (a.causal && j0 + 32 > qw + 31));
          float t0[16], t1[16];
          scores(j0, t0, j0 + 32 <= a.sk && !a.has_mask && (!a.causal || j0 + 31 <= qw));
          if (two) {
            scores(j0 + 32, t1, j0 + 64 <= a.sk && !a.has_mask && (!a.causal || j0 + 63 <= qw));
          } else {
#pragma unroll
            for (int e = 0; e < 16; e++) t1[e] = -__builtin_inff();
          }
          float tm = t0[0];
#pragma unroll
          for (int e = 1; e < 16; e++) tm = __builtin_fmaxf(tm, t0[e]);
#pragma unroll
          for (int e = 0; e < 16; e++) tm = __builtin_fmaxf(tm, t1[e]);
          tm = __builtin_fmaxf(tm, xor32(tm));  // this query's maximum over the tile, both halves agree
          // The reference of the exponentials follows the maximum lazily: it moves only when a
          // tile's maximum lies more than 2^8 above it (or when it is the first thing the query
          // sees). In between the exponentials are taken against the older, smaller reference and
          // may reach 256: harmless in f32 and in the 16-bit rounding, which is relative, and the
          // row sum carries the same reference. Following every new maximum exactly rescaled the
          // 32 output accumulators of every lane in most steps (with 32 queries per wave one of
          // them often sees a new maximum). The exponential is the bare hardware 2^x of one fused
          // multiply-add: about 1e-6 relative, three orders below the 16-bit rounding that follows
          // (the six-instruction form is kept where the quotient is rounded instead).
          const bool first = m_run == -__builtin_inff();
          const bool grow = tm > m_run && (first || __builtin_fmaf(tm, a.c2, -m_run * a.c2) > 8.0f);
          const float m_new = grow ? tm : m_run;
          const float m_ref = m_new == -__builtin_inff() ? 0.0f : m_new;
          const float mc = -m_ref * a.c2;
          const float alpha = grow ? __builtin_amdgcn_exp2f(__builtin_fmaf(m_run, a.c2, mc)) : 1.0f;
          if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
            for (int ot = 0; ot < OT; ot++)
#pragma unroll
              for (int e = 0; e < 16; e++) oacc[ot][e] = oacc[ot][e] * alpha;
          }
          uint32_t pk0[8], pk1[8];
          float sum0 = 0.0f, sum1 = 0.0f;
#pragma unroll
          for (int e = 0; e < 16; e += 2) {
            const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(t0[e], a.c2, mc));
            const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(t0[e + 1], a.c2, mc));
            sum0 = sum0 + p0 + p1;
            pk0[e >> 1] = narrow2<EL>(p0, p1);
          }
          times_v(0, pk0);
          if (two) {
#pragma unroll
            for (int e = 0; e < 16; e += 2) {
              const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(t1[e], a.c2, mc));
              const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(t1[e + 1], a.c2, mc));
              sum1 = sum1 + p0 + p1;
              pk1[e >> 1] = narrow2<EL>(p0, p1);
            }
            times_v(1, pk1);
          }
          l_run = __builtin_fmaf(l_run, alpha, sum0 + sum1);
          m_run = m_new;
          continue;
        }
      }
#pragma unroll
      for (int sub = 0; sub < KEYS / 32; sub++) {
        const int j0 = kt * KEYS + sub * 32;
        // nothing of this sub-tile is visible to the wave's queries
        if (j0 >= a.sk || (a.causal && j0 > qw + 31)) continue;
        float t[16];
        scores(j0, t, j0 + 32 <= a.sk && !a.has_mask && (!a.causal || j0 + 31 <= qw));
        if (pass == 0) {
          // The hardware maximum skips NaNs; a NaN score reaches the row through the
          // sum of exponentials instead (every probability of the row is then NaN, as
          // after the primitive's NaN-keeping max), or through the scan below while
          // nothing of the row has been visible yet.
          float tm = t[0];
#pragma unroll
          for (int e = 1; e < 16; e++) tm = __builtin_fmaxf(tm, t[e]);
          float m_new = __builtin_fmaxf(m_run, tm);
          m_new = __builtin_fmaxf(m_new, xor32(m_new));  // both halves of a query agree on the maximum
          if (m_new != -__builtin_inff()) {
            float s = 0.0f;
#pragma unroll
            for (int e = 0; e < 16; e++) s = s + exp_nonpositive(t[e] - m_new);
            l_run = l_run * exp_nonpositive(m_run - m_new) + s;
          } else {
            bool nan = false;
#pragma unroll
            for (int e = 0; e < 16; e++) nan = nan || t[e] != t[e];
            if (nan) l_run = __builtin_nanf("");
          }
          m_run = m_new;
        } else {
          // rounded probabilities, two per register, in accumulator order
          uint32_t pk[8];
          if constexpr (ONLINE) {
            // One walk over the keys: the exponentials are taken against the maximum seen so
            // far, rounded, and multiplied into the output at once; when a later tile raises
            // the maximum, what has been accumulated (output and row sum, all of it this
            // lane's own query) is scaled down by e^(old - new). The division by the row sum
            // is left for the end.
            float tm = t[0];
#pragma unroll
            for (int e = 1; e < 16; e++) tm = __builtin_fmaxf(tm, t[e]);
            tm = __builtin_fmaxf(tm, xor32(tm));  // this query's maximum over the sub-tile, both halves agree
            // (the raw form took the merged step above; here the scores are scaled and masked)
            float sum = 0.0f;
            const float m_new = __builtin_fmaxf(m_run, tm);
            // nothing visible yet: exponentials of -inf against 0 are 0, not NaN
            const float m_ref = m_new == -__builtin_inff() ? 0.0f : m_new;
            const float alpha = exp_nonpositive(m_run - m_ref);
#pragma unroll
            for (int e = 0; e < 16; e += 2) {
              const float p0 = exp_nonpositive(t[e] - m_ref), p1 = exp_nonpositive(t[e + 1] - m_ref);
              sum = sum + p0 + p1;
              pk[e >> 1] = narrow2<EL>(p0, p1);
            }
            l_run = __builtin_fmaf(l_run, alpha, sum);
            if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
              for (int ot = 0; ot < OT; ot++)
#pragma unroll
                for (int e = 0; e < 16; e++) oacc[ot][e] = oacc[ot][e] * alpha;
            }
            m_run = m_new;
          } else {
#pragma unroll
            for (int e = 0; e < 16; e += 2) {
              const float p0 = div_by_reciprocal(exp_nonpositive(t[e] - m_run), l_total, l_recip);
              const float p1 = div_by_reciprocal(exp_nonpositive(t[e + 1] - m_run), l_total, l_recip);
              pk[e >> 1] = narrow2<EL>(p0, p1);
            }
          }
          times_v(sub, pk);
        }
      }
    }
  }
  if constexpr (ONLINE) {
    const float l_total = l_run + xor32(l_run);
#pragma unroll
    for (int ot = 0; ot < OT; ot++)
#pragma unroll
      for (int e = 0; e < 16; e++) oacc[ot][e] = oacc[ot][e] / l_total;
  }
  // O^T element e of tile ot: d = ot*32 + (e/4)*8 + g*4 + e%4, query qi
  if (qi < a.sq) {
    S *orow = O + (int64_t)qi * a.out.row;
#pragma unroll
    for (int ot = 0; ot < OT; ot++)
#pragma unroll
      for (int e = 0; e < 16; e += 4) {
        const int d = ot * 32 + (e >> 2) * 8 + g * 4;
        uint2 w;
        w.x = narrow2<EL>(oacc[ot][e], oacc[ot][e + 1]);
        w.y = narrow2<EL>(oacc[ot][e + 2], oacc[ot][e + 3]);
        *reinterpret_cast<uint2 *>(orow + d) = w;
      }
  }
}

// The one-pass form with the scale in the exponent (AttArgs::raw), four waves per 64-query
// tile instead of two. What bounds the two-wave kernel under a causal mask is not throughput but
// the chain of its longest tiles: a wave walks up to sixteen key tiles one after the other and
// each step is a string of dependent latencies (LDS tile, score MFMAs, maximum, exponentials,
// the exchange with lane ^ 32, the MFMAs with V); at batch 2 the kernel takes as long as at
// batch 8. Here waves 2p and 2p + 1 share the 32 queries of pair p and split every key tile
// between them, keys 0..31 and 32..63: half the scores, exponentials and V products per step
// and wave. Each wave keeps its own running reference, row sum and output; at the end the odd
// wave hands its three to the even one through LDS and they are merged against the larger
// reference, O = O_a 2^((m_a - m) c) + O_b 2^((m_b - m) c) and the same for the row sum, before
// the one division. Rounding points are those of the two-wave form; only the f32 sums of the
// output and of the row sum are added in another order.
// (Asking the compiler for four waves per SIMD at head dim 64, 128 registers instead of the 136
// it takes, changed nothing at batch 8 or 16: the kernel is bound by what it issues.)
template <class EL, int DHEAD>
__global__ __launch_bounds__(256) void attention_split_kernel(AttArgs a) {
  using S = uint16_t;
  constexpr int KSTEPS = DHEAD / 16, OT = DHEAD / 32, PK = DHEAD + 8, PV = DHEAD + 16, VPR = DHEAD / 8;
  __shared__ __attribute__((aligned(16))) S Ks[KEYS * PK];
  __shared__ __attribute__((aligned(16))) S Vs[KEYS * PV];
  __shared__ float mrg[2][OT * 16 + 2][64];

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, c32 = lane & 31, g = lane >> 5;
  const int qh = wave >> 1, kh = wave & 1;
  const int64_t bid = blockIdx.x;
  const int tile = a.qtiles - 1 - (int)(bid / a.batches);  // late (long) tiles first
  int64_t batch = bid % a.batches;
  int64_t qo = 0, ko = 0, vo = 0, oo = 0, mo = 0;
  for (int d = a.nouter - 1; d >= 0; d--) {
    const int64_t c = batch % a.oshape[d];
    batch /= a.oshape[d];
    qo += c * a.q.outer[d];
    ko += c * a.k.outer[d];
    vo += c * a.v.outer[d];
    oo += c * a.out.outer[d];
    mo += c * a.mask.outer[d];
  }
  const S *Q = reinterpret_cast<const S *>(a.q.base) + qo;
  const S *K = reinterpret_cast<const S *>(a.k.base) + ko;
  const S *V = reinterpret_cast<const S *>(a.v.base) + vo;
  S *O = reinterpret_cast<S *>(const_cast<char *>(a.out.base)) + oo;
  const uint8_t *M = reinterpret_cast<const uint8_t *>(a.mask.base) + mo;

  const int qw = tile * 64 + qh * 32;          // first query of the pair
  const int qi = qw + c32;                     // this lane's query
  const int qrow = qi < a.sq ? qi : a.sq - 1;  // clamp: rows past the end are never stored
  V16 qf[KSTEPS];
#pragma unroll
  for (int s = 0; s < KSTEPS; s++)
    qf[s] = *reinterpret_cast<const V16 *>(Q + (int64_t)qrow * a.q.row + s * 16 + g * 8);
  const int qend = (tile + 1) * 64;
  const int klimit = a.causal ? (qend < a.sk ? qend : a.sk) : a.sk;
  const int ktiles = (klimit + KEYS - 1) / KEYS;

  float m_run = -__builtin_inff(), l_run = 0.0f;
  f32x16 oacc[OT];
#pragma unroll
  for (int t = 0; t < OT; t++)
#pragma unroll
    for (int e = 0; e < 16; e++) oacc[t][e] = 0.0f;

  // t[e]: the unscaled score of key j0 + (e/4)*8 + g*4 + e%4 against query qi, -inf where masked
  auto scores = [&](int j0, float (&t)[16], bool inner) {
    f32x16 acc;
#pragma unroll
    for (int e = 0; e < 16; e++) acc[e] = 0.0f;
    const S *kr = Ks + (j0 % KEYS + c32) * PK + g * 8;
#pragma unroll
    for (int s = 0; s < KSTEPS; s++) {
      const V16 kf = *reinterpret_cast<const V16 *>(kr + s * 16);
      gemm_tile::mfma_step<EL>(acc, kf, qf[s]);
    }
    if (inner) {
#pragma unroll
      for (int e = 0; e < 16; e++) t[e] = acc[e];
      return;
    }
#pragma unroll
    for (int e = 0; e < 16; e++) {
      const int j = j0 + (e >> 2) * 8 + g * 4 + (e & 3);
      bool keep = true;
      if (a.causal) keep = j <= qi;
      else if (a.has_mask) keep = M[(int64_t)qrow * a.mask.row + (int64_t)(j < a.sk ? j : a.sk - 1) * a.mask_col] != 0;
      t[e] = keep && j < a.sk ? acc[e] : -__builtin_inff();  // (the fill of this form is -inf)
    }
  };

  constexpr int NV = KEYS * VPR / 256;
  static_assert(NV >= 1 && NV * 256 == KEYS * VPR, "whole vectors per lane");
  V16 kpre[NV], vpre[NV];
  // this lane's vectors inside a key tile as element offsets from the tile's first row: a whole
  // tile then costs one uniform base per operand and no address arithmetic per load
  uint32_t koff[NV], voff[NV];
  const bool short_offsets = (int64_t)KEYS * a.k.row < ((int64_t)1 << 31) && (int64_t)KEYS * a.v.row < ((int64_t)1 << 31) &&
                             a.k.row >= 0 && a.v.row >= 0;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const int v = threadIdx.x + i * 256;
    const int r = v / VPR, c = (v % VPR) * 8;
    koff[i] = (uint32_t)(r * a.k.row + c);
    voff[i] = (uint32_t)(r * a.v.row + c);
  }
  auto prefetch = [&](int kt) {
    if (short_offsets && (kt + 1) * KEYS <= a.sk) {  // uniform: every key of the tile exists
      const S *kb = K + (int64_t)kt * KEYS * a.k.row, *vb = V + (int64_t)kt * KEYS * a.v.row;
#pragma unroll
      for (int i = 0; i < NV; i++) {
        kpre[i] = *reinterpret_cast<const V16 *>(kb + koff[i]);
        vpre[i] = *reinterpret_cast<const V16 *>(vb + voff[i]);
      }
      return;
    }
#pragma unroll
    for (int i = 0; i < NV; i++) {
      const int v = threadIdx.x + i * 256;
      const int r = v / VPR, c = (v % VPR) * 8;
      int key = kt * KEYS + r;
      key = key < a.sk ? key : a.sk - 1;
      kpre[i] = *reinterpret_cast<const V16 *>(K + (int64_t)key * a.k.row + c);
      vpre[i] = *reinterpret_cast<const V16 *>(V + (int64_t)key * a.v.row + c);
    }
  };
  prefetch(0);
  for (int kt = 0; kt < ktiles; kt++) {
    __syncthreads();  // the previous tile has been consumed
#pragma unroll
    for (int i = 0; i < NV; i++) {
      const int v = threadIdx.x + i * 256;
      const int r = v / VPR, c = (v % VPR) * 8;
      *reinterpret_cast<V16 *>(Ks + r * PK + c) = kpre[i];
      *reinterpret_cast<V16 *>(Vs + r * PV + c) = vpre[i];
    }
    __syncthreads();
    if (kt + 1 < ktiles) prefetch(kt + 1);
    const int j0 = kt * KEYS + kh * 32;
    // nothing of this wave's half of the tile is visible to its queries
    if (j0 >= a.sk || (a.causal && j0 > qw + 31)) continue;
    float t[16];
    scores(j0, t, j0 + 32 <= a.sk && !a.has_mask && (!a.causal || j0 + 31 <= qw));
    float tm = t[0];
#pragma unroll
    for (int e = 1; e < 16; e++) tm = __builtin_fmaxf(tm, t[e]);
    tm = __builtin_fmaxf(tm, xor32(tm));  // this query's maximum over the half tile, both lane halves agree
    // the reference follows the maximum lazily, as in the two-wave kernel
    const bool first = m_run == -__builtin_inff();
    const bool grow = tm > m_run && (first || __builtin_fmaf(tm, a.c2, -m_run * a.c2) > 8.0f);
    const float m_new = grow ? tm : m_run;
    const float m_ref = m_new == -__builtin_inff() ? 0.0f : m_new;
    const float mc = -m_ref * a.c2;
    const float alpha = grow ? __builtin_amdgcn_exp2f(__builtin_fmaf(m_run, a.c2, mc)) : 1.0f;
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
      for (int ot = 0; ot < OT; ot++)
#pragma unroll
        for (int e = 0; e < 16; e++) oacc[ot][e] = oacc[ot][e] * alpha;
    }
    uint32_t pk[8];
    float sum = 0.0f;
#pragma unroll
    for (int e = 0; e < 16; e += 2) {
      const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(t[e], a.c2, mc));
      const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(t[e + 1], a.c2, mc));
      sum = sum + p0 + p1;
      pk[e >> 1] = narrow2<EL>(p0, p1);
    }
    // O^T += V^T P^T for this wave's 32 keys (the B operand wants keys g*8 + 0..7 per k-step: the
    // accumulator gave g*4 + 0..3 and 8 + g*4 + 0..3, so one half is swapped with lane ^ 32)
#pragma unroll
    for (int ks = 0; ks < 2; ks++) {
      const uint32_t a0 = pk[ks * 4 + 0], a1 = pk[ks * 4 + 1];
      const uint32_t b0 = pk[ks * 4 + 2], b1 = pk[ks * 4 + 3];
      const uint32_t s0 = g == 0 ? b0 : a0, s1 = g == 0 ? b1 : a1;
      const uint32_t r0 = (uint32_t)__shfl_xor((int)s0, 32, 64), r1 = (uint32_t)__shfl_xor((int)s1, 32, 64);
      const V16 pf = g == 0 ? V16{a0, a1, r0, r1} : V16{r0, r1, b0, b1};
#pragma unroll
      for (int ot = 0; ot < OT; ot++) {
        const int kk = kh * 32 + ks * 16 + g * 8 + ((lane & 15) >> 2);
        const int rr = ot * 32 + ((lane >> 4) & 1) * 16 + (lane & 3) * 4;
        const S *src = Vs + kk * PV + rr;
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)src);
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(src + 4 * PV));
        typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
        const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
        gemm_tile::mfma_step<EL>(oacc[ot], V16{l2[0], l2[1], h2[0], h2[1]}, pf);
      }
    }
    l_run = __builtin_fmaf(l_run, alpha, sum);
    m_run = m_new;
  }
  // the odd wave of a pair hands over, the even one merges, divides and stores
  if (kh == 1) {
#pragma unroll
    for (int ot = 0; ot < OT; ot++)
#pragma unroll
      for (int e = 0; e < 16; e++) mrg[qh][ot * 16 + e][lane] = oacc[ot][e];
    mrg[qh][OT * 16][lane] = m_run;
    mrg[qh][OT * 16 + 1][lane] = l_run;
  }
  __syncthreads();
  if (kh == 1) return;
  {
    const float m_b = mrg[qh][OT * 16][lane], l_b = mrg[qh][OT * 16 + 1][lane];
    const float m = __builtin_fmaxf(m_run, m_b);
    const float m_ref = m == -__builtin_inff() ? 0.0f : m;
    // (a wave that saw nothing has reference -inf, sum 0 and output 0: its factor is 2^-inf = 0)
    const float s_a = __builtin_amdgcn_exp2f((m_run - m_ref) * a.c2), s_b = __builtin_amdgcn_exp2f((m_b - m_ref) * a.c2);
    l_run = l_run * s_a + l_b * s_b;
#pragma unroll
    for (int ot = 0; ot < OT; ot++)
#pragma unroll
      for (int e = 0; e < 16; e++) oacc[ot][e] = oacc[ot][e] * s_a + mrg[qh][ot * 16 + e][lane] * s_b;
  }
  const float l_total = l_run + xor32(l_run);
#pragma unroll
  for (int ot = 0; ot < OT; ot++)
#pragma unroll
    for (int e = 0; e < 16; e++) oacc[ot][e] = oacc[ot][e] / l_total;
  if (qi < a.sq) {
    S *orow = O + (int64_t)qi * a.out.row;
#pragma unroll
    for (int ot = 0; ot < OT; ot++)
#pragma unroll
      for (int e = 0; e < 16; e += 4) {
        const int d = ot * 32 + (e >> 2) * 8 + g * 4;
        uint2 w;
        w.x = narrow2<EL>(oacc[ot][e], oacc[ot][e + 1]);
        w.y = narrow2<EL>(oacc[ot][e + 2], oacc[ot][e + 3]);
        *reinterpret_cast<uint2 *>(orow + d) = w;
      }
  }
}

// NXH_ATTENTION=twopass selects the form that rounds each probability after the division by
// the full row sum, as the primitive sequence does; the default walks the keys once.
bool two_pass_wanted() {
  const char *e = getenv("NXH_ATTENTION");  // read per call: a test switches it inside one process
  return e && strcmp(e, "twopass") == 0;
}

template <class EL, bool ONLINE>
int attention_launch(nxh_context *ctx, const char *op, const AttArgs &a, int hd) {
  const int64_t blocks = a.batches * a.qtiles;
  if (blocks > 0x7fffffffLL) return nxh_fail(NXH_FAILURE, op, "too many elements for one launch");
  const dim3 grid((unsigned)blocks), block(128);
  if constexpr (ONLINE) {
    if (a.raw) {  // the four-wave form ([b,12,1024,64] causal, b = 1 / 2 / 4 / 8 / 16: 19.9 / 20.9 / 23.4 / 37.3 / 74.0 us
                  // against 29.2 / 30.4 / 32.4 / 42.5 / 80.8 us with two waves per tile)
      switch (hd) {
        case 32: hipLaunchKernelGGL((attention_split_kernel<EL, 32>), grid, dim3(256), 0, ctx->stream, a); break;
        case 64: hipLaunchKernelGGL((attention_split_kernel<EL, 64>), grid, dim3(256), 0, ctx->stream, a); break;
        case 128: hipLaunchKernelGGL((attention_split_kernel<EL, 128>), grid, dim3(256), 0, ctx->stream, a); break;
        default: return nxh_fail(NXH_FAILURE, op, "head dimension must be 32, 64 or 128");
      }
      return NXH_OK;
    }
  }
  switch (hd) {
    case 32: hipLaunchKernelGGL((attention_kernel<EL, 32, ONLINE>), grid, block, 0, ctx->stream, a); break;
    case 64: hipLaunchKernelGGL((attention_kernel<EL, 64, ONLINE>), grid, block, 0, ctx->stream, a); break;
    case 128: hipLaunchKernelGGL((attention_kernel<EL, 128, ONLINE>), grid, block, 0, ctx->stream, a); break;
    default: return nxh_fail(NXH_FAILURE, op, "head dimension must be 32, 64 or 128");
  }
  return NXH_OK;
}

// Rows of `t` must be contiguous and 16-byte aligned (8-byte for the output).
bool rows_aligned(const nxh_tensor *t, int bytes) {
  const int nd = t->ndim;
  if (t->shape[nd - 1] > 1 && t->strides[nd - 1] != 1) return false;
  if ((((uintptr_t)t->data + t->offset * 2) % (uintptr_t)bytes) != 0) return false;
  for (int d = 0; d < nd - 1; d++)
    if (t->shape[d] > 1 && (t->strides[d] * 2) % bytes != 0) return false;
  return true;
}

}  // namespace

NXH_EXPORT int nxh_attention(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *q, const nxh_tensor *k,
                             const nxh_tensor *v, const void *scale, const nxh_tensor *mask,
                             const void *masked_value, int causal) {
  NXH_DEFER_TOUCH(ctx, 1, out, q, k, v, mask);
  const char *op = "attention";
  if (!ctx || !out || !q || !k || !v || (mask && !masked_value) || (causal && !masked_value))
    return nxh_fail(NXH_INVALID_ARGUMENT, op, "null argument");
  if (causal && mask) return nxh_fail(NXH_INVALID_ARGUMENT, op, "give either a mask or causal, not both");
  int rc = NXH_OK;
  for (const nxh_tensor *t : {out, q, k, v, mask})
    if (t && !rc) rc = nxh_check_tensor(op, t);
  if (rc) return rc;
  const int dt = q->dtype, nd = q->ndim;
  if ((dt != NXH_BF16 && dt != NXH_F16) || k->dtype != dt || v->dtype != dt || out->dtype != dt ||
      (mask && mask->dtype != NXH_BOOL))
    return nxh_fail(NXH_FAILURE, op, NXH_ERR_UNSUPPORTED);
  if (nd < 2 || k->ndim != nd || v->ndim != nd || out->ndim != nd || (mask && mask->ndim != nd))
    return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
  if (nd - 2 > ATT_MAXB) return nxh_fail(NXH_FAILURE, op, "more than 4 batch dimensions");
  AttArgs a;
  const int64_t sq = q->shape[nd - 2], sk = k->shape[nd - 2], hd = q->shape[nd - 1];
  if (k->shape[nd - 1] != hd || v->shape[nd - 1] != hd || v->shape[nd - 2] != sk || out->shape[nd - 2] != sq ||
      out->shape[nd - 1] != hd || (mask && (mask->shape[nd - 2] != sq || mask->shape[nd - 1] != sk)))
    return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
  a.batches = 1;
  a.nouter = nd - 2;
  for (int d = 0; d < nd - 2; d++) {
    const int64_t e = q->shape[d];
    if (k->shape[d] != e || v->shape[d] != e || out->shape[d] != e || (mask && mask->shape[d] != e))
      return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
    if (e > 0xffffffffLL) return nxh_fail(NXH_FAILURE, op, "extent exceeds 32 bits");
    a.oshape[d] = (uint32_t)e;
    a.batches *= e;
  }
  if (causal && sq != sk) return nxh_fail(NXH_INVALID_ARGUMENT, op, "causal needs as many queries as keys");
  // The causal form skips the key tiles above the diagonal, which equals the
  // `where mask scores masked_value` of the sequence only when the masked scores
  // vanish from the softmax, i.e. for -inf (what attention.ml fills in). Any other
  // fill gives the hidden keys a weight: the caller passes the mask tensor then.
  if (causal && !(*(const float *)masked_value == -__builtin_inff()))
    return nxh_fail(NXH_FAILURE, op, "the causal form needs masked_value = -inf; pass the mask tensor for any other fill");
  if (a.batches == 0 || sq == 0) return NXH_OK;
  if (sk == 0) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_EMPTY_REDUCE);
  if (sq > 0x3fffffff || sk > 0x3fffffff) return nxh_fail(NXH_FAILURE, op, "sequence longer than 2^30");
  for (int d = 0; d < nd; d++)
    if (out->shape[d] > 1 && out->strides[d] == 0) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_OUT_ALIASED);
  if (!rows_aligned(q, 16) || !rows_aligned(k, 16) || !rows_aligned(v, 16) || !rows_aligned(out, 8))
    return nxh_fail(NXH_FAILURE, op, "rows must be contiguous and 16-byte aligned");
  auto operand = [&](const nxh_tensor *t, AttOperand &o, int es) {
    o.base = t ? (const char *)t->data + t->offset * es : nullptr;
    for (int d = 0; d < ATT_MAXB; d++) o.outer[d] = (t && d < nd - 2) ? t->strides[d] : 0;
    o.row = t ? t->strides[nd - 2] : 0;
  };
  operand(q, a.q, 2);
  operand(k, a.k, 2);
  operand(v, a.v, 2);
  operand(out, a.out, 2);
  operand(mask, a.mask, 1);
  a.mask_col = mask ? mask->strides[nd - 1] : 0;
  a.sq = (int)sq;
  a.sk = (int)sk;
  a.qtiles = (int)((sq + 63) / 64);
  a.causal = causal ? 1 : 0;
  a.has_mask = mask ? 1 : 0;
  a.has_scale = scale ? 1 : 0;
  a.scale = scale ? *(const float *)scale : 1.0f;
  a.masked = masked_value ? *(const float *)masked_value : 0.0f;
  a.raw = a.scale > 0.0f && a.scale < __builtin_inff() && (!(mask || causal) || a.masked == -__builtin_inff());
  a.c2 = a.scale * 0x1.715476p+0f;
  std::lock_guard<std::mutex> guard(ctx->mu);
  NXH_HIP(op, hipSetDevice(ctx->device));
  nxh_set_path("attention_fused");
  if (two_pass_wanted())
    rc = dt == NXH_BF16 ? attention_launch<gemm_tile::ElBF16, false>(ctx, op, a, (int)hd)
                        : attention_launch<gemm_tile::ElF16, false>(ctx, op, a, (int)hd);
  else
    rc = dt == NXH_BF16 ? attention_launch<gemm_tile::ElBF16, true>(ctx, op, a, (int)hd)
                        : attention_launch<gemm_tile::ElF16, true>(ctx, op, a, (int)hd);
  if (rc) return rc;
  NXH_HIP(op, hipGetLastError());
  return NXH_OK;
}
