// gemm_dl.hpp — the 16-bit tiled GEMM with operands fetched from global memory straight
// into LDS, v_mfma_f32_16x16x32, eight waves per block. Two block shapes:
//   256 x 256  2 x 4 waves of 128 x 64   large products
//   128 x 192  2 x 4 waves of  64 x 48   products of a few hundred 128-row tiles: with
//                                        N = 768 (GPT-2's linears) [8192, 768] is exactly
//                                        256 blocks, one per compute unit, and N = 2304 or
//                                        3072 whole multiples of that
// Same contract as gemm_tile.hpp (f32 accumulation, one rounding per output element,
// batched with broadcastable batch dims, the fused linear's epilogue and grouped launch),
// for whole tiles only: M and N multiples of the block, K a multiple of 64 (the host runs a
// ragged last column block as a launch of its own). What differs
// from gemm_tile:
//   * No register staging. A slab (64 k-values of every row of both operands) is
//     requested with global_load_lds_dwordx4: each of the 64 lanes of a load delivers
//     16 bytes to consecutive LDS addresses, so the staging registers and every
//     ds_write of the staged form disappear. LDS holds a ring of two slabs; the loads
//     of slab t + 2 are issued as soon as every wave has read its last fragments of
//     slab t, behind the block's one barrier per slab.
//   * No padding. A load writes 1 KiB without gaps, so bank conflicts are avoided by
//     choosing WHICH 16 bytes each lane fetches: the 16-byte units of a k-contiguous
//     row are XOR-ed with bits of the row number, those of a row-contiguous k-row with
//     bits of k. Fragment reads apply the same XOR and touch every bank once per
//     half-wave (ds_read_b128 for k-contiguous tiles, ds_read_b64_tr_b16 otherwise).
//   * The wide side of a wave's outputs is A, whose k-contiguous fragments come with
//     ds_read_b128 (about 180 B/clk/CU measured), the narrow side B, whose
//     row-contiguous tile needs the slower transposing read (about 111 B/clk).
//   * v_mfma_f32_16x16x32 instead of 32x32x16: the same LDS bytes and MFMA cycles per
//     flop, but a quarter of the accumulator registers rewritten per instruction.
//     Under the board's power limit (random N(0, 0.02) operands pull this chip from
//     2.4 to about 1.8 GHz inside a GEMM) that is worth 4-7 % of throughput; on
//     all-zero operands, where the clock holds, the two forms time the same.
// The loads are written as assembly on purpose: the compiler then sees no LDS
// writes, so it places no vmcnt(0) in front of the fragment reads (it cannot tell
// the two slabs of the ring apart) and the waits are the explicit ones below.
#pragma once

#include "gemm_tile.hpp"

namespace gemm_dl {
using namespace gemm_tile;

constexpr int BK = 64;
constexpr int UPR = BK / 8;  // 16-byte units per row of a k-contiguous tile

// NS: slabs in the LDS ring. Two leave room for a second 128 x 192 block on the compute unit
// (2 x 80 KiB), which is what hides a block's barriers and epilogue when a launch is several
// rounds of blocks; a launch of at most one block per compute unit takes a deeper ring
// instead: its operands come from memory, not from L2, and one slab of lookahead (about
// 0.8 us) does not cover that latency. The order of additions does not depend on NS.
template <int BM_, int BN_, int NS_>
struct Shape {
  static constexpr int BM = BM_, BN = BN_, NS = NS_, WVM = 2, WVN = 4, WAVES = WVM * WVN, THREADS = 64 * WAVES;
  static constexpr int WM = BM / WVM, WN = BN / WVN;   // a wave's outputs
  static constexpr int FA = WM / 16, FB = WN / 16;     // 16-row fragments of A, 16-column fragments of B per wave
  static constexpr int LA = BM / 8 / WAVES, LB = BN / 8 / WAVES, LPW = LA + LB;  // load instructions per wave and slab
  static_assert(LA * 8 * WAVES == BM && LB * 8 * WAVES == BN && FA * 16 * WVM == BM && FB * 16 * WVN == BN, "shape");
  static constexpr int A_BYTES = BM * BK * 2, STAGE_BYTES = (BM + BN) * BK * 2;
  static constexpr int PATCH_PITCH = WN + 8;           // epilogue: a wave's WM x WN patch, padded rows (elements)
  static constexpr size_t PATCH_BYTES = (size_t)WAVES * WM * PATCH_PITCH * 2;
  static constexpr size_t LDS_BYTES = PATCH_BYTES > (size_t)NS * STAGE_BYTES ? PATCH_BYTES : (size_t)NS * STAGE_BYTES;
};
using Shape256x256 = Shape<256, 256, 2>;
using Shape128x192 = Shape<128, 192, 2>;
using Shape128x192Deep = Shape<128, 192, 4>;
static_assert(Shape128x192Deep::LDS_BYTES <= 160 * 1024 && Shape256x256::LDS_BYTES <= 160 * 1024, "LDS");

template <int N>
__device__ __forceinline__ void wait_loads_and_meet() {
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(N) : "memory");
}

// LDS position (16-byte unit) <-> which data it holds.
// k-contiguous tile [row][unit kv]: physical unit = kv ^ ((row >> 1) & 7): sixteen consecutive
// rows reading the same logical unit cover the sixteen 16-byte bank groups once.
// row-contiguous tile [k][UPK units nv]: physical unit = nv ^ swz_rc(k). A half-wave's
// transposing read touches two neighbouring units in each of the eight k-rows
// {0..3, 8..11} (+ 4, + 16): the XOR must send those to eight different 32-byte bank pairs.
// With a pitch of 256 or 512 bytes every k-row starts at bank 0 and three bits are needed;
// with 384 bytes (192 columns) odd k-rows already sit 128 bytes further on and two bits,
// which stay inside the row's groups of eight units, are enough.
__device__ __forceinline__ int swz_kc(int row) { return (row >> 1) & 7; }
template <int UPK>
__device__ __forceinline__ int swz_rc(int k) {
  if constexpr (UPK % 16 == 0) return ((k & 3) << 2) | (((k >> 3) & 1) << 1);
  else return (((k >> 1) & 1) | (((k >> 3) & 1) << 1)) << 1;
}

template <class EL, bool A_KC, bool B_KC, class SH, bool EPI>
__global__ __launch_bounds__(SH::THREADS) void kernel(Args a) {
  using S = typename EL::S;
  static_assert(!EL::F32, "16-bit operands only");
  constexpr int BM = SH::BM, BN = SH::BN, NS = SH::NS, FA = SH::FA, FB = SH::FB, LA = SH::LA, LB = SH::LB, LPW = SH::LPW;
  constexpr int STAGE_BYTES = SH::STAGE_BYTES, A_BYTES = SH::A_BYTES;
  constexpr int UPK_A = BM / 8, UPK_B = BN / 8;  // units per k-row of a row-contiguous tile
  static_assert(UPK_A % 8 == 0 && UPK_B % 8 == 0, "swizzle groups");
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  uint32_t batch, tm, tn;
  tile_of_block(a, gridDim.x - 1 - blockIdx.x, batch, tm, tn);
  int64_t ao = 0, bo = 0, co = 0, ro = 0;
  if constexpr (EPI) {
    if (a.ngroup > 1) {
      const uint32_t member = tn / a.gtn;
      tn -= member * a.gtn;
      if (member) {
        bo = member == 1 ? a.goff_b[0] : a.goff_b[1];
        co = member == 1 ? a.goff_c[0] : a.goff_c[1];
        if (a.bias) a.bias = (const S *)a.bias + (member == 1 ? a.goff_bias[0] : a.goff_bias[1]);
      }
    }
  }
  {
    uint32_t idx = batch;
#pragma unroll
    for (int i = 3; i >= 0; i--) {
      if (i < a.nbd) {
        uint32_t q = idx / a.bshape[i], c = idx - q * a.bshape[i];
        idx = q;
        ao += (int64_t)c * a.ba[i];
        bo += (int64_t)c * a.bb[i];
        co += (int64_t)c * a.bc[i];
        if constexpr (EPI) ro += (int64_t)c * a.br[i];
      }
    }
  }
  const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;
  const S *gA = (const S *)a.A + ao + (A_KC ? m0 * a.lda : m0);
  const S *gB = (const S *)a.B + bo + (B_KC ? n0 * a.ldb : n0);
  const int64_t stepA = A_KC ? BK : (int64_t)BK * a.lda;
  const int64_t stepB = B_KC ? BK : (int64_t)BK * a.ldb;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = (wave / SH::WVN) * SH::WM, wn = (wave % SH::WVN) * SH::WN;

  // Byte offset, from the slab's origin in global memory, of the 16 bytes this lane
  // fetches with load j of an operand: that load fills units [64 j, 64 j + 64) of its tile.
  auto off_kc = [&](int j, int64_t ld) -> uint32_t {
    const int row = j * (64 / UPR) + lane / UPR, kp = lane % UPR;
    return (uint32_t)((row * ld + (kp ^ swz_kc(row)) * 8) * 2);
  };
  auto off_rc = [&](int j, int64_t ld, auto upk_c) -> uint32_t {
    constexpr int UPK = decltype(upk_c)::value;
    const int u = j * 64 + lane, k = u / UPK, p = u % UPK;
    return (uint32_t)((k * ld + (p ^ swz_rc<UPK>(k)) * 8) * 2);
  };
  using upk_a = std::integral_constant<int, UPK_A>;
  using upk_b = std::integral_constant<int, UPK_B>;
  uint32_t offA[LA], offB[LB];
#pragma unroll
  for (int i = 0; i < LA; i++) offA[i] = A_KC ? off_kc(wave * LA + i, a.lda) : off_rc(wave * LA + i, a.lda, upk_a{});
#pragma unroll
  for (int i = 0; i < LB; i++) offB[i] = B_KC ? off_kc(wave * LB + i, a.ldb) : off_rc(wave * LB + i, a.ldb, upk_b{});
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)smem_raw;
  // m0 carries the LDS address of lane 0's 16 bytes. It is not declared as clobbered: the
  // compiler treats it as reserved and writes it itself right in front of each of its own uses.
  auto load1 = [&](const S *base, uint32_t off_bytes, uint32_t lds) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds), "v"(off_bytes), "s"(base)
                 : "memory");
  };
  auto issue = [&](int t, int buf) {
    const uint32_t sb = lds0 + buf * STAGE_BYTES;
    const S *pa = gA + (int64_t)t * stepA, *pb = gB + (int64_t)t * stepB;
#pragma unroll
    for (int i = 0; i < LA; i++) load1(pa, offA[i], sb + (wave * LA + i) * 1024);
#pragma unroll
    for (int i = 0; i < LB; i++) load1(pb, offB[i], sb + A_BYTES + (wave * LB + i) * 1024);
  };

  // Fragments of v_mfma_f32_16x16x32: lane 16 g + q holds row (column) q and k = 8 g .. 8 g + 7 of the 32.
  const int q16 = lane & 15, g16 = lane >> 4;
  const int kc_sw = (lane >> 1) & 7;  // swz_kc(row0 + q16): row0 is a multiple of 16
  const int kc_row = q16 * (UPR * 16);
  const int rc_k = g16 * 8 + (q16 >> 2);
  auto frag = [&](const unsigned char *tile, bool kcont, auto upk_c, int row0, int k32) -> V16 {
    constexpr int UPK = decltype(upk_c)::value;
    if (kcont) return *reinterpret_cast<const V16 *>(tile + row0 * (UPR * 16) + kc_row + (((k32 * 4 + g16) ^ kc_sw) << 4));
    // transposing read (gemm_tile.hpp): lane q of a 16-lane group addresses the 8 bytes at
    // k-row (q >> 2), rows 4 (q & 3) .. + 3; the second read takes the k-rows four further on
    // (the XOR leaves out bit 2 of k and everything above bit 3: the same for both reads)
    const int rc_sw = swz_rc<UPK>(rc_k);
    const int r = row0 + (q16 & 3) * 4;
    const unsigned char *p = tile + (k32 * 32 + rc_k) * (UPK * 16) + (((r >> 3) ^ rc_sw) << 4) + (r & 7) * 2;
    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)p);
    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(p + 4 * (UPK * 16)));
    typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
    const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
    return V16{l2[0], l2[1], h2[0], h2[1]};
  };

  f32x4 acc[FA][FB];
#pragma unroll
  for (int i = 0; i < FA; i++)
#pragma unroll
    for (int j = 0; j < FB; j++)
#pragma unroll
      for (int e = 0; e < 4; e++) acc[i][j][e] = 0.0f;

  const int nt = (int)(a.K / BK);
#pragma unroll
  for (int s = 0; s < NS; s++)
    if (s < nt) issue(s, s);
  if (nt >= NS) wait_loads_and_meet<(NS - 1) * LPW>();
  else wait_loads_and_meet<0>();

  // A step is FA x FB MFMAs: the wave's 16-row fragments of A against its 16-column fragments
  // of B over 32 k-values; a slab is two steps. The reads of step s + 1 are issued among the
  // MFMAs of step s, one behind each MFMA (scheduling groups below): a wave then never queues
  // all its LDS reads in one burst in front of a cold MFMA pipe, which is worth 3-5 % here.
  V16 fa[2][FA], fb[2][FB];
  auto load_step = [&](int buf, int k32) {
    const unsigned char *sa = smem_raw + buf * STAGE_BYTES, *sb = sa + A_BYTES;
#pragma unroll
    for (int i = 0; i < FA; i++) fa[k32][i] = frag(sa, A_KC, upk_a{}, wm + i * 16, k32);
#pragma unroll
    for (int j = 0; j < FB; j++) fb[k32][j] = frag(sb, B_KC, upk_b{}, wn + j * 16, k32);
  };
  load_step(0, 0);
  int buf = 0;
  // In a slab's last step: wait for this wave's share of the next slab, meet the other waves
  // (now the next slab is complete and nobody reads this one any more), request slab t + NS
  // into this slab's buffer, fetch the next slab's first fragments among the last MFMAs.
  auto slab = [&](int t, auto fetch_c, auto last_c) {
    constexpr bool FETCH = decltype(fetch_c)::value, LAST = decltype(last_c)::value;
    const int nbuf = buf + 1 == NS ? 0 : buf + 1;
#pragma unroll
    for (int k32 = 0; k32 < 2; k32++) {
      if (k32 == 0) {
        load_step(buf, 1);
      } else if constexpr (!LAST) {
        if constexpr (FETCH) wait_loads_and_meet<(NS - 2) * LPW>();
        else wait_loads_and_meet<0>();
        if constexpr (FETCH) issue(t + NS, buf);
        load_step(nbuf, 0);
      }
#pragma unroll
      for (int i = 0; i < FA; i++)
#pragma unroll
        for (int j = 0; j < FB; j++) {
          f32x4 &c = acc[i][j];
          if constexpr (EL::BF16)
            c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, fa[k32][i]), __builtin_bit_cast(bf16x8, fb[k32][j]), c, 0, 0, 0);
          else
            c = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, fa[k32][i]), __builtin_bit_cast(f16x8, fb[k32][j]), c, 0, 0, 0);
        }
#pragma unroll
      for (int x = 0; x < FA * FB; x++) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // one LDS read
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    buf = nbuf;
  };
  using yes = std::integral_constant<bool, true>;
  using no = std::integral_constant<bool, false>;
  int t = 0;
  for (; t + NS < nt; t++) slab(t, yes{}, no{});
  for (; t + 1 < nt; t++) slab(t, no{}, no{});
  slab(t, no{}, yes{});

  // Epilogue: element e of accumulator (i, j) is C[16 i + 4 g + e][16 j + q]. Each wave parks its
  // rounded WM x WN patch in LDS and sends it out as whole 16-byte row segments; the fused
  // linear's bias, residual and GELU are applied to those segments on the way
  // (gemm_tile.hpp: each step rounded to the dtype).
  S *C = (S *)a.C + co;
  auto narrow = [](float x) -> S { return EL::BF16 ? f32_to_bf16(x) : f32_to_f16(x); };
  // The GELU table (bfloat16, when the host passes one and the idle stage memory behind the
  // patches holds it): each lane requests at most one 16-byte piece now, and the pieces are
  // put into LDS behind the barrier, while the patches are written.
  constexpr bool LUT_ROOM = EPI && EL::BF16 && SH::PATCH_BYTES + 8192 <= SH::LDS_BYTES;
  const bool use_lut = LUT_ROOM && a.gelu && a.gelu_lut != nullptr;
  uint16_t *lut = reinterpret_cast<uint16_t *>(smem_raw + SH::PATCH_BYTES);
  V16 lut_piece = {0, 0, 0, 0};
  const bool lut_mine = use_lut && threadIdx.x < a.lut_n * 2 / 8;
  if constexpr (LUT_ROOM)
    if (lut_mine) lut_piece = reinterpret_cast<const V16 *>(a.gelu_lut)[threadIdx.x];
  // The epilogue's first bias and residual pieces are requested here already: their trip to
  // memory then runs under the barrier and the patch writes instead of behind them. (The slab
  // loads have all been waited for by now, so the barrier below need not wait for memory.)
  constexpr int CPR = SH::WN / 8;             // 16-byte pieces per patch row
  constexpr int NIT = SH::WM * CPR / 64;      // pieces per lane
  static_assert(NIT * 64 == SH::WM * CPR, "whole passes");
  constexpr int G = NIT <= 8 ? NIT : 4;       // pieces in flight per lane
  static_assert(NIT % G == 0, "whole groups");
  const S *btile = nullptr, *rtile = nullptr;
  V16 bq0[G], rq0[G];
  if constexpr (EPI) {
    btile = a.bias ? (const S *)a.bias + n0 + wn : nullptr;
    rtile = a.R ? (const S *)a.R + ro + (m0 + wm) * a.ldr + n0 + wn : nullptr;
#pragma unroll
    for (int i = 0; i < G; i++) {
      const int ch = i * 64 + lane, row = ch / CPR, col = (ch % CPR) * 8;
      if (btile) bq0[i] = *reinterpret_cast<const V16 *>(btile + col);
      if (rtile) rq0[i] = *reinterpret_cast<const V16 *>(rtile + (int64_t)row * a.ldr + col);
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");  // every wave has read its last fragments
  } else {
    wait_loads_and_meet<0>();  // every wave has read its last fragments; no load is in flight
  }
  constexpr int PITCH = SH::PATCH_PITCH;
  S *patch = reinterpret_cast<S *>(smem_raw) + wave * (SH::WM * PITCH);
#pragma unroll
  for (int i = 0; i < FA; i++)
#pragma unroll
    for (int j = 0; j < FB; j++)
#pragma unroll
      for (int e = 0; e < 4; e++) patch[(i * 16 + g16 * 4 + e) * PITCH + j * 16 + q16] = narrow(acc[i][j][e]);
  if constexpr (LUT_ROOM) {
    if (use_lut) {  // (uniform over the block)
      if (lut_mine) reinterpret_cast<V16 *>(lut)[threadIdx.x] = lut_piece;
      __syncthreads();
    }
  }
  // the patch is read back by lanes of the same wave only: LDS serves a wave in order
  S *ctile = C + (m0 + wm) * a.ldc + n0 + wn;
  if constexpr (EPI) {
    // the bias and residual pieces of a group are requested before the first one is used
#pragma unroll
    for (int i0 = 0; i0 < NIT; i0 += G) {
      V16 bq[G], rq[G];
#pragma unroll
      for (int i = 0; i < G; i++) {
        if (i0 == 0) {  // (requested in front of the barrier above)
          bq[i] = bq0[i];
          rq[i] = rq0[i];
          continue;
        }
        const int ch = (i0 + i) * 64 + lane, row = ch / CPR, col = (ch % CPR) * 8;
        if (btile) bq[i] = *reinterpret_cast<const V16 *>(btile + col);
        if (rtile) rq[i] = *reinterpret_cast<const V16 *>(rtile + (int64_t)row * a.ldr + col);
      }
#pragma unroll
      for (int i = 0; i < G; i++) {
        const int ch = (i0 + i) * 64 + lane, row = ch / CPR, col = (ch % CPR) * 8;
        V16 q = *reinterpret_cast<const V16 *>(patch + row * PITCH + col);
#pragma unroll
        for (int w = 0; w < 4; w++) {
          if (btile) q[w] = epi_add2<EL>(q[w], bq[i][w]);
          if (rtile) q[w] = epi_add2<EL>(q[w], rq[i][w]);
        }
        if (!rtile && a.gelu) {
          bool by_table = false;
          if constexpr (LUT_ROOM) {
            // a register with an input of magnitude bits >= 0x7f00 (the last finite binade,
            // infinities, NaN) sends the whole piece through the arithmetic
            uint32_t top = 0;
#pragma unroll
            for (int w = 0; w < 4; w++) {
              const uint32_t lo16 = q[w] & 0x7fffu, hi16 = (q[w] >> 16) & 0x7fffu;
              top = top > lo16 ? top : lo16;
              top = top > hi16 ? top : hi16;
            }
            by_table = use_lut && top < 0x7f00u;
            if (by_table) {
#pragma unroll
              for (int w = 0; w < 4; w++) q[w] = epi_gelu_lut2(q[w], lut, a.lut_lo, a.lut_n, a.gc[3]);
            }
          }
          if (!by_table) {
#pragma unroll
            for (int w = 0; w < 4; w++) q[w] = epi_gelu2<EL>(q[w], a.gc[0], a.gc[1], a.gc[2], a.gc[3]);
          }
        }
        *reinterpret_cast<V16 *>(ctile + (int64_t)row * a.ldc + col) = q;
      }
    }
  } else {
    // C's rows need not be 16-byte aligned here (a row pitch of 50257 elements, GPT-2's tied
    // head): the hardware takes a 16-byte store at any element boundary, and a lane's eight
    // neighbours in one store beat eight 2-byte stores by a wide margin
    typedef V16 V16_any __attribute__((aligned(2)));
#pragma unroll
    for (int i = 0; i < NIT; i++) {
      const int ch = i * 64 + lane, row = ch / CPR, col = (ch % CPR) * 8;
      const V16 v = *reinterpret_cast<const V16 *>(patch + row * PITCH + col);
      V16_any *dst = reinterpret_cast<V16_any *>(ctile + (int64_t)row * a.ldc + col);
      // (streaming only ever with aligned rows, decided on the host; written as an instruction because
      // the optimiser merges two stores that differ only in the hint)
      if (a.stream_c) asm volatile("global_store_dwordx4 %0, %1, off sc1 nt\n\ts_nop 0" : : "v"(dst), "v"(v) : "memory");
      else *dst = v;
    }
  }
}

}  // namespace gemm_dl
