// window.hip — unfold (im2col) and fold (col2im), packages/nx/lib/backend_c/
// nx_c_move.c:588-870.
//
// unfold: (leading..., spatial...) -> (leading..., prod(kernel), L). Output
// element (lead, tap kf, window w) is one input element, or zero when the tap
// falls into the padding; every output is written once. A block owns one
// leading index (several, when the rows are short) and a run of windows (the
// contiguous axis), each lane eight of them 256 apart, and walks all taps of
// them: the leading index and the window coordinates are decoded once per
// lane, and from then on windows advance by an odometer step and taps by
// another, so no division is left in the per-element work.
//
// fold: (leading..., prod(kernel), L) -> (leading..., output...). One lane per
// OUTPUT element sums the taps that land on it, in ascending tap order and in
// the dtype's compute type, as nx_c_move.c:745-787 does: no atomics, no zeroing
// pass, and float results equal the reference's bit for bit. With window stride 1 and rows of
// whole 16-byte vectors a lane owns a vector of adjacent outputs (fold_vec_kernel).
//
// Limits: at most 6 window dims and 8 leading dims (the reference allows 32 in
// total); beyond that the call fails with Failure.

#include "nxh_common.hpp"
#include "stream_access.hpp"

namespace {

constexpr int WIN_MAXK = 6;
constexpr int WIN_MAXLEAD = 8;
constexpr int WINDOWS_PER_LANE = 8;

// Window dims are right-aligned in arrays of the kernel's compile-time rank KT
// (1, 2, 3 or 6); unused leading slots hold a neutral dim (extent, kernel,
// window count, stride, dilation 1; padding 0; tensor stride 0).
struct WindowArgs {
  const char *in;
  char *out;
  int ld;
  int64_t total, rows;  // elements launched over; (leading, tap) rows of the windowed tensor
  int64_t kernel_prod, L;
  int64_t lshape[WIN_MAXLEAD], l_in[WIN_MAXLEAD], l_out[WIN_MAXLEAD];
  int64_t kernel[WIN_MAXK], stride[WIN_MAXK], dilation[WIN_MAXK], before[WIN_MAXK];
  int64_t win[WIN_MAXK], win_cp[WIN_MAXK];
  int64_t step[WIN_MAXK];       // 256 written in the mixed radix of win[]
  int64_t extent[WIN_MAXK];     // spatial extents of the un-windowed tensor
  int64_t sp_stride[WIN_MAXK];  // its strides along those dims
  int64_t tap_stride, win_stride;  // strides of the windowed tensor's last two dims
  // unfold: the vector stores go past the memory-side cache (decided per call on the host,
  // runtime.hip, nxh_cache_hints); [8,64,128,128] f32, 3 x 3: 84 -> 61 us when nothing reads the
  // 302 MB of windows back. (Streaming loads of the windows in fold changed nothing: 75 -> 78 us.)
  uint32_t stream_out;
};

// I is the type the index arithmetic runs in: int32_t whenever every extent,
// element count and window coordinate fits (64-bit division is an order of
// magnitude slower on this machine), int64_t otherwise. Memory offsets are
// always 64-bit. `leads_per_block` > 1 packs several leading indices with short
// rows into one block, one window per lane.
// AL > 0 (VW = 4 only): the last window dim has stride AL (1 or 2) over a unit-stride
// input dim whose rows are whole, aligned 4-element vectors. The 3 AL + 1 input elements
// behind a unit of four windows then lie in two or three aligned vectors, which are
// fetched whole (a vector is inside the row or in the padding as a whole) and picked
// apart in registers: the position of the first element inside its vector is the tap
// offset modulo 4, the same for the whole row. Four separate element loads per lane,
// 16 or 32 bytes apart from lane to lane, made the address path the bound.
template <class E, class I, int KT, int VW, int AL = 0>
__global__ __launch_bounds__(256) void unfold_kernel(WindowArgs a, I wblocks, int leads_per_block, int taps_per_block) {
  // With VW > 1 a "window" below is a unit of VW consecutive windows of the last
  // window dim (a.L and a.win[KT-1] count units); the unit is stored as one vector.
  // A block owns one leading index (several when the rows are short) and a run of windows, and
  // walks ALL taps of them: the leading index and the window coordinates are decoded once per
  // lane for kernel_prod x up to eight stores (one (leading, tap) row per block left 14 x 14
  // images with one store per decode and a block per 196 outputs), and the taps of a window
  // read neighbouring input elements, which the first tap leaves in the L1. When that leaves
  // too few blocks to fill the chip, the taps are shared out over blockIdx.y.
  const I L = (I)a.L;
  I lead, w0;
  int reps = WINDOWS_PER_LANE;
  if (leads_per_block > 1) {
    const I lanes_per_lead = 256 / leads_per_block;
    lead = (I)blockIdx.x * leads_per_block + (I)threadIdx.x / lanes_per_lead;
    w0 = (I)threadIdx.x % lanes_per_lead;
    reps = 1;
    if (w0 >= L) return;
  } else {
    lead = (I)(blockIdx.x / (unsigned)wblocks);
    w0 = (I)(blockIdx.x % (unsigned)wblocks) * (256 * WINDOWS_PER_LANE) + (I)threadIdx.x;
  }
  if (lead >= (I)(a.rows / a.kernel_prod)) return;
  I oo_lead = 0, io = 0;  // element offsets: I is 32 bits wide only when both spans fit
  for (int d = a.ld - 1; d >= 0; d--) {
    const I c = lead % (I)a.lshape[d];
    lead /= (I)a.lshape[d];
    oo_lead += c * (I)a.l_out[d];
    io += c * (I)a.l_in[d];
  }
  I tap[KT], wc0[KT], wc[KT], kc[KT];  // tap: kc * dilation - pad_before; wc: window coordinate
  I rest = w0;
  const I kf0 = (I)blockIdx.y * taps_per_block;
  I kfr = kf0;
#pragma unroll
  for (int d = KT - 1; d >= 0; d--) {
    kc[d] = kfr % (I)a.kernel[d];
    kfr /= (I)a.kernel[d];
    wc0[d] = rest % (I)a.win[d];
    rest /= (I)a.win[d];
  }
  const E *in = reinterpret_cast<const E *>(a.in);
  E *out = reinterpret_cast<E *>(a.out);
  struct alignas(sizeof(E) * VW) Pack {
    E v[VW];
  };
  I oo = 0;
  auto units = [&](auto r_c) {
    constexpr int R = decltype(r_c)::value;  // AL > 0: first element's place in its aligned vector
#pragma unroll
    for (int u = 0; u < WINDOWS_PER_LANE; u++) {
      const I wf = w0 + (I)u * 256;
      if (u >= reps || wf >= L) break;
      bool valid = true;
      I off = io;
#pragma unroll
      for (int d = 0; d < KT - 1; d++) {
        const I sp = wc[d] * (I)a.stride[d] + tap[d];
        valid = valid && sp >= 0 && sp < (I)a.extent[d];
        off += sp * (I)a.sp_stride[d];
      }
      Pack pk;
      if constexpr (AL > 0) {
        static_assert(AL == 0 || VW == 4, "aligned rows come in units of four windows");
        constexpr int NV = (R + 3 * AL + 1 + 3) / 4;
        const I q = wc[KT - 1] * (VW * AL) + tap[KT - 1] - R;  // a multiple of 4, possibly negative
        E e[NV * 4];
#pragma unroll
        for (int j = 0; j < NV; j++) {
          const I at = q + 4 * j;
          Pack got;
#pragma unroll
          for (int v = 0; v < 4; v++) got.v[v] = E{};
          if (valid && at >= 0 && at < (I)a.extent[KT - 1]) got = *reinterpret_cast<const Pack *>(in + (off + at));
#pragma unroll
          for (int v = 0; v < 4; v++) e[4 * j + v] = got.v[v];
        }
#pragma unroll
        for (int v = 0; v < VW; v++) pk.v[v] = e[R + v * AL];
      } else {
#pragma unroll
        for (int v = 0; v < VW; v++) {
          const I sp = (wc[KT - 1] * VW + v) * (I)a.stride[KT - 1] + tap[KT - 1];
          const bool ok = valid && sp >= 0 && sp < (I)a.extent[KT - 1];
          pk.v[v] = E{};
          if (ok) pk.v[v] = in[off + sp * (I)a.sp_stride[KT - 1]];
        }
      }
      if constexpr (VW == 1) out[oo + wf * (I)a.win_stride] = pk.v[0];
      else if (a.stream_out) store_stream(reinterpret_cast<Pack *>(out + (oo + wf * VW)), pk);
      else *reinterpret_cast<Pack *>(out + (oo + wf * VW)) = pk;
      // 256 windows further: add the digits of 256, carrying towards the front
      I carry = 0;
#pragma unroll
      for (int d = KT - 1; d >= 0; d--) {
        const I t = wc[d] + (I)a.step[d] + carry;
        carry = t >= (I)a.win[d] ? 1 : 0;
        wc[d] = carry ? t - (I)a.win[d] : t;
      }
    }
  };
  const I taps = kf0 + taps_per_block < (I)a.kernel_prod ? kf0 + taps_per_block : (I)a.kernel_prod;
  for (I kf = kf0; kf < taps; kf++) {
    oo = oo_lead + kf * (I)a.tap_stride;
#pragma unroll
    for (int d = 0; d < KT; d++) {
      tap[d] = kc[d] * (I)a.dilation[d] - (I)a.before[d];
      wc[d] = wc0[d];
    }
    if constexpr (AL > 0) {
      switch ((int)(tap[KT - 1] & 3)) {  // two's complement: also right for negative offsets
        case 0: units(std::integral_constant<int, 0>{}); break;
        case 1: units(std::integral_constant<int, 1>{}); break;
        case 2: units(std::integral_constant<int, 2>{}); break;
        default: units(std::integral_constant<int, 3>{}); break;
      }
    } else {
      units(std::integral_constant<int, 0>{});
    }
    // next tap: the odometer over the kernel dims
    bool carry = true;
#pragma unroll
    for (int d = KT - 1; d >= 0; d--) {
      if (carry) {
        kc[d]++;
        carry = kc[d] >= (I)a.kernel[d];
        if (carry) kc[d] = 0;
      }
    }
  }
}

// UNIT: every window stride is 1, so no tap needs a division to find its window.
template <int DT, class I, int KT, bool UNIT>
__global__ __launch_bounds__(256) void fold_kernel(WindowArgs a) {
  using TR = Tr<DT>;
  using S = typename TR::S;
  using C = typename TR::C;
  const int64_t it64 = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (it64 >= a.total) return;
  I ol = (I)it64;
  I oc[KT];  // position in the padded frame
  I oo = 0, il = 0;  // element offsets: I is 32 bits wide only when both tensors' spans fit
#pragma unroll
  for (int d = KT - 1; d >= 0; d--) {
    const I c = ol % (I)a.extent[d];
    ol /= (I)a.extent[d];
    oc[d] = c + (I)a.before[d];
    oo += c * (I)a.sp_stride[d];
  }
  for (int d = a.ld - 1; d >= 0; d--) {
    const I c = ol % (I)a.lshape[d];
    ol /= (I)a.lshape[d];
    oo += c * (I)a.l_out[d];
    il += c * (I)a.l_in[d];
  }
  const S *in = reinterpret_cast<const S *>(a.in);
  C acc;
  if constexpr (TR::cat == CAT_COMPLEX) acc = C{0, 0};
  else acc = (C)0;
  // Taps in ascending flat order kf; kc[] is kf's odometer over the kernel dims. They are
  // taken TB at a time: the addresses of a batch first (a tap that misses reads element 0
  // of this leading index instead and is not added), then all its loads, then the sums in
  // order. One load per loop turn left every wave waiting out a memory latency per tap.
  constexpr int TB = 9;
  I kc[KT];
#pragma unroll
  for (int d = 0; d < KT; d++) kc[d] = 0;
  const I taps = (I)a.kernel_prod;
  for (I kf0 = 0; kf0 < taps; kf0 += TB) {
    bool ok[TB];
    I at[TB];
#pragma unroll
    for (int j = 0; j < TB; j++) {
      bool valid = kf0 + j < taps;
      I wf = 0;
#pragma unroll
      for (int d = 0; d < KT; d++) {
        const I num = oc[d] - kc[d] * (I)a.dilation[d];
        I wc = num;
        if constexpr (!UNIT) {
          const I st = (I)a.stride[d];
          wc = num / st;
          valid = valid && num % st == 0;
        }
        valid = valid && num >= 0 && wc < (I)a.win[d];
        wf += wc * (I)a.win_cp[d];
      }
      ok[j] = valid;
      at[j] = valid ? il + (kf0 + j) * (I)a.tap_stride + wf * (I)a.win_stride : il;
      bool carry = true;
#pragma unroll
      for (int d = KT - 1; d >= 0; d--) {
        if (carry) {
          kc[d]++;
          carry = kc[d] >= (I)a.kernel[d];
          if (carry) kc[d] = 0;
        }
      }
    }
    S raw[TB];
#pragma unroll
    for (int j = 0; j < TB; j++) raw[j] = in[at[j]];
#pragma unroll
    for (int j = 0; j < TB; j++) {
      const C v = TR::ld(raw[j]);
      C sum;
      if constexpr (TR::cat == CAT_SINT) sum = (C)((uint64_t)acc + (uint64_t)v);
      else sum = (C)(acc + v);
      acc = ok[j] ? sum : acc;
    }
  }
  reinterpret_cast<S *>(a.out)[oo] = TR::st(acc);
}

// The same sums with V adjacent outputs of the last dim per lane (V x sizeof(S) = 16 bytes), for
// window stride 1 everywhere, a unit-stride last output dim whose extent is a multiple of V and
// a plain row-major windowed tensor of `in_elems` elements. The V outputs share everything about
// a tap but their position in the last window dim, so a tap is one (unaligned) 16-byte load at
// the first output's window and V selects; the address and validity arithmetic, which bounded
// the one-output-per-lane form, is done once per V outputs. A vector that straddles the row's
// ends is loaded whole and its outside elements are not added; it lies inside the tensor except
// at the tensor's very first and last elements, where the elements are fetched one by one.
// Every output still adds its taps in ascending order.
template <int DT, int KT, int V>
__global__ __launch_bounds__(256) void fold_vec_kernel(WindowArgs a, int32_t in_elems) {
  using TR = Tr<DT>;
  using S = typename TR::S;
  using C = typename TR::C;
  using I = int32_t;
  struct __attribute__((packed, aligned(alignof(S)))) VecU {
    S v[V];
  };
  struct alignas(16) VecA {
    S v[V];
  };
  const int64_t it64 = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (it64 >= a.total / V) return;
  I ol = (I)it64;
  I oc[KT];  // position in the padded frame (of the lane's first output, in the last dim)
  I oo = 0, il = 0;
  {
    const I ev = (I)a.extent[KT - 1] / V, c = (ol % ev) * V;
    ol /= ev;
    oc[KT - 1] = c + (I)a.before[KT - 1];
    oo += c;
  }
#pragma unroll
  for (int d = KT - 2; d >= 0; d--) {
    const I c = ol % (I)a.extent[d];
    ol /= (I)a.extent[d];
    oc[d] = c + (I)a.before[d];
    oo += c * (I)a.sp_stride[d];
  }
  for (int d = a.ld - 1; d >= 0; d--) {
    const I c = ol % (I)a.lshape[d];
    ol /= (I)a.lshape[d];
    oo += c * (I)a.l_out[d];
    il += c * (I)a.l_in[d];
  }
  const S *in = reinterpret_cast<const S *>(a.in);
  C acc[V];
#pragma unroll
  for (int e = 0; e < V; e++) {
    if constexpr (TR::cat == CAT_COMPLEX) acc[e] = C{0, 0};
    else acc[e] = (C)0;
  }
  auto add = [](C x, C v) -> C {
    if constexpr (TR::cat == CAT_SINT) return (C)((uint64_t)x + (uint64_t)v);
    else return (C)(x + v);
  };
  constexpr int TB = 9;
  const I win_last = (I)a.win[KT - 1];
  I kc[KT];
#pragma unroll
  for (int d = 0; d < KT; d++) kc[d] = 0;
  const I taps = (I)a.kernel_prod;
  for (I kf0 = 0; kf0 < taps; kf0 += TB) {
    bool whole[TB], piecewise[TB];  // loaded as one vector / element by element (the tensor's two ends)
    I at[TB], first[TB];            // offset of the first output's window; its coordinate in the last window dim
#pragma unroll
    for (int j = 0; j < TB; j++) {
      bool valid = kf0 + j < taps;
      I wf = 0;
#pragma unroll
      for (int d = 0; d < KT; d++) {
        const I num = oc[d] - kc[d] * (I)a.dilation[d];
        if (d == KT - 1) {
          first[j] = num;
          valid = valid && num > -V && num < win_last;  // some output of the V has a window here
        } else {
          valid = valid && num >= 0 && num < (I)a.win[d];
        }
        wf += num * (I)a.win_cp[d];
      }
      const I off = il + (kf0 + j) * (I)a.tap_stride + wf;
      const bool inside = off >= 0 && off + V <= in_elems;
      whole[j] = valid && inside;
      piecewise[j] = valid && !inside;
      at[j] = off;
      bool carry = true;
#pragma unroll
      for (int d = KT - 1; d >= 0; d--) {
        if (carry) {
          kc[d]++;
          carry = kc[d] >= (I)a.kernel[d];
          if (carry) kc[d] = 0;
        }
      }
    }
    VecU raw[TB];
#pragma unroll
    for (int j = 0; j < TB; j++) raw[j] = *reinterpret_cast<const VecU *>(in + (whole[j] ? at[j] : 0));
#pragma unroll
    for (int j = 0; j < TB; j++) {
#pragma unroll
      for (int e = 0; e < V; e++) {
        const bool ok = whole[j] && (uint32_t)(first[j] + e) < (uint32_t)win_last;
        const C sum = add(acc[e], TR::ld(raw[j].v[e]));
        acc[e] = ok ? sum : acc[e];
      }
      if (piecewise[j]) {
        for (int e = 0; e < V; e++)
          if ((uint32_t)(first[j] + e) < (uint32_t)win_last) acc[e] = add(acc[e], TR::ld(in[at[j] + e]));
      }
    }
  }
  VecA res;
#pragma unroll
  for (int e = 0; e < V; e++) res.v[e] = TR::st(acc[e]);
  *reinterpret_cast<VecA *>(reinterpret_cast<S *>(a.out) + oo) = res;
}

struct G16w {
  uint64_t lo, hi;
};

// 32-bit index arithmetic is exact when every quantity that is divided, and
// every coordinate built from the quotients, stays below 2^31.
bool fits_int32(const WindowArgs &a) {
  const int64_t lim = (int64_t)1 << 31;
  if (a.total >= lim || a.rows >= lim || a.L + 256 * WINDOWS_PER_LANE >= lim || a.kernel_prod >= lim) return false;
  for (int d = 0; d < WIN_MAXK; d++) {
    const int64_t reach = (a.win[d] + 256) * a.stride[d] + a.kernel[d] * a.dilation[d] + a.before[d] + a.extent[d];
    if (reach >= lim) return false;
  }
  return true;
}
// Element offsets fit 32 bits too: the spans of the windowed tensor (`windows` along its last
// dim) and of the plain one.
bool spans_fit_int32(const WindowArgs &a, int64_t windows) {
  int64_t cols_span = (a.kernel_prod - 1) * std::llabs(a.tap_stride) + (windows - 1) * std::llabs(a.win_stride), plain_span = 0;
  for (int d = 0; d < a.ld; d++) {
    // l_in / l_out: which of the two is the windowed tensor depends on the direction; bound both by the larger
    const int64_t m = std::max(std::llabs(a.l_in[d]), std::llabs(a.l_out[d]));
    cols_span += (a.lshape[d] - 1) * m;
    plain_span += (a.lshape[d] - 1) * m;
  }
  for (int d = 0; d < WIN_MAXK; d++) plain_span += (a.extent[d] - 1) * std::llabs(a.sp_stride[d]);
  return cols_span < ((int64_t)1 << 31) && plain_span < ((int64_t)1 << 31);
}
int rank_class(int K) { return K <= 3 ? K : WIN_MAXK; }

typedef void (*fold_launch_fn)(nxh_context *, const WindowArgs &, int, bool);
// `plain_in`: the windowed tensor is row-major without gaps (its offsets then lie in [0, rows x L)).
template <int DT>
void fold_launch(nxh_context *ctx, const WindowArgs &a, int kt, bool plain_in) {
  const dim3 grid((unsigned)((a.total + 255) / 256)), block(256);
  const bool narrow = fits_int32(a) && spans_fit_int32(a, a.L);  // 32-bit index arithmetic, offsets included
  bool unit = true;
  for (int d = 0; d < WIN_MAXK; d++) unit = unit && a.stride[d] == 1;
  // 16 bytes of adjacent outputs per lane
  constexpr int V = 16 / (int)sizeof(typename Tr<DT>::S);
  if constexpr (V == 2 || V == 4 || V == 8) {
    const int last = (kt <= 3 ? kt : WIN_MAXK) - 1;
    // (offsets of the windowed tensor, plus a vector, stay below 2^31)
    bool vec = narrow && unit && plain_in && a.rows * a.L >= V && a.rows * a.L < ((int64_t)1 << 31) - 16 &&
               a.extent[last] % V == 0 && a.sp_stride[last] == 1 && (uintptr_t)a.out % 16 == 0;
    for (int d = 0; d < last; d++) vec = vec && (a.extent[d] == 1 || a.sp_stride[d] % V == 0);
    for (int d = 0; d < a.ld; d++) vec = vec && (a.lshape[d] == 1 || a.l_out[d] % V == 0);
    if (vec) {
      nxh_set_path("fold_16B");
      const dim3 vgrid((unsigned)((a.total / V + 255) / 256));
      const int32_t in_elems = (int32_t)(a.rows * a.L);
      switch (kt) {
        case 1: hipLaunchKernelGGL((fold_vec_kernel<DT, 1, V>), vgrid, block, 0, ctx->stream, a, in_elems); break;
        case 2: hipLaunchKernelGGL((fold_vec_kernel<DT, 2, V>), vgrid, block, 0, ctx->stream, a, in_elems); break;
        case 3: hipLaunchKernelGGL((fold_vec_kernel<DT, 3, V>), vgrid, block, 0, ctx->stream, a, in_elems); break;
        default: hipLaunchKernelGGL((fold_vec_kernel<DT, WIN_MAXK, V>), vgrid, block, 0, ctx->stream, a, in_elems); break;
      }
      return;
    }
  }
#define NXH_FOLD_CASE(KT)                                                                                        \
  case KT:                                                                                                       \
    if (narrow && unit) hipLaunchKernelGGL((fold_kernel<DT, int32_t, KT, true>), grid, block, 0, ctx->stream, a); \
    else if (narrow) hipLaunchKernelGGL((fold_kernel<DT, int32_t, KT, false>), grid, block, 0, ctx->stream, a);  \
    else hipLaunchKernelGGL((fold_kernel<DT, int64_t, KT, false>), grid, block, 0, ctx->stream, a);              \
    break;
  switch (kt) {
    NXH_FOLD_CASE(1)
    NXH_FOLD_CASE(2)
    NXH_FOLD_CASE(3)
    NXH_FOLD_CASE(WIN_MAXK)
  }
#undef NXH_FOLD_CASE
}

template <class E, int VW, int AL = 0>
int unfold_launch_v(nxh_context *ctx, const char *op, const WindowArgs &a, int kt) {
  const int64_t leads = a.rows / a.kernel_prod;
  int leads_per_block = 1;
  int64_t wblocks = (a.L + 256 * WINDOWS_PER_LANE - 1) / (256 * WINDOWS_PER_LANE), blocks = leads * wblocks;
  if (a.L <= 256) {  // short rows: a power-of-two share of the block per leading index, one unit per lane
    int lanes = 1;
    while (lanes < a.L) lanes <<= 1;
    leads_per_block = 256 / lanes;
    blocks = (leads + leads_per_block - 1) / leads_per_block;
  }
  if (blocks > 0x7fffffffLL) return nxh_fail(NXH_FAILURE, op, "too many elements for one launch");
  // all taps in one block unless that leaves the chip short of blocks (about 16 per compute unit)
  const int64_t want = ((int64_t)(ctx->compute_units > 0 ? ctx->compute_units : 256) * 16 + blocks - 1) / blocks;
  const int64_t groups = std::max<int64_t>(1, std::min<int64_t>(std::min<int64_t>(want, a.kernel_prod), 65535));
  const int taps_per_block = (int)((a.kernel_prod + groups - 1) / groups);
  const dim3 grid((unsigned)blocks, (unsigned)((a.kernel_prod + taps_per_block - 1) / taps_per_block)), block(256);
  const bool narrow = fits_int32(a) && spans_fit_int32(a, a.L * VW);
#define NXH_UNFOLD_CASE(KT)                                                                                     \
  case KT:                                                                                                      \
    if (narrow)                                                                                                 \
      hipLaunchKernelGGL((unfold_kernel<E, int32_t, KT, VW, AL>), grid, block, 0, ctx->stream, a,               \
                         (int32_t)wblocks, leads_per_block, taps_per_block);                                    \
    else                                                                                                        \
      hipLaunchKernelGGL((unfold_kernel<E, int64_t, KT, VW, AL>), grid, block, 0, ctx->stream, a, wblocks,      \
                         leads_per_block, taps_per_block);                                                      \
    break;
  switch (kt) {
    NXH_UNFOLD_CASE(1)
    NXH_UNFOLD_CASE(2)
    NXH_UNFOLD_CASE(3)
    NXH_UNFOLD_CASE(WIN_MAXK)
  }
#undef NXH_UNFOLD_CASE
  return NXH_OK;
}

// Four consecutive windows of the last window dim become one store when the
// output allows it: that dim's window count a multiple of 4, windows
// contiguous, every row of the output starting on a 4-element boundary.
// `aligned_rows`: the input side of the aligned form (see unfold_kernel) holds.
// `pair_ok`: the same for pairs of windows (a 14 x 14 image has 196-element rows of windows,
// whole vectors, but 14 windows per image row: pairs never straddle an image row, fours do).
template <class E>
int unfold_launch(nxh_context *ctx, const char *op, WindowArgs &a, int kt, bool vector_ok, bool aligned_rows,
                  bool pair_ok) {
  constexpr int VW = sizeof(E) <= 4 ? 4 : 1;
  auto in_units_of = [&](int vw) {
    a.L /= vw;
    a.win[kt - 1] /= vw;
    int64_t rest = 256;
    for (int s = kt - 1; s >= 0; s--) {  // 256 units further, in the new radix
      a.step[s] = rest % a.win[s];
      rest /= a.win[s];
    }
  };
  if constexpr (sizeof(E) <= 8) {
    if (pair_ok && a.win[kt - 1] % 2 == 0 && !(VW > 1 && vector_ok && a.win[kt - 1] % VW == 0)) {
      in_units_of(2);
      nxh_set_path("unfold_pairs");
      return unfold_launch_v<E, 2>(ctx, op, a, kt);
    }
  }
  if constexpr (VW > 1) {
    if (vector_ok && a.win[kt - 1] % VW == 0) {
      a.L /= VW;
      a.win[kt - 1] /= VW;
      int64_t rest = 256;
      for (int s = kt - 1; s >= 0; s--) {  // 256 units further, in the new radix
        a.step[s] = rest % a.win[s];
        rest /= a.win[s];
      }
      if (aligned_rows && a.stride[kt - 1] == 1) {
        nxh_set_path("unfold_aligned");
        return unfold_launch_v<E, VW, 1>(ctx, op, a, kt);
      }
      if (aligned_rows && a.stride[kt - 1] == 2) {
        nxh_set_path("unfold_aligned");
        return unfold_launch_v<E, VW, 2>(ctx, op, a, kt);
      }
      return unfold_launch_v<E, VW>(ctx, op, a, kt);
    }
  }
  return unfold_launch_v<E, 1>(ctx, op, a, kt);
}

// Parameters common to both directions. `plain` is the un-windowed tensor
// (unfold's input, fold's output), `cols` the windowed one. Returns the
// kernels' compile-time rank in *kt.
int window_setup(const char *op, const nxh_tensor *plain, const nxh_tensor *cols, int K, const int64_t *spatial,
                 const int64_t *kernel, const int64_t *stride, const int64_t *dilation, const int64_t *padding,
                 WindowArgs &a, int *kt) {
  if (K < 1 || plain->ndim < K || cols->ndim < 2) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
  const int ld = plain->ndim - K;
  if (cols->ndim != ld + 2) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
  if (K > WIN_MAXK || ld > WIN_MAXLEAD) return nxh_fail(NXH_FAILURE, op, "more than 6 window or 8 leading dimensions");
  a.ld = ld;
  for (int d = 0; d < ld; d++) {
    if (plain->shape[d] != cols->shape[d]) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
    a.lshape[d] = plain->shape[d];
  }
  const int KT = rank_class(K), shift = KT - K;
  *kt = KT;
  for (int d = 0; d < WIN_MAXK; d++) {
    a.kernel[d] = a.stride[d] = a.dilation[d] = a.win[d] = a.extent[d] = 1;
    a.before[d] = a.step[d] = a.sp_stride[d] = a.win_cp[d] = 0;
  }
  int64_t kp = 1, L = 1;
  for (int d = 0; d < K; d++) {
    if (kernel[d] < 1 || stride[d] < 1 || dilation[d] < 1 || padding[2 * d] < 0 || padding[2 * d + 1] < 0)
      return nxh_fail(NXH_INVALID_ARGUMENT, op, "kernel, stride and dilation must be positive, padding non-negative");
    const int s = d + shift;
    a.kernel[s] = kernel[d];
    a.stride[s] = stride[d];
    a.dilation[s] = dilation[d];
    a.before[s] = padding[2 * d];
    a.extent[s] = spatial[d];
    if (plain->shape[ld + d] != spatial[d]) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
    a.sp_stride[s] = plain->strides[ld + d];
    const int64_t eff = dilation[d] * (kernel[d] - 1) + 1;
    const int64_t padded = spatial[d] + padding[2 * d] + padding[2 * d + 1];
    const int64_t win = (padded - eff) / stride[d] + 1;
    a.win[s] = win < 1 ? 1 : win;  // nx_c_move.c:640
    kp *= kernel[d];
    L *= a.win[s];
  }
  int64_t cp = 1, rest = 256;
  for (int s = KT - 1; s >= 0; s--) {
    a.win_cp[s] = cp;
    cp *= a.win[s];
    a.step[s] = rest % a.win[s];
    rest /= a.win[s];
  }
  a.kernel_prod = cols->shape[ld];
  a.L = cols->shape[ld + 1];
  // the windowed tensor must hold exactly the taps and windows of this geometry
  if (a.kernel_prod != kp || a.L != L) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
  a.tap_stride = cols->strides[ld];
  a.win_stride = cols->strides[ld + 1];
  return NXH_OK;
}

}  // namespace

// The cache policy's view of an unfold / fold: the windowed tensor, kernel_prod times the size of the
// other one, is written (unfold) or read (fold) exactly once.
static uint32_t window_cache_hints(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *x, uint32_t allow) {
  const void *base[2] = {out->data, x->data};
  uint64_t bytes[2];
  for (int k = 0; k < 2; k++) {
    const nxh_tensor *t = k ? x : out;
    uint64_t n = 1;
    for (int d = 0; d < t->ndim; d++)
      if (t->strides[d] != 0) n *= (uint64_t)t->shape[d];
    bytes[k] = n * (uint64_t)nxh_elem_size(t->dtype);
  }
  return nxh_cache_hints(ctx, 2, base, bytes, allow);
}

NXH_EXPORT int nxh_unfold(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *x, int n_window_dims,
                          const int64_t *kernel_size, const int64_t *stride, const int64_t *dilation,
                          const int64_t *padding) {
  NXH_DEFER_SETTLE(ctx, 1, out, x);
  const char *op = "unfold";
  if (!ctx || !out || !x || !kernel_size || !stride || !dilation || !padding)
    return nxh_fail(NXH_INVALID_ARGUMENT, op, "null argument");
  int rc = nxh_check_tensor(op, out);
  if (!rc) rc = nxh_check_tensor(op, x);
  if (rc) return rc;
  if (nxh_is_packed(out->dtype)) return nxh_fail(NXH_FAILURE, op, NXH_ERR_PACKED);
  if (x->dtype != out->dtype) return nxh_fail(NXH_FAILURE, op, NXH_ERR_UNSUPPORTED);
  WindowArgs a;
  int kt = 0;
  const int K = n_window_dims;
  if (K < 1 || x->ndim < K) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_SHAPE);
  if ((rc = window_setup(op, x, out, K, &x->shape[x->ndim - K], kernel_size, stride, dilation, padding, a, &kt))) return rc;
  for (int d = 0; d < out->ndim; d++)
    if (out->shape[d] > 1 && out->strides[d] == 0) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_OUT_ALIASED);
  const int es = (int)nxh_elem_size(out->dtype);
  for (int d = 0; d < a.ld; d++) {
    a.l_in[d] = x->strides[d];
    a.l_out[d] = out->strides[d];
  }
  a.rows = a.kernel_prod;
  for (int d = 0; d < a.ld; d++) a.rows *= a.lshape[d];
  a.total = a.rows * a.L;
  if (a.total == 0) return NXH_OK;
  if (a.total > 0x7fffffffLL * 256) return nxh_fail(NXH_FAILURE, op, "too many elements for one launch");
  a.in = (const char *)x->data + x->offset * es;
  a.out = (char *)out->data + out->offset * es;
  bool vector_ok = a.win_stride == 1 && a.tap_stride % 4 == 0 && ((uintptr_t)a.out % (uintptr_t)(4 * es)) == 0;
  for (int d = 0; d < a.ld; d++)
    if (a.lshape[d] > 1 && a.l_out[d] % 4 != 0) vector_ok = false;
  // the input side of the aligned form: unit stride along the last window dim, whose rows
  // are whole 4-element vectors, every other step of the input a multiple of 4 elements
  bool pair_ok = a.win_stride == 1 && a.tap_stride % 2 == 0 && ((uintptr_t)a.out % (uintptr_t)(2 * es)) == 0;
  for (int d = 0; d < a.ld; d++)
    if (a.lshape[d] > 1 && a.l_out[d] % 2 != 0) pair_ok = false;
  bool aligned_rows = a.sp_stride[kt - 1] == 1 && a.extent[kt - 1] % 4 == 0 && ((uintptr_t)a.in % (uintptr_t)(4 * es)) == 0;
  for (int d = 0; d < kt - 1; d++)
    if (a.extent[d] > 1 && a.sp_stride[d] % 4 != 0) aligned_rows = false;
  for (int d = 0; d < a.ld; d++)
    if (a.lshape[d] > 1 && a.l_in[d] % 4 != 0) aligned_rows = false;
  std::lock_guard<std::mutex> guard(ctx->mu);
  NXH_HIP(op, hipSetDevice(ctx->device));
  nxh_set_path("unfold");
  a.stream_out = (window_cache_hints(ctx, out, x, NXH_STREAM_OUT) & NXH_STREAM_OUT) != 0;
  switch (es) {
    case 1: rc = unfold_launch<uint8_t>(ctx, op, a, kt, vector_ok, aligned_rows, pair_ok); break;
    case 2: rc = unfold_launch<uint16_t>(ctx, op, a, kt, vector_ok, aligned_rows, pair_ok); break;
    case 4: rc = unfold_launch<uint32_t>(ctx, op, a, kt, vector_ok, aligned_rows, pair_ok); break;
    case 8: rc = unfold_launch<uint64_t>(ctx, op, a, kt, vector_ok, aligned_rows, pair_ok); break;
    default: rc = unfold_launch<G16w>(ctx, op, a, kt, vector_ok, false, false); break;
  }
  if (rc) return rc;
  NXH_HIP(op, hipGetLastError());
  return NXH_OK;
}

NXH_EXPORT int nxh_fold(nxh_context *ctx, const nxh_tensor *out, const nxh_tensor *x, int n_window_dims,
                        const int64_t *output_size, const int64_t *kernel_size, const int64_t *stride,
                        const int64_t *dilation, const int64_t *padding) {
  NXH_DEFER_SETTLE(ctx, 1, out, x);
  const char *op = "fold";
  if (!ctx || !out || !x || !output_size || !kernel_size || !stride || !dilation || !padding)
    return nxh_fail(NXH_INVALID_ARGUMENT, op, "null argument");
  int rc = nxh_check_tensor(op, out);
  if (!rc) rc = nxh_check_tensor(op, x);
  if (rc) return rc;
  const int dt = out->dtype;
  if (nxh_is_packed(dt)) return nxh_fail(NXH_FAILURE, op, NXH_ERR_PACKED);
  if (x->dtype != dt) return nxh_fail(NXH_FAILURE, op, NXH_ERR_UNSUPPORTED);
  WindowArgs a;
  int kt = 0;
  const int K = n_window_dims;
  if ((rc = window_setup(op, out, x, K, output_size, kernel_size, stride, dilation, padding, a, &kt))) return rc;
  for (int d = 0; d < out->ndim; d++)
    if (out->shape[d] > 1 && out->strides[d] == 0) return nxh_fail(NXH_INVALID_ARGUMENT, op, NXH_ERR_OUT_ALIASED);
  const int es = (int)nxh_elem_size(dt);
  for (int d = 0; d < a.ld; d++) {
    a.l_in[d] = x->strides[d];
    a.l_out[d] = out->strides[d];
  }
  a.total = 1;
  for (int d = 0; d < a.ld; d++) a.total *= a.lshape[d];
  a.rows = a.total * a.kernel_prod;
  for (int d = 0; d < K; d++) a.total *= output_size[d];
  if (a.total == 0) return NXH_OK;
  if (a.total > 0x7fffffffLL * 256) return nxh_fail(NXH_FAILURE, op, "too many elements for one launch");
  a.in = (const char *)x->data + x->offset * es;
  a.out = (char *)out->data + out->offset * es;
  struct Table {
    fold_launch_fn fn[NXH_DTYPE_COUNT] = {};
    Table() {
#define NXH_FD(DT) fn[DT] = &fold_launch<DT>;
      NXH_FOR_COMPUTE_DTYPES(NXH_FD)
#undef NXH_FD
    }
  };
  static const Table table;
  if (!table.fn[dt]) return nxh_fail(NXH_FAILURE, op, NXH_ERR_UNSUPPORTED);
  std::lock_guard<std::mutex> guard(ctx->mu);
  NXH_HIP(op, hipSetDevice(ctx->device));
  nxh_set_path("fold");
  a.stream_out = 0;
  (void)window_cache_hints(ctx, out, x, 0);  // (the accounting only)
  bool plain_in = a.win_stride == 1 && a.tap_stride == a.L;
  for (int64_t d = a.ld - 1, run = a.kernel_prod * a.L; d >= 0; d--) {
    if (a.lshape[d] > 1 && a.l_in[d] != run) plain_in = false;
    run *= a.lshape[d];
  }
  table.fn[dt](ctx, a, kt, plain_in);
  NXH_HIP(op, hipGetLastError());
  return NXH_OK;
}
