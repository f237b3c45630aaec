// stream_access.hpp — device helpers for accesses that go past the memory-side cache
// (non-temporal loads and stores), for global-memory pointers that went through an asm
// statement, and the explicit wait behind a group of loads. Used by the elementwise and
// the reduction kernels; which launches stream is decided on the host (runtime.hip,
// nxh_cache_hints).
#pragma once

#include "nxh_common.hpp"

// Streaming (non-temporal) access to one vector: the bytes go past the memory-side cache
// instead of displacing what it holds. A kernel holds both forms of its loads and of its
// stores and takes one of each by a flag that is uniform over the launch, branching once
// around a whole group of accesses. Loads use the compiler's non-temporal load. Stores are
// written as instructions: two stores that differ only in the hint are merged into one
// plain store by the optimiser. Nothing may overwrite the data registers of a store wider
// than 8 bytes in the cycle after it, which the compiler cannot see here: the no-op covers it.
template <int BYTES>
struct StreamWord;
#define NXH_STREAM_WORD(BYTES, TYPE, STORE)                                                        \
  template <>                                                                                      \
  struct StreamWord<BYTES> {                                                                       \
    typedef TYPE T;                                                                                \
    __device__ __forceinline__ static void store(T *p, T v) {                                      \
      asm volatile(STORE " %0, %1, off sc1 nt\n\ts_nop 0" : : "v"(p), "v"(v) : "memory");          \
    }                                                                                              \
  };
template <> struct StreamWord<1> { typedef uint8_t T; };
template <> struct StreamWord<2> { typedef uint16_t T; };
typedef uint32_t stream_u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t stream_u32x4 __attribute__((ext_vector_type(4)));
NXH_STREAM_WORD(4, uint32_t, "global_store_dword")
NXH_STREAM_WORD(8, stream_u32x2, "global_store_dwordx2")
NXH_STREAM_WORD(16, stream_u32x4, "global_store_dwordx4")
#undef NXH_STREAM_WORD
template <class VT>
static constexpr bool stream_ok = sizeof(VT) == 4 || sizeof(VT) == 8 || (sizeof(VT) >= 16 && sizeof(VT) % 16 == 0);
template <class VT>
__device__ __forceinline__ VT load_stream(const VT *p) {
  if constexpr (stream_ok<VT>) {
    constexpr int S = (int)sizeof(VT), W = S < 16 ? S : 16;
    using WT = typename StreamWord<W>::T;
    struct Pieces { WT w[S / W]; } t;
#pragma unroll
    for (int i = 0; i < S / W; i++) t.w[i] = __builtin_nontemporal_load(reinterpret_cast<const WT *>(p) + i);
    return __builtin_bit_cast(VT, t);
  } else {
    return *p;
  }
}
template <class VT>
__device__ __forceinline__ void store_stream(VT *p, const VT &v) {
  if constexpr (stream_ok<VT>) {
    constexpr int S = (int)sizeof(VT), W = S < 16 ? S : 16;
    using WT = typename StreamWord<W>::T;
    struct Pieces { WT w[S / W]; };
    const Pieces t = __builtin_bit_cast(Pieces, v);
#pragma unroll
    for (int i = 0; i < S / W; i++) StreamWord<W>::store(reinterpret_cast<WT *>(p) + i, t.w[i]);
  } else {
    *p = v;
  }
}

// A vector read through a pointer that is known to be global memory (address space 1), in
// pieces of at most 16 bytes. For addresses that went through an asm statement: a plain
// pointer that comes out of one is no longer known to be global, and its loads would be
// flat loads, which also count as LDS operations.
#define NXH_GLOBAL __attribute__((address_space(1)))
template <bool STREAM, class VT>
__device__ __forceinline__ VT load_global(const NXH_GLOBAL char *p) {
  constexpr int S = (int)sizeof(VT), W = S < 16 ? S : 16;
  static_assert(S % W == 0 && (W & (W - 1)) == 0, "vector size");
  using WT = typename StreamWord<W>::T;
  struct Pieces { WT w[S / W]; } t;
  const NXH_GLOBAL WT *q = (const NXH_GLOBAL WT *)p;
#pragma unroll
  for (int i = 0; i < S / W; i++) {
    if constexpr (STREAM && stream_ok<VT>) t.w[i] = __builtin_nontemporal_load(q + i);
    else t.w[i] = q[i];
  }
  return __builtin_bit_cast(VT, t);
}

// All outstanding vector-memory operations of the wave (s_waitcnt vmcnt(0), the other
// counters left alone). Written out where a kernel has issued every load of a phase: behind
// it the compiler knows that nothing is in flight and puts no conservative waits between
// the stores of the lanes' separately guarded vectors.
__device__ __forceinline__ void wait_for_loads() { __builtin_amdgcn_s_waitcnt(0x0F70); }

