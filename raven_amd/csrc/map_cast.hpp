// map_cast.hpp — the cast conversion policy (nx_c_map.c:182-218) as one functor
// per (src, dst) pair: load src to its compute type, convert by category, store
// through the dst converter. Float -> int saturates through double with
// NaN -> 0 (nx_c.h:234-250); int -> int wraps on store; -> bool is (v != 0), so
// NaN is true; complex -> real keeps the real part; real -> complex is re + 0i.
#pragma once
#include "map_ops.hpp"

template <int SRC, int DST>
struct CastF {
  using TS = Tr<SRC>;
  using TD = Tr<DST>;
  static constexpr int NIN = 1;
  using Out = typename TD::S;
  using In0 = typename TS::S;
  using In1 = Unused;
  using In2 = Unused;
  __device__ __forceinline__ static Out apply(In0 x) {
    using SC = typename TS::C;
    using DC = typename TD::C;
    SC v = TS::ld(x);
    if constexpr (TD::cat == CAT_FLOAT) {
      if constexpr (TS::cat == CAT_COMPLEX) return TD::st((DC)v.re);
      else return TD::st((DC)v);
    } else if constexpr (TD::cat == CAT_COMPLEX) {
      using R = decltype(DC{}.re);
      if constexpr (TS::cat == CAT_COMPLEX) return TD::st(DC{(R)v.re, (R)v.im});
      else return TD::st(DC{(R)v, (R)0});
    } else if constexpr (TD::cat == CAT_BOOL) {
      if constexpr (TS::cat == CAT_COMPLEX) return TD::st((DC)(v.re != 0 || v.im != 0));
      else return TD::st((DC)(v != 0));
    } else {
      if constexpr (TS::cat == CAT_FLOAT) return TD::st((DC)f2i_sat<Out>((double)v));
      else if constexpr (TS::cat == CAT_COMPLEX) return TD::st((DC)f2i_sat<Out>((double)v.re));
      else return TD::st((DC)v);
    }
  }
};

template <int SRC>
struct CastRow : MapRow {
  template <int DST>
  void set() { fn[DST] = &map_launch<CastF<SRC, DST>>; }
  CastRow() {
#define NXH_SET(DT) set<DT>();
    NXH_FOR_COMPUTE_DTYPES(NXH_SET)
#undef NXH_SET
  }
};
