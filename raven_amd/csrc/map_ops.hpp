// map_ops.hpp — scalar semantics of every elementwise op, per dtype category.
//
// Each Op states, per category (signed int, unsigned int, float, complex,
// bool), whether the reference defines it (`ok`) and the expression it computes
// in the dtype's compute type (`eval`). The expressions restate
// packages/nx/lib/backend_c/nx_c_map.c:300-803; unsupported pairs are holes in
// the dispatch tables and are rejected, never identity.
#pragma once
#include <type_traits>

#include "map_kernels.hpp"

// ── libm by compute type ────────────────────────────────────────────────────
#define NXH_M1(name, ff, fd)                                      \
  __device__ __forceinline__ float name(float x) { return ff(x); } \
  __device__ __forceinline__ double name(double x) { return fd(x); }
NXH_M1(m_sqrt, ::sqrtf, ::sqrt)
NXH_M1(m_exp, ::expf, ::exp)
NXH_M1(m_log, ::logf, ::log)
NXH_M1(m_sin, ::sinf, ::sin)
NXH_M1(m_cos, ::cosf, ::cos)
NXH_M1(m_tan, ::tanf, ::tan)
NXH_M1(m_asin, ::asinf, ::asin)
NXH_M1(m_acos, ::acosf, ::acos)
NXH_M1(m_atan, ::atanf, ::atan)
NXH_M1(m_sinh, ::sinhf, ::sinh)
NXH_M1(m_cosh, ::coshf, ::cosh)
NXH_M1(m_tanh, ::tanhf, ::tanh)
NXH_M1(m_trunc, ::truncf, ::trunc)
NXH_M1(m_ceil, ::ceilf, ::ceil)
NXH_M1(m_floor, ::floorf, ::floor)
NXH_M1(m_round, ::roundf, ::round)
NXH_M1(m_erf, ::erff, ::erf)
NXH_M1(m_fabs, ::fabsf, ::fabs)
__device__ __forceinline__ float m_hypot(float a, float b) { return ::hypotf(a, b); }
__device__ __forceinline__ double m_hypot(double a, double b) { return ::hypot(a, b); }
__device__ __forceinline__ float m_atan2(float a, float b) { return ::atan2f(a, b); }
__device__ __forceinline__ double m_atan2(double a, double b) { return ::atan2(a, b); }
__device__ __forceinline__ float m_pow(float a, float b) { return ::powf(a, b); }
__device__ __forceinline__ double m_pow(double a, double b) { return ::pow(a, b); }
__device__ __forceinline__ float m_fmod(float a, float b) { return ::fmodf(a, b); }
__device__ __forceinline__ double m_fmod(double a, double b) { return ::fmod(a, b); }
__device__ __forceinline__ float m_copysign(float a, float b) { return ::copysignf(a, b); }
__device__ __forceinline__ double m_copysign(double a, double b) { return ::copysign(a, b); }

// ── complex elementary functions (C99 principal branches) ───────────────────
template <class R>
__device__ __forceinline__ R c_abs(cplx<R> z) { return m_hypot(z.re, z.im); }
template <class R>
__device__ cplx<R> c_sqrt(cplx<R> z) {
  if (z.re == 0 && z.im == 0) return {0, z.im};
  R t = m_sqrt((m_fabs(z.re) + c_abs(z)) * (R)0.5);
  if (z.re >= 0) return {t, z.im / (2 * t)};
  return {m_fabs(z.im) / (2 * t), m_copysign(t, z.im)};
}
template <class R>
__device__ cplx<R> c_exp(cplx<R> z) {
  R e = m_exp(z.re);
  return {e * m_cos(z.im), e * m_sin(z.im)};
}
template <class R>
__device__ cplx<R> c_log(cplx<R> z) { return {m_log(c_abs(z)), m_atan2(z.im, z.re)}; }
template <class R>
__device__ cplx<R> c_sin(cplx<R> z) { return {m_sin(z.re) * m_cosh(z.im), m_cos(z.re) * m_sinh(z.im)}; }
template <class R>
__device__ cplx<R> c_cos(cplx<R> z) { return {m_cos(z.re) * m_cosh(z.im), -(m_sin(z.re) * m_sinh(z.im))}; }
template <class R>
__device__ cplx<R> c_sinh(cplx<R> z) { return {m_sinh(z.re) * m_cos(z.im), m_cosh(z.re) * m_sin(z.im)}; }
template <class R>
__device__ cplx<R> c_cosh(cplx<R> z) { return {m_cosh(z.re) * m_cos(z.im), m_sinh(z.re) * m_sin(z.im)}; }
template <class R>
__device__ cplx<R> c_tan(cplx<R> z) { return c_sin(z) / c_cos(z); }
template <class R>
__device__ cplx<R> c_tanh(cplx<R> z) { return c_sinh(z) / c_cosh(z); }
template <class R>
__device__ cplx<R> c_asin(cplx<R> z) {
  // -i log(iz + sqrt(1 - z^2))
  cplx<R> one{1, 0}, iz{-z.im, z.re};
  cplx<R> w = c_log(iz + c_sqrt(one - z * z));
  return {w.im, -w.re};
}
template <class R>
__device__ cplx<R> c_acos(cplx<R> z) {
  cplx<R> a = c_asin(z);
  return {(R)1.5707963267948966 - a.re, -a.im};
}
template <class R>
__device__ cplx<R> c_atan(cplx<R> z) {
  // (i/2) (log(1 - iz) - log(1 + iz))
  cplx<R> one{1, 0}, iz{-z.im, z.re};
  cplx<R> d = c_log(one - iz) - c_log(one + iz);
  return {-(R)0.5 * d.im, (R)0.5 * d.re};
}
template <class R>
__device__ cplx<R> c_pow(cplx<R> a, cplx<R> b) {
  if (a.re == 0 && a.im == 0) {
    if (b.re == 0 && b.im == 0) return {1, 0};
    return {0, 0};
  }
  return c_exp(b * c_log(a));
}

// ── integer helpers (nx_c_map.c:147-165) ────────────────────────────────────
__device__ inline int64_t ipow_s(int64_t base, int64_t e) {
  if (e < 0) return (base == 1) ? 1 : (base == -1) ? ((e & 1) ? -1 : 1) : 0;
  uint64_t b = (uint64_t)base, r = 1;
  while (e > 0) {
    if (e & 1) r *= b;
    e >>= 1;
    if (e) b *= b;
  }
  return (int64_t)r;
}
__device__ inline uint64_t ipow_u(uint64_t b, uint64_t e) {
  uint64_t r = 1;
  while (e > 0) {
    if (e & 1) r *= b;
    e >>= 1;
    if (e) b *= b;
  }
  return r;
}

constexpr bool cat_num(Cat c) { return c != CAT_BOOL; }                       // sint,uint,float,complex
constexpr bool cat_fc(Cat c) { return c == CAT_FLOAT || c == CAT_COMPLEX; }   // float,complex
constexpr bool cat_f(Cat c) { return c == CAT_FLOAT; }
constexpr bool cat_if(Cat c) { return c == CAT_SINT || c == CAT_UINT || c == CAT_FLOAT; }
constexpr bool cat_ord(Cat c) { return c != CAT_COMPLEX; }                    // sint,uint,float,bool
constexpr bool cat_bw(Cat c) { return c == CAT_SINT || c == CAT_UINT || c == CAT_BOOL; }
constexpr bool cat_all(Cat) { return true; }

// ── unary ops (nx_c_map.c:300-488) ──────────────────────────────────────────
struct OpNeg {
  static constexpr bool ok(Cat c) { return cat_num(c); }
  template <Cat cat, class C>
  __device__ __forceinline__ static C eval(C x) {
    if constexpr (cat == CAT_SINT) return (C)(-(uint64_t)x);
    else return -x;
  }
};
struct OpRecip {
  static constexpr bool ok(Cat c) { return cat_num(c); }
  template <Cat cat, class C>
  __device__ __forceinline__ static C eval(C x) {
    // integer 1/x is 1, -1 or 0; x == 0 gives 0
    if constexpr (cat == CAT_SINT) return x == 1 ? (C)1 : (x == -1 ? (C)-1 : (C)0);
    else if constexpr (cat == CAT_UINT) return x == 1 ? (C)1 : (C)0;
    else if constexpr (cat == CAT_COMPLEX) return C{1, 0} / x;
    else return (C)1 / x;
  }
};
struct OpAbs {
  static constexpr bool ok(Cat c) { return cat_num(c); }
  template <Cat cat, class C>
  __device__ __forceinline__ static C eval(C x) {
    if constexpr (cat == CAT_SINT) return x < 0 ? (C)(-(uint64_t)x) : x;
    else if constexpr (cat == CAT_UINT) return x;
    else if constexpr (cat == CAT_COMPLEX) return C{c_abs(x), 0};
    else return m_fabs(x);
  }
};
struct OpSign {
  static constexpr bool ok(Cat c) { return cat_num(c); }
  template <Cat cat, class C>
  __device__ __forceinline__ static C eval(C x) {
    if constexpr (cat == CAT_SINT) return (C)((x > 0) - (x < 0));
    else if constexpr (cat == CAT_UINT) return (C)(x != 0);
    else if constexpr (cat == CAT_COMPLEX) {
      auto m = c_abs(x);
      if (m == 0) return C{0, 0};
      return C{x.re / m, x.im / m};
    } else return (x != x) ? x : (C)((x > 0) - (x < 0));
  }
};
#define NXH_TRANS_OP(Name, fn)                                 \
  struct Name {                                                \
    static constexpr bool ok(Cat c) { return cat_fc(c); }      \
    template <Cat cat, class C>                                \
    __device__ __forceinline__ static C eval(C x) {            \
      if constexpr (cat == CAT_COMPLEX) return c_##fn(x);      \
      else return m_##fn(x);                                   \
    }                                                          \
  };
NXH_TRANS_OP(OpSqrt, sqrt)
NXH_TRANS_OP(OpExp, exp)
NXH_TRANS_OP(OpLog, log)
NXH_TRANS_OP(OpSin, sin)
NXH_TRANS_OP(OpCos, cos)
NXH_TRANS_OP(OpTan, tan)
NXH_TRANS_OP(OpAsin, asin)
NXH_TRANS_OP(OpAcos, acos)
NXH_TRANS_OP(OpAtan, atan)
NXH_TRANS_OP(OpSinh, sinh)
NXH_TRANS_OP(OpCosh, cosh)
NXH_TRANS_OP(OpTanh, tanh)
#define NXH_ROUND_OP(Name, fn)                                 \
  struct Name {                                                \
    static constexpr bool ok(Cat c) { return cat_if(c); }      \
    template <Cat cat, class C>                                \
    __device__ __forceinline__ static C eval(C x) {            \
      if constexpr (cat == CAT_FLOAT) return m_##fn(x);        \
      else return x;                                           \
    }                                                          \
  };
NXH_ROUND_OP(OpTrunc, trunc)
NXH_ROUND_OP(OpCeil, ceil)
NXH_ROUND_OP(OpFloor, floor)
NXH_ROUND_OP(OpRound, round)
struct OpErf {
  static constexpr bool ok(Cat c) { return cat_f(c); }
  template <Cat cat, class C>
  __device__ __forceinline__ static C eval(C x) { return m_erf(x); }
};

// ── binary ops (nx_c_map.c:494-695) ─────────────────────────────────────────
#define NXH_ARITH_OP(Name, sym)                                          \
  struct Name {                                                          \
    static constexpr bool ok(Cat c) { return cat_num(c); }               \
    template <Cat cat, class C>                                          \
    __device__ __forceinline__ static C eval(C a, C b) {                 \
      if constexpr (cat == CAT_SINT) return (C)((uint64_t)a sym(uint64_t) b); \
      else return a sym b;                                               \
    }                                                                    \
  };
NXH_ARITH_OP(OpAdd, +)
NXH_ARITH_OP(OpSub, -)
NXH_ARITH_OP(OpMul, *)
struct OpIdiv {
  static constexpr bool ok(Cat c) { return cat_if(c); }
  template <Cat cat, class C>
  __device__ __forceinline__ static C eval(C a, C b) {
    if constexpr (cat == CAT_SINT) return b == 0 ? (C)0 : (b == -1 ? (C)(-(uint64_t)a) : a / b);
    else if constexpr (cat == CAT_UINT) return b == 0 ? (C)0 : a / b;
    else return m_trunc(a / b);
  }
};
struct OpFdiv {
  static constexpr bool ok(Cat c) { return cat_fc(c); }
  template <Cat cat, class C>
  __device__ __forceinline__ static C eval(C a, C b) { return a / b; }
};
struct OpMod {
  static constexpr bool ok(Cat c) { return cat_if(c); }
  template <Cat cat, class C>
  __device__ __forceinline__ static C eval(C a, C b) {
    if constexpr (cat == CAT_SINT) return b == 0 ? (C)0 : (b == -1 ? (C)0 : a % b);
    else if constexpr (cat == CAT_UINT) return b == 0 ? (C)0 : a % b;
    else return m_fmod(a, b);
  }
};
#define NXH_MINMAX_OP(Name, sym)                                          \
  struct Name {                                                           \
    static constexpr bool ok(Cat c) { return cat_ord(c); }                \
    template <Cat cat, class C>                                           \
    __device__ __forceinline__ static C eval(C a, C b) {                  \
      if constexpr (cat == CAT_FLOAT)                                     \
        return (a != a || b != b) ? (C)__builtin_nanf("") : (a sym b ? a : b); \
      else return a sym b ? a : b;                                        \
    }                                                                     \
  };
NXH_MINMAX_OP(OpMax, >)
NXH_MINMAX_OP(OpMin, <)
struct OpPow {
  static constexpr bool ok(Cat c) { return cat_num(c); }
  template <Cat cat, class C>
  __device__ __forceinline__ static C eval(C a, C b) {
    if constexpr (cat == CAT_SINT) return (C)ipow_s(a, b);
    else if constexpr (cat == CAT_UINT) return (C)ipow_u((uint64_t)a, (uint64_t)b);
    else if constexpr (cat == CAT_COMPLEX) return c_pow(a, b);
    else return m_pow(a, b);
  }
};
struct OpAtan2 {
  static constexpr bool ok(Cat c) { return cat_f(c); }
  template <Cat cat, class C>
  __device__ __forceinline__ static C eval(C a, C b) { return m_atan2(a, b); }
};
#define NXH_BITWISE_OP(Name, sym)                                  \
  struct Name {                                                    \
    static constexpr bool ok(Cat c) { return cat_bw(c); }          \
    template <Cat cat, class C>                                    \
    __device__ __forceinline__ static C eval(C a, C b) { return (C)(a sym b); } \
  };
NXH_BITWISE_OP(OpXor, ^)
NXH_BITWISE_OP(OpOr, |)
NXH_BITWISE_OP(OpAnd, &)

// ── comparisons (nx_c_map.c:746-803) ────────────────────────────────────────
struct OpEq {
  static constexpr bool ok(Cat c) { return cat_all(c); }
  template <Cat cat, class C>
  __device__ __forceinline__ static bool eval(C a, C b) { return a == b; }
};
struct OpNe {
  static constexpr bool ok(Cat c) { return cat_all(c); }
  template <Cat cat, class C>
  __device__ __forceinline__ static bool eval(C a, C b) { return a != b; }
};
struct OpLt {
  static constexpr bool ok(Cat c) { return cat_ord(c); }
  template <Cat cat, class C>
  __device__ __forceinline__ static bool eval(C a, C b) { return a < b; }
};
struct OpLe {
  static constexpr bool ok(Cat c) { return cat_ord(c); }
  template <Cat cat, class C>
  __device__ __forceinline__ static bool eval(C a, C b) { return a <= b; }
};

// ── functors the kernels are instantiated on ────────────────────────────────
template <class OP, int DT>
struct UnaryF {
  using T = Tr<DT>;
  static constexpr int NIN = 1;
  using Out = typename T::S;
  using In0 = typename T::S;
  using In1 = Unused;
  using In2 = Unused;
  __device__ __forceinline__ static Out apply(In0 a) {
    if constexpr (std::is_same<OP, OpTanh>::value && (DT == NXH_BF16 || DT == NXH_F16)) return T::st(tanh_for_16bit(T::ld(a)));
    else return T::st(OP::template eval<T::cat, typename T::C>(T::ld(a)));
  }
};
template <class OP, int DT>
struct BinaryF {
  using T = Tr<DT>;
  static constexpr int NIN = 2;
  using Out = typename T::S;
  using In0 = typename T::S;
  using In1 = typename T::S;
  using In2 = Unused;
  __device__ __forceinline__ static Out apply(In0 a, In1 b) {
    return T::st(OP::template eval<T::cat, typename T::C>(T::ld(a), T::ld(b)));
  }
};
template <class OP, int DT>
struct CompareF {
  using T = Tr<DT>;
  static constexpr int NIN = 2;
  using Out = uint8_t;
  using In0 = typename T::S;
  using In1 = typename T::S;
  using In2 = Unused;
  __device__ __forceinline__ static Out apply(In0 a, In1 b) {
    return (uint8_t)OP::template eval<T::cat, typename T::C>(T::ld(a), T::ld(b));
  }
};

// Per-op dispatch row: a launcher per dtype, nullptr where the op has no
// meaning for the dtype's category.
struct MapRow {
  map_launch_fn fn[NXH_DTYPE_COUNT] = {};
};
template <template <class, int> class FUN, class OP>
struct MapRowOf : MapRow {
  template <int DT>
  void set() {
    if constexpr (OP::ok(Tr<DT>::cat)) fn[DT] = &map_launch<FUN<OP, DT>>;
  }
  MapRowOf() {
#define NXH_SET(DT) set<DT>();
    NXH_FOR_COMPUTE_DTYPES(NXH_SET)
#undef NXH_SET
  }
};
