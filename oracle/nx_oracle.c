/* nx_oracle.c — CPU restatement of the Nx C backend's hot path.

   TEST INFRASTRUCTURE ONLY. This file is the parity checker for libnxhip: the
   tests, the smoke check and the cpu_baseline leg of the benchmark call it;
   nothing in the product links, imports or executes it.

   Each function restates, in plain C, the algorithm of the reference file:line
   it cites (raven-ml/raven, packages/nx/lib/backend_c/ and packages/nx/lib/
   buffer/); paths below are relative to packages/nx/lib/.

   Pinning (what fixes each function independently of this file):
   - f16/bf16/fp8 converters: the reference's bit-pattern fixtures
     (packages/nx/test/fixtures/{f16,bf16}_bit_exact.safetensors), numpy's
     float16, and torch's bfloat16/float8 casts, exhaustively where the domain
     is 2^16 or 2^8 — tests/test_oracle_pins.py.
   - integer / compare / where / gather / cast: closed forms in numpy int64
     arithmetic with wrap, plus the reference tests' edge vectors
     (packages/nx/test/backend_contract.ml:1522-1601, 2437-2817).
   - float add/sub/mul/div/sqrt/rounding/max/min: IEEE-exact, numpy agrees bit
     for bit.
   - transcendentals: glibc libm, checked against numpy within the reference
     contract's tolerance (backend_contract.ml:159-168).
   - float sums: invariants the reference tests hold (2^25 ones in f32, 4096
     ones in f16, 512 ones in bf16 are exact; backend_contract.ml:2611-2644)
     and an f64 sum within k * eps.
   - matmul: f64 triple loop on the quantised inputs with the reference's
     tolerances (backend_c/test/matmul_test.ml:831-974) and its cancellation
     witness (matmul_test.ml:182-230).
   - pad / cat / scan / threefry / scatter / sort / argsort / unfold / fold: the
     reference tests' vectors (backend_contract.ml:1431-1457, 1661-1666,
     1727-1925, 2504-2580, 2782-2810; Random123's known answers for threefry)
     and numpy or brute-force statements of each (pad, concatenate, cumsum,
     stable sorts, a serial scatter walk, a direct im2col / col2im).
   Parity unpinned bit-for-bit (tolerance only, by the reference's own
   contract): the exact rounding of float sums, transcendental results and GEMM
   last bits. The value sort fixes the order of IEEE +0 / -0, which the
   reference leaves unspecified (nx_c_sort.c:262-292), to ascending original
   index. */

#include <complex.h>
#include <math.h>
#include <stdbool.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#include "../include/nxhip.h"

typedef float _Complex c32_t;
typedef double _Complex c64_t;

#define NXO_EXPORT __attribute__((visibility("default")))

static __thread const char *nxo_err = "";
NXO_EXPORT const char *nxo_last_error(void) { return nxo_err; }
static int fail(int kind, const char *msg) {
  nxo_err = msg;
  return kind;
}

/* ── storage converters (buffer/nx_buffer_stubs.h:70-302) ─────────────────── */

static inline uint32_t f2u(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}
static inline float u2f(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* nx_buffer_stubs.h:73-86: NaN keeps sign and top payload, forced quiet;
   otherwise round to nearest even on the dropped 16 bits. */
NXO_EXPORT uint16_t nxo_f32_to_bf16(float f) {
  uint32_t u = f2u(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
  uint32_t lsb = (u >> 16) & 1u;
  return (uint16_t)((u + 0x7fffu + lsb) >> 16);
}
/* nx_buffer_stubs.h:88-95 */
NXO_EXPORT float nxo_bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

/* nx_buffer_stubs.h:99-148: IEEE binary16, RNE, subnormals; a NaN carries its
   top 10 payload bits and is bumped to stay a NaN when they are all zero. */
NXO_EXPORT uint16_t nxo_f32_to_f16(float f) {
  uint32_t u = f2u(f);
  uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
  uint32_t e = (u >> 23) & 0xffu;
  uint32_t m = u & 0x7fffffu;
  if (e == 0xffu) {
    if (m == 0) return (uint16_t)(sign | 0x7c00u);
    uint16_t r = (uint16_t)(0x7c00u + (m >> 13));
    if (r == 0x7c00u) r++;
    return (uint16_t)(sign + r);
  }
  if (e >= 143u) return (uint16_t)(sign | 0x7c00u); /* >= 2^16: overflow */
  if (e <= 112u) {                                  /* < 2^-14: subnormal/zero */
    if (e < 102u) return sign;                      /* < 2^-25 */
    uint32_t full = m | 0x800000u;                  /* 24-bit significand */
    uint32_t shift = 126u - e;                      /* 14..24 */
    uint32_t q = full >> shift;
    uint32_t rem = full & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1u);
    if (rem > half || (rem == half && (q & 1u))) q++;
    return (uint16_t)(sign + q);
  }
  uint32_t q = ((e - 112u) << 10) | (m >> 13);
  uint32_t rem = m & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) q++; /* carry may reach inf */
  return (uint16_t)(sign + q);
}

/* nx_buffer_stubs.h:150-182: NaN is quieted (mantissa MSB set). */
NXO_EXPORT float nxo_f16_to_f32(uint16_t h) {
  uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
  uint32_t e = (h >> 10) & 0x1fu;
  uint32_t m = h & 0x3ffu;
  if (e == 0x1fu)
    return u2f(sign | 0x7f800000u | (m ? ((m << 13) | 0x400000u) : 0u));
  if (e == 0) {
    if (m == 0) return u2f(sign);
    int sh = 0;
    while (!(m & 0x400u)) {
      m <<= 1;
      sh++;
    }
    return u2f(sign | ((uint32_t)(113 - sh) << 23) | ((m & 0x3ffu) << 13));
  }
  return u2f(sign | ((e + 112u) << 23) | (m << 13));
}

/* Shared 8-bit encoder: `mbits` mantissa bits, exponent bias `bias`. */
static uint8_t f32_to_fp8_bits(float f, int mbits, int bias, uint32_t *out_bits) {
  uint32_t u = f2u(f);
  int exp = (int)((u >> 23) & 0xffu) - 127;
  int emin = 1 - bias;
  uint32_t q;
  if (exp >= emin) {
    uint32_t sig = u & 0x7fffffu;
    int drop = 23 - mbits;
    q = sig >> drop;
    uint32_t rem = sig & ((1u << drop) - 1u);
    uint32_t half = 1u << (drop - 1);
    if (rem > half || (rem == half && (q & 1u))) q++;
    *out_bits = ((uint32_t)(exp + bias) << mbits) + q;
    return 1;
  }
  uint32_t sig = (u & 0x7fffffu) | 0x800000u;
  int shift = (23 - mbits) + (emin - exp);
  if (shift > 24) {
    *out_bits = 0;
    return 1;
  }
  q = sig >> shift;
  uint32_t rem = sig & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1);
  if (rem > half || (rem == half && (q & 1u))) q++;
  *out_bits = q;
  return 1;
}

/* nx_buffer_stubs.h:189-223: e4m3fn — no infinities; NaN, inf and finite
   overflow past 448 all become S.1111.111. */
NXO_EXPORT uint8_t nxo_f32_to_f8e4m3(float f) {
  if (isnan(f)) return 0x7f;
  if (isinf(f)) return signbit(f) ? 0xff : 0x7f;
  uint8_t sign = (uint8_t)((f2u(f) >> 31) << 7);
  uint32_t bits;
  f32_to_fp8_bits(f, 3, 7, &bits);
  if (bits >= 0x7fu) return (uint8_t)(sign | 0x7f);
  return (uint8_t)(sign | bits);
}
/* nx_buffer_stubs.h:225-240 */
NXO_EXPORT float nxo_f8e4m3_to_f32(uint8_t v) {
  uint32_t e = (v >> 3) & 0xfu, m = v & 7u;
  if (e == 0xfu && m == 7u) return NAN;
  float r = e == 0 ? ldexpf((float)m, -9) : ldexpf(1.0f + (float)m / 8.0f, (int)e - 7);
  return (v & 0x80) ? -r : r;
}
/* nx_buffer_stubs.h:244-278: e5m2 — IEEE-like; NaN -> 0x7F, overflow -> inf. */
NXO_EXPORT uint8_t nxo_f32_to_f8e5m2(float f) {
  if (isnan(f)) return 0x7f;
  if (isinf(f)) return signbit(f) ? 0xfc : 0x7c;
  uint8_t sign = (uint8_t)((f2u(f) >> 31) << 7);
  uint32_t bits;
  f32_to_fp8_bits(f, 2, 15, &bits);
  if (bits >= 0x7cu) return (uint8_t)(sign | 0x7c);
  return (uint8_t)(sign | bits);
}
/* nx_buffer_stubs.h:280-302 */
NXO_EXPORT float nxo_f8e5m2_to_f32(uint8_t v) {
  uint32_t e = (v >> 2) & 0x1fu, m = v & 3u;
  bool neg = (v & 0x80) != 0;
  if (e == 0x1fu) {
    if (m == 0) return neg ? -INFINITY : INFINITY;
    return NAN;
  }
  float r;
  if (e == 0) {
    if (m == 0) return neg ? -0.0f : 0.0f;
    r = ldexpf((float)m / 4.0f, -14);
  } else {
    r = ldexpf(1.0f + (float)m / 4.0f, (int)e - 15);
  }
  return neg ? -r : r;
}

/* ── the dtype table (backend_c/nx_c.h:130-168) ─────────────────────────────
   X(tag, sfx, storage, compute, LD, ST, category)                           */
#define ID_(x) (x)
#define BOOLN_(x) ((x) != 0)
#define NXO_TABLE(X)                                                          \
  X(NXH_F16, f16, uint16_t, float, nxo_f16_to_f32, nxo_f32_to_f16, FLOAT)     \
  X(NXH_F32, f32, float, float, ID_, ID_, FLOAT)                              \
  X(NXH_F64, f64, double, double, ID_, ID_, FLOAT)                            \
  X(NXH_BF16, bf16, uint16_t, float, nxo_bf16_to_f32, nxo_f32_to_bf16, FLOAT) \
  X(NXH_F8E4M3, f8e4m3, uint8_t, float, nxo_f8e4m3_to_f32, nxo_f32_to_f8e4m3, \
    FLOAT)                                                                    \
  X(NXH_F8E5M2, f8e5m2, uint8_t, float, nxo_f8e5m2_to_f32, nxo_f32_to_f8e5m2, \
    FLOAT)                                                                    \
  X(NXH_I8, i8, int8_t, int64_t, ID_, ID_, SINT)                              \
  X(NXH_U8, u8, uint8_t, int64_t, ID_, ID_, UINT)                             \
  X(NXH_I16, i16, int16_t, int64_t, ID_, ID_, SINT)                           \
  X(NXH_U16, u16, uint16_t, int64_t, ID_, ID_, UINT)                          \
  X(NXH_I32, i32, int32_t, int64_t, ID_, ID_, SINT)                           \
  X(NXH_U32, u32, uint32_t, uint64_t, ID_, ID_, UINT)                         \
  X(NXH_I64, i64, int64_t, int64_t, ID_, ID_, SINT)                           \
  X(NXH_U64, u64, uint64_t, uint64_t, ID_, ID_, UINT)                         \
  X(NXH_C32, c32, c32_t, c32_t, ID_, ID_, COMPLEX)                            \
  X(NXH_C64, c64, c64_t, c64_t, ID_, ID_, COMPLEX)                            \
  X(NXH_BOOL, bool_, uint8_t, uint8_t, BOOLN_, BOOLN_, BOOL)

/* nx_c.h:219-226 */
#define LDST(tag, sfx, S, C, LD, ST, cat)                                     \
  static inline C ld_##sfx(const void *p) { return (C)(LD(*(const S *)p)); }  \
  static inline void st_##sfx(void *p, C v) { *(S *)p = (S)(ST(v)); }
NXO_TABLE(LDST)

static const int64_t elem_size_tab[NXH_DTYPE_COUNT] = {
    [NXH_F16] = 2, [NXH_F32] = 4, [NXH_F64] = 8, [NXH_BF16] = 2, [NXH_F8E4M3] = 1,
    [NXH_F8E5M2] = 1, [NXH_I4] = 0, [NXH_U4] = 0, [NXH_I8] = 1, [NXH_U8] = 1,
    [NXH_I16] = 2, [NXH_U16] = 2, [NXH_I32] = 4, [NXH_U32] = 4, [NXH_I64] = 8,
    [NXH_U64] = 8, [NXH_C32] = 8, [NXH_C64] = 16, [NXH_BOOL] = 1};
static bool is_packed(int dt) { return dt == NXH_I4 || dt == NXH_U4; }
NXO_EXPORT int64_t nxo_elem_size(int dt) {
  return (unsigned)dt < NXH_DTYPE_COUNT ? elem_size_tab[dt] : 0;
}

/* nx_c.h:234-250: saturating double -> integer storage. */
#define F2I_SINT(sfx, S)                                                      \
  static inline S f2i_##sfx(double v) {                                       \
    int w = (int)sizeof(S) * 8;                                               \
    double lim = ldexp(1.0, w - 1);                                           \
    if (isnan(v)) return 0;                                                   \
    if (v <= -lim) return (S)((uintmax_t)1 << (w - 1));                       \
    if (v >= lim) return (S)(((uintmax_t)1 << (w - 1)) - 1);                  \
    return (S)v;                                                              \
  }
#define F2I_UINT(sfx, S)                                                      \
  static inline S f2i_##sfx(double v) {                                       \
    double lim = ldexp(1.0, (int)sizeof(S) * 8);                              \
    if (isnan(v)) return 0;                                                   \
    if (v <= 0.0) return 0;                                                   \
    if (v >= lim) return (S)(~(uintmax_t)0);                                  \
    return (S)v;                                                              \
  }
#define F2I_FLOAT(sfx, S)
#define F2I_COMPLEX(sfx, S)
#define F2I_BOOL(sfx, S)
#define F2I_ROW(tag, sfx, S, C, LD, ST, cat) F2I_##cat(sfx, S)
NXO_TABLE(F2I_ROW)

/* ── kernels: one 1-D run, byte steps (nx_c.h:462-467) ──────────────────── */
typedef void map_fn(char *const *p, const int64_t *s, int64_t n);

#define MSUF_float(fn) fn##f
#define MSUF_double(fn) fn
#define MFN(fn, C) MSUF_##C(fn)

/* unary body generator */
#define UK(name, sfx, C, EXPR)                                                \
  static void name##_##sfx(char *const *p, const int64_t *s, int64_t n) {     \
    for (int64_t i = 0; i < n; i++) {                                         \
      C vx = ld_##sfx(p[1] + i * s[1]);                                       \
      st_##sfx(p[0] + i * s[0], (EXPR));                                      \
    }                                                                         \
  }
#define BK(name, sfx, C, EXPR)                                                \
  static void name##_##sfx(char *const *p, const int64_t *s, int64_t n) {     \
    for (int64_t i = 0; i < n; i++) {                                         \
      C va = ld_##sfx(p[1] + i * s[1]);                                       \
      C vb = ld_##sfx(p[2] + i * s[2]);                                       \
      st_##sfx(p[0] + i * s[0], (EXPR));                                      \
    }                                                                         \
  }
#define CK(name, sfx, C, EXPR)                                                \
  static void name##_##sfx(char *const *p, const int64_t *s, int64_t n) {     \
    for (int64_t i = 0; i < n; i++) {                                         \
      C va = ld_##sfx(p[1] + i * s[1]);                                       \
      C vb = ld_##sfx(p[2] + i * s[2]);                                       \
      *(uint8_t *)(p[0] + i * s[0]) = (uint8_t)(EXPR);                        \
    }                                                                         \
  }
#define NONE(...)

/* Per-category selectors: SEL_<cats>(cat) expands its argument for listed
   categories only. */
#define ON(...) __VA_ARGS__
#define OFF(...)

typedef struct {
  map_fn *fn[NXH_DTYPE_COUNT];
} map_table;

/* ---- unary (nx_c_map.c:300-488) ---- */
/* neg: signed in the unsigned width (nx_c_map.c:305-312) */
#define NEG_SINT(sfx, C) UK(neg, sfx, C, (C)(-(uint64_t)(vx)))
#define NEG_UINT(sfx, C) UK(neg, sfx, C, (-(vx)))
#define NEG_FLOAT(sfx, C) UK(neg, sfx, C, (-(vx)))
#define NEG_COMPLEX(sfx, C) UK(neg, sfx, C, (-(vx)))
#define NEG_BOOL(sfx, C)
#define NEG_ROW(tag, sfx, S, C, LD, ST, cat) NEG_##cat(sfx, C)
NXO_TABLE(NEG_ROW)
/* recip (nx_c_map.c:318-326) */
#define RECIP_SINT(sfx, C) UK(recip, sfx, C, ((vx) == 0 ? 0 : 1 / (vx)))
#define RECIP_UINT(sfx, C) UK(recip, sfx, C, ((vx) == 0 ? 0 : 1 / (vx)))
#define RECIP_FLOAT(sfx, C) UK(recip, sfx, C, ((C)1 / (vx)))
#define RECIP_COMPLEX(sfx, C) UK(recip, sfx, C, ((C)1 / (vx)))
#define RECIP_BOOL(sfx, C)
#define RECIP_ROW(tag, sfx, S, C, LD, ST, cat) RECIP_##cat(sfx, C)
NXO_TABLE(RECIP_ROW)
/* abs (nx_c_map.c:333-343) */
static inline float cabs_c32(c32_t z) { return cabsf(z); }
static inline double cabs_c64(c64_t z) { return cabs(z); }
#define ABS_SINT(sfx, C) UK(abs, sfx, C, ((vx) < 0 ? (C)(-(uint64_t)(vx)) : (vx)))
#define ABS_UINT(sfx, C) UK(abs, sfx, C, (vx))
#define ABS_FLOAT(sfx, C) UK(abs, sfx, C, MFN(fabs, C)(vx))
#define ABS_COMPLEX(sfx, C) UK(abs, sfx, C, (C)cabs_##sfx(vx))
#define ABS_BOOL(sfx, C)
#define ABS_ROW(tag, sfx, S, C, LD, ST, cat) ABS_##cat(sfx, C)
NXO_TABLE(ABS_ROW)
/* sign (nx_c_map.c:350-363) */
#define SIGN_SINT(sfx, C) UK(sign, sfx, C, (C)(((vx) > 0) - ((vx) < 0)))
#define SIGN_UINT(sfx, C) UK(sign, sfx, C, (C)((vx) != 0))
#define SIGN_FLOAT(sfx, C) \
  UK(sign, sfx, C, (isnan(vx) ? (vx) : (C)(((vx) > 0) - ((vx) < 0))))
#define SIGN_COMPLEX(sfx, C) \
  UK(sign, sfx, C, (cabs_##sfx(vx) == 0 ? (C)0 : (vx) / cabs_##sfx(vx)))
#define SIGN_BOOL(sfx, C)
#define SIGN_ROW(tag, sfx, S, C, LD, ST, cat) SIGN_##cat(sfx, C)
NXO_TABLE(SIGN_ROW)

/* transcendentals: float via libm, complex via c<fn> (nx_c_map.c:388-440) */
#define CFN_c32(fn) c##fn##f
#define CFN_c64(fn) c##fn
#define TR_FLOAT(op, sfx, C) UK(op, sfx, C, MFN(op, C)(vx))
#define TR_COMPLEX(op, sfx, C) UK(op, sfx, C, CFN_##sfx(op)(vx))
#define TR_SINT(op, sfx, C)
#define TR_UINT(op, sfx, C)
#define TR_BOOL(op, sfx, C)
/* The table macro cannot carry an extra argument, so each op spells its row. */
#define TR_ROW_sqrt(tag, sfx, S, C, LD, ST, cat) TR_##cat(sqrt, sfx, C)
#define TR_ROW_exp(tag, sfx, S, C, LD, ST, cat) TR_##cat(exp, sfx, C)
#define TR_ROW_log(tag, sfx, S, C, LD, ST, cat) TR_##cat(log, sfx, C)
#define TR_ROW_sin(tag, sfx, S, C, LD, ST, cat) TR_##cat(sin, sfx, C)
#define TR_ROW_cos(tag, sfx, S, C, LD, ST, cat) TR_##cat(cos, sfx, C)
#define TR_ROW_tan(tag, sfx, S, C, LD, ST, cat) TR_##cat(tan, sfx, C)
#define TR_ROW_asin(tag, sfx, S, C, LD, ST, cat) TR_##cat(asin, sfx, C)
#define TR_ROW_acos(tag, sfx, S, C, LD, ST, cat) TR_##cat(acos, sfx, C)
#define TR_ROW_atan(tag, sfx, S, C, LD, ST, cat) TR_##cat(atan, sfx, C)
#define TR_ROW_sinh(tag, sfx, S, C, LD, ST, cat) TR_##cat(sinh, sfx, C)
#define TR_ROW_cosh(tag, sfx, S, C, LD, ST, cat) TR_##cat(cosh, sfx, C)
#define TR_ROW_tanh(tag, sfx, S, C, LD, ST, cat) TR_##cat(tanh, sfx, C)
NXO_TABLE(TR_ROW_sqrt)
NXO_TABLE(TR_ROW_exp)
NXO_TABLE(TR_ROW_log)
NXO_TABLE(TR_ROW_sin)
NXO_TABLE(TR_ROW_cos)
NXO_TABLE(TR_ROW_tan)
NXO_TABLE(TR_ROW_asin)
NXO_TABLE(TR_ROW_acos)
NXO_TABLE(TR_ROW_atan)
NXO_TABLE(TR_ROW_sinh)
NXO_TABLE(TR_ROW_cosh)
NXO_TABLE(TR_ROW_tanh)
/* erf: float only (nx_c_map.c:442-456) */
#define ERF_FLOAT(sfx, C) UK(erf, sfx, C, MFN(erf, C)(vx))
#define ERF_SINT(sfx, C)
#define ERF_UINT(sfx, C)
#define ERF_COMPLEX(sfx, C)
#define ERF_BOOL(sfx, C)
#define ERF_ROW(tag, sfx, S, C, LD, ST, cat) ERF_##cat(sfx, C)
NXO_TABLE(ERF_ROW)
/* rounding: identity on ints, libm on floats (nx_c_map.c:458-488) */
#define RN_SINT(op, sfx, C) UK(op, sfx, C, (vx))
#define RN_UINT(op, sfx, C) UK(op, sfx, C, (vx))
#define RN_FLOAT(op, sfx, C) UK(op, sfx, C, MFN(op, C)(vx))
#define RN_COMPLEX(op, sfx, C)
#define RN_BOOL(op, sfx, C)
#define RN_ROW_trunc(tag, sfx, S, C, LD, ST, cat) RN_##cat(trunc, sfx, C)
#define RN_ROW_ceil(tag, sfx, S, C, LD, ST, cat) RN_##cat(ceil, sfx, C)
#define RN_ROW_floor(tag, sfx, S, C, LD, ST, cat) RN_##cat(floor, sfx, C)
#define RN_ROW_round(tag, sfx, S, C, LD, ST, cat) RN_##cat(round, sfx, C)
NXO_TABLE(RN_ROW_trunc)
NXO_TABLE(RN_ROW_ceil)
NXO_TABLE(RN_ROW_floor)
NXO_TABLE(RN_ROW_round)

/* table builders: which categories an op supports (nx_c_map.c:224-294) */
#define NUM_SINT(op, tag, sfx) T_(op, tag, sfx)
#define NUM_UINT(op, tag, sfx) T_(op, tag, sfx)
#define NUM_FLOAT(op, tag, sfx) T_(op, tag, sfx)
#define NUM_COMPLEX(op, tag, sfx) T_(op, tag, sfx)
#define NUM_BOOL(op, tag, sfx)
#define FC_SINT(op, tag, sfx)
#define FC_UINT(op, tag, sfx)
#define FC_FLOAT(op, tag, sfx) T_(op, tag, sfx)
#define FC_COMPLEX(op, tag, sfx) T_(op, tag, sfx)
#define FC_BOOL(op, tag, sfx)
#define FO_SINT(op, tag, sfx)
#define FO_UINT(op, tag, sfx)
#define FO_FLOAT(op, tag, sfx) T_(op, tag, sfx)
#define FO_COMPLEX(op, tag, sfx)
#define FO_BOOL(op, tag, sfx)
#define IF_SINT(op, tag, sfx) T_(op, tag, sfx)
#define IF_UINT(op, tag, sfx) T_(op, tag, sfx)
#define IF_FLOAT(op, tag, sfx) T_(op, tag, sfx)
#define IF_COMPLEX(op, tag, sfx)
#define IF_BOOL(op, tag, sfx)
#define MM_SINT(op, tag, sfx) T_(op, tag, sfx)
#define MM_UINT(op, tag, sfx) T_(op, tag, sfx)
#define MM_FLOAT(op, tag, sfx) T_(op, tag, sfx)
#define MM_COMPLEX(op, tag, sfx)
#define MM_BOOL(op, tag, sfx) T_(op, tag, sfx)
#define BW_SINT(op, tag, sfx) T_(op, tag, sfx)
#define BW_UINT(op, tag, sfx) T_(op, tag, sfx)
#define BW_FLOAT(op, tag, sfx)
#define BW_COMPLEX(op, tag, sfx)
#define BW_BOOL(op, tag, sfx) T_(op, tag, sfx)
#define AL_SINT(op, tag, sfx) T_(op, tag, sfx)
#define AL_UINT(op, tag, sfx) T_(op, tag, sfx)
#define AL_FLOAT(op, tag, sfx) T_(op, tag, sfx)
#define AL_COMPLEX(op, tag, sfx) T_(op, tag, sfx)
#define AL_BOOL(op, tag, sfx) T_(op, tag, sfx)

/* Because a row macro cannot take the op as an argument, tables are built with
   a current-op macro, redefined before each table. */
#define ROW_NUM(tag, sfx, S, C, LD, ST, cat) NUM_##cat(CUR, tag, sfx)
#define ROW_FC(tag, sfx, S, C, LD, ST, cat) FC_##cat(CUR, tag, sfx)
#define ROW_FO(tag, sfx, S, C, LD, ST, cat) FO_##cat(CUR, tag, sfx)
#define ROW_IF(tag, sfx, S, C, LD, ST, cat) IF_##cat(CUR, tag, sfx)
#define ROW_MM(tag, sfx, S, C, LD, ST, cat) MM_##cat(CUR, tag, sfx)
#define ROW_BW(tag, sfx, S, C, LD, ST, cat) BW_##cat(CUR, tag, sfx)
#define ROW_AL(tag, sfx, S, C, LD, ST, cat) AL_##cat(CUR, tag, sfx)
/* T_ pastes CUR after expansion through one more level */
#define T_(op, tag, sfx) T2_(op, tag, sfx)
#define T2_(op, tag, sfx) [tag] = op##_##sfx,

#define CUR neg
static const map_table t_neg = {.fn = {NXO_TABLE(ROW_NUM)}};
#undef CUR
#define CUR recip
static const map_table t_recip = {.fn = {NXO_TABLE(ROW_NUM)}};
#undef CUR
#define CUR abs
static const map_table t_abs = {.fn = {NXO_TABLE(ROW_NUM)}};
#undef CUR
#define CUR sign
static const map_table t_sign = {.fn = {NXO_TABLE(ROW_NUM)}};
#undef CUR
#define CUR sqrt
static const map_table t_sqrt = {.fn = {NXO_TABLE(ROW_FC)}};
#undef CUR
#define CUR exp
static const map_table t_exp = {.fn = {NXO_TABLE(ROW_FC)}};
#undef CUR
#define CUR log
static const map_table t_log = {.fn = {NXO_TABLE(ROW_FC)}};
#undef CUR
#define CUR sin
static const map_table t_sin = {.fn = {NXO_TABLE(ROW_FC)}};
#undef CUR
#define CUR cos
static const map_table t_cos = {.fn = {NXO_TABLE(ROW_FC)}};
#undef CUR
#define CUR tan
static const map_table t_tan = {.fn = {NXO_TABLE(ROW_FC)}};
#undef CUR
#define CUR asin
static const map_table t_asin = {.fn = {NXO_TABLE(ROW_FC)}};
#undef CUR
#define CUR acos
static const map_table t_acos = {.fn = {NXO_TABLE(ROW_FC)}};
#undef CUR
#define CUR atan
static const map_table t_atan = {.fn = {NXO_TABLE(ROW_FC)}};
#undef CUR
#define CUR sinh
static const map_table t_sinh = {.fn = {NXO_TABLE(ROW_FC)}};
#undef CUR
#define CUR cosh
static const map_table t_cosh = {.fn = {NXO_TABLE(ROW_FC)}};
#undef CUR
#define CUR tanh
static const map_table t_tanh = {.fn = {NXO_TABLE(ROW_FC)}};
#undef CUR
#define CUR trunc
static const map_table t_trunc = {.fn = {NXO_TABLE(ROW_IF)}};
#undef CUR
#define CUR ceil
static const map_table t_ceil = {.fn = {NXO_TABLE(ROW_IF)}};
#undef CUR
#define CUR floor
static const map_table t_floor = {.fn = {NXO_TABLE(ROW_IF)}};
#undef CUR
#define CUR round
static const map_table t_round = {.fn = {NXO_TABLE(ROW_IF)}};
#undef CUR
#define CUR erf
static const map_table t_erf = {.fn = {NXO_TABLE(ROW_FO)}};
#undef CUR

static const map_table *const unary_tables[NXH_UNARY_COUNT] = {
    [NXH_NEG] = &t_neg,     [NXH_RECIP] = &t_recip, [NXH_ABS] = &t_abs,
    [NXH_SIGN] = &t_sign,   [NXH_SQRT] = &t_sqrt,   [NXH_EXP] = &t_exp,
    [NXH_LOG] = &t_log,     [NXH_SIN] = &t_sin,     [NXH_COS] = &t_cos,
    [NXH_TAN] = &t_tan,     [NXH_ASIN] = &t_asin,   [NXH_ACOS] = &t_acos,
    [NXH_ATAN] = &t_atan,   [NXH_SINH] = &t_sinh,   [NXH_COSH] = &t_cosh,
    [NXH_TANH] = &t_tanh,   [NXH_TRUNC] = &t_trunc, [NXH_CEIL] = &t_ceil,
    [NXH_FLOOR] = &t_floor, [NXH_ROUND] = &t_round, [NXH_ERF] = &t_erf};
static const char *const unary_names[NXH_UNARY_COUNT] = {
    "neg",  "recip", "abs",  "sign", "sqrt", "exp",   "log",
    "sin",  "cos",   "tan",  "asin", "acos", "atan",  "sinh",
    "cosh", "tanh",  "trunc", "ceil", "floor", "round", "erf"};

/* ---- binary (nx_c_map.c:494-695) ---- */
/* add/sub/mul: signed forms in the unsigned width (nx_c_map.c:499-507) */
#define AR_SINT(op, sym, sfx, C) BK(op, sfx, C, (C)((uint64_t)(va)sym(uint64_t)(vb)))
#define AR_UINT(op, sym, sfx, C) BK(op, sfx, C, ((va)sym(vb)))
#define AR_FLOAT(op, sym, sfx, C) BK(op, sfx, C, ((va)sym(vb)))
#define AR_COMPLEX(op, sym, sfx, C) BK(op, sfx, C, ((va)sym(vb)))
#define AR_BOOL(op, sym, sfx, C)
#define ADD_ROW(tag, sfx, S, C, LD, ST, cat) AR_##cat(add, +, sfx, C)
#define SUB_ROW(tag, sfx, S, C, LD, ST, cat) AR_##cat(sub, -, sfx, C)
#define MUL_ROW(tag, sfx, S, C, LD, ST, cat) AR_##cat(mul, *, sfx, C)
NXO_TABLE(ADD_ROW)
NXO_TABLE(SUB_ROW)
NXO_TABLE(MUL_ROW)
/* idiv (nx_c_map.c:535-546) */
#define IDIV_SINT(sfx, C) \
  BK(idiv, sfx, C, ((vb) == 0 ? (C)0 : (vb) == -1 ? (C)(-(uint64_t)(va)) : (va) / (vb)))
#define IDIV_UINT(sfx, C) BK(idiv, sfx, C, ((vb) == 0 ? (C)0 : (va) / (vb)))
#define IDIV_FLOAT(sfx, C) BK(idiv, sfx, C, MFN(trunc, C)((va) / (vb)))
#define IDIV_COMPLEX(sfx, C)
#define IDIV_BOOL(sfx, C)
#define IDIV_ROW(tag, sfx, S, C, LD, ST, cat) IDIV_##cat(sfx, C)
NXO_TABLE(IDIV_ROW)
/* fdiv (nx_c_map.c:556-562) */
#define FDIV_FLOAT(sfx, C) BK(fdiv, sfx, C, ((va) / (vb)))
#define FDIV_COMPLEX(sfx, C) BK(fdiv, sfx, C, ((va) / (vb)))
#define FDIV_SINT(sfx, C)
#define FDIV_UINT(sfx, C)
#define FDIV_BOOL(sfx, C)
#define FDIV_ROW(tag, sfx, S, C, LD, ST, cat) FDIV_##cat(sfx, C)
NXO_TABLE(FDIV_ROW)
/* mod (nx_c_map.c:573-582) */
#define MOD_SINT(sfx, C) \
  BK(mod, sfx, C, ((vb) == 0 ? (C)0 : (vb) == -1 ? (C)0 : (va) % (vb)))
#define MOD_UINT(sfx, C) BK(mod, sfx, C, ((vb) == 0 ? (C)0 : (va) % (vb)))
#define MOD_FLOAT(sfx, C) BK(mod, sfx, C, MFN(fmod, C)(va, vb))
#define MOD_COMPLEX(sfx, C)
#define MOD_BOOL(sfx, C)
#define MOD_ROW(tag, sfx, S, C, LD, ST, cat) MOD_##cat(sfx, C)
NXO_TABLE(MOD_ROW)
/* max/min (nx_c_map.c:594-607): NaN-propagating on floats */
#define MX_SINT(op, sym, sfx, C) BK(op, sfx, C, ((va)sym(vb) ? (va) : (vb)))
#define MX_UINT(op, sym, sfx, C) BK(op, sfx, C, ((va)sym(vb) ? (va) : (vb)))
#define MX_BOOL(op, sym, sfx, C) BK(op, sfx, C, ((va)sym(vb) ? (va) : (vb)))
#define MX_FLOAT(op, sym, sfx, C) \
  BK(op, sfx, C, ((isnan(va) || isnan(vb)) ? (C)NAN : ((va)sym(vb) ? (va) : (vb))))
#define MX_COMPLEX(op, sym, sfx, C)
#define MAX_ROW(tag, sfx, S, C, LD, ST, cat) MX_##cat(max, >, sfx, C)
#define MIN_ROW(tag, sfx, S, C, LD, ST, cat) MX_##cat(min, <, sfx, C)
NXO_TABLE(MAX_ROW)
NXO_TABLE(MIN_ROW)
/* pow (nx_c_map.c:147-165, 629-638) */
static int64_t ipow_s(int64_t base, int64_t e) {
  if (e < 0) return (base == 1) ? 1 : (base == -1) ? ((e & 1) ? -1 : 1) : 0;
  uint64_t b = (uint64_t)base, r = 1;
  for (; e > 0; e >>= 1) {
    if (e & 1) r *= b;
    b *= b;
  }
  return (int64_t)r;
}
static uint64_t ipow_u(uint64_t b, uint64_t e) {
  uint64_t r = 1;
  for (; e > 0; e >>= 1) {
    if (e & 1) r *= b;
    b *= b;
  }
  return r;
}
#define POW_SINT(sfx, C) BK(pow, sfx, C, ipow_s((va), (vb)))
#define POW_UINT(sfx, C) BK(pow, sfx, C, ipow_u((va), (vb)))
#define POW_FLOAT(sfx, C) BK(pow, sfx, C, MFN(pow, C)((va), (vb)))
#define POW_COMPLEX(sfx, C) BK(pow, sfx, C, CFN_##sfx(pow)((va), (vb)))
#define POW_BOOL(sfx, C)
#define POW_ROW(tag, sfx, S, C, LD, ST, cat) POW_##cat(sfx, C)
NXO_TABLE(POW_ROW)
/* atan2 (nx_c_map.c:648-654) */
#define AT2_FLOAT(sfx, C) BK(atan2, sfx, C, MFN(atan2, C)((va), (vb)))
#define AT2_SINT(sfx, C)
#define AT2_UINT(sfx, C)
#define AT2_COMPLEX(sfx, C)
#define AT2_BOOL(sfx, C)
#define AT2_ROW(tag, sfx, S, C, LD, ST, cat) AT2_##cat(sfx, C)
NXO_TABLE(AT2_ROW)
/* xor/or/and (nx_c_map.c:665-672) */
#define BWK_SINT(op, sym, sfx, C) BK(op, sfx, C, ((va)sym(vb)))
#define BWK_UINT(op, sym, sfx, C) BK(op, sfx, C, ((va)sym(vb)))
#define BWK_BOOL(op, sym, sfx, C) BK(op, sfx, C, ((va)sym(vb)))
#define BWK_FLOAT(op, sym, sfx, C)
#define BWK_COMPLEX(op, sym, sfx, C)
#define XOR_ROW(tag, sfx, S, C, LD, ST, cat) BWK_##cat(xor, ^, sfx, C)
#define OR_ROW(tag, sfx, S, C, LD, ST, cat) BWK_##cat(or, |, sfx, C)
#define AND_ROW(tag, sfx, S, C, LD, ST, cat) BWK_##cat(and, &, sfx, C)
NXO_TABLE(XOR_ROW)
NXO_TABLE(OR_ROW)
NXO_TABLE(AND_ROW)

#define CUR add
static const map_table t_add = {.fn = {NXO_TABLE(ROW_NUM)}};
#undef CUR
#define CUR sub
static const map_table t_sub = {.fn = {NXO_TABLE(ROW_NUM)}};
#undef CUR
#define CUR mul
static const map_table t_mul = {.fn = {NXO_TABLE(ROW_NUM)}};
#undef CUR
#define CUR idiv
static const map_table t_idiv = {.fn = {NXO_TABLE(ROW_IF)}};
#undef CUR
#define CUR fdiv
static const map_table t_fdiv = {.fn = {NXO_TABLE(ROW_FC)}};
#undef CUR
#define CUR mod
static const map_table t_mod = {.fn = {NXO_TABLE(ROW_IF)}};
#undef CUR
#define CUR pow
static const map_table t_pow = {.fn = {NXO_TABLE(ROW_NUM)}};
#undef CUR
#define CUR atan2
static const map_table t_atan2 = {.fn = {NXO_TABLE(ROW_FO)}};
#undef CUR
#define CUR max
static const map_table t_max = {.fn = {NXO_TABLE(ROW_MM)}};
#undef CUR
#define CUR min
static const map_table t_min = {.fn = {NXO_TABLE(ROW_MM)}};
#undef CUR
#define CUR xor
static const map_table t_xor = {.fn = {NXO_TABLE(ROW_BW)}};
#undef CUR
#define CUR or
static const map_table t_or = {.fn = {NXO_TABLE(ROW_BW)}};
#undef CUR
#define CUR and
static const map_table t_and = {.fn = {NXO_TABLE(ROW_BW)}};
#undef CUR
static const map_table *const binary_tables[NXH_BINARY_COUNT] = {
    [NXH_ADD] = &t_add,   [NXH_SUB] = &t_sub,   [NXH_MUL] = &t_mul,
    [NXH_IDIV] = &t_idiv, [NXH_FDIV] = &t_fdiv, [NXH_MOD] = &t_mod,
    [NXH_POW] = &t_pow,   [NXH_ATAN2] = &t_atan2, [NXH_MAX] = &t_max,
    [NXH_MIN] = &t_min,   [NXH_XOR] = &t_xor,   [NXH_OR] = &t_or,
    [NXH_AND] = &t_and};
static const char *const binary_names[NXH_BINARY_COUNT] = {
    "add", "sub", "mul", "idiv", "fdiv", "mod", "pow",
    "atan2", "max", "min", "xor", "or", "and"};

/* ---- comparisons (nx_c_map.c:746-803) ---- */
#define CEQ_ROW(tag, sfx, S, C, LD, ST, cat) CK(cmpeq, sfx, C, ((va) == (vb)))
#define CNE_ROW(tag, sfx, S, C, LD, ST, cat) CK(cmpne, sfx, C, ((va) != (vb)))
NXO_TABLE(CEQ_ROW)
NXO_TABLE(CNE_ROW)
#define CO_SINT(op, sym, sfx, C) CK(op, sfx, C, ((va)sym(vb)))
#define CO_UINT(op, sym, sfx, C) CK(op, sfx, C, ((va)sym(vb)))
#define CO_FLOAT(op, sym, sfx, C) CK(op, sfx, C, ((va)sym(vb)))
#define CO_BOOL(op, sym, sfx, C) CK(op, sfx, C, ((va)sym(vb)))
#define CO_COMPLEX(op, sym, sfx, C)
#define CLT_ROW(tag, sfx, S, C, LD, ST, cat) CO_##cat(cmplt, <, sfx, C)
#define CLE_ROW(tag, sfx, S, C, LD, ST, cat) CO_##cat(cmple, <=, sfx, C)
NXO_TABLE(CLT_ROW)
NXO_TABLE(CLE_ROW)
#define CUR cmpeq
static const map_table t_cmpeq = {.fn = {NXO_TABLE(ROW_AL)}};
#undef CUR
#define CUR cmpne
static const map_table t_cmpne = {.fn = {NXO_TABLE(ROW_AL)}};
#undef CUR
#define CUR cmplt
static const map_table t_cmplt = {.fn = {NXO_TABLE(ROW_MM)}};
#undef CUR
#define CUR cmple
static const map_table t_cmple = {.fn = {NXO_TABLE(ROW_MM)}};
#undef CUR
static const map_table *const compare_tables[NXH_COMPARE_COUNT] = {
    &t_cmpeq, &t_cmpne, &t_cmplt, &t_cmple};
static const char *const compare_names[NXH_COMPARE_COUNT] = {"cmpeq", "cmpne",
                                                             "cmplt", "cmple"};

/* ---- where (nx_c_map.c:809-839): storage-typed select ---- */
#define WK(tag, sfx, S, C, LD, ST, cat)                                       \
  static void where_##sfx(char *const *p, const int64_t *s, int64_t n) {      \
    for (int64_t i = 0; i < n; i++) {                                         \
      uint8_t c = *(const uint8_t *)(p[1] + i * s[1]);                        \
      *(S *)(p[0] + i * s[0]) =                                               \
          c ? *(const S *)(p[2] + i * s[2]) : *(const S *)(p[3] + i * s[3]);  \
    }                                                                         \
  }
NXO_TABLE(WK)
#define CUR where
static const map_table t_where = {.fn = {NXO_TABLE(ROW_AL)}};
#undef CUR

/* ---- copy (nx_c_move.c:61-84) ---- */
#define CPK(tag, sfx, S, C, LD, ST, cat)                                      \
  static void copy_##sfx(char *const *p, const int64_t *s, int64_t n) {       \
    if (s[0] == (int64_t)sizeof(S) && s[1] == (int64_t)sizeof(S)) {           \
      memcpy(p[0], p[1], (size_t)n * sizeof(S));                              \
      return;                                                                 \
    }                                                                         \
    for (int64_t i = 0; i < n; i++)                                           \
      *(S *)(p[0] + i * s[0]) = *(const S *)(p[1] + i * s[1]);                \
  }
NXO_TABLE(CPK)
#define CUR copy
static const map_table t_copy = {.fn = {NXO_TABLE(ROW_AL)}};
#undef CUR

/* ---- cast matrix (nx_c_map.c:182-218, 1003-1044) ---- */
#define SREAL_SINT(v) (v)
#define SREAL_UINT(v) (v)
#define SREAL_FLOAT(v) (v)
#define SREAL_BOOL(v) (v)
#define SREAL_COMPLEX(v) creal(v)
#define TOINT_SINT(dsfx, v) (v)
#define TOINT_UINT(dsfx, v) (v)
#define TOINT_BOOL(dsfx, v) (v)
#define TOINT_FLOAT(dsfx, v) f2i_##dsfx((double)(v))
#define TOINT_COMPLEX(dsfx, v) f2i_##dsfx((double)creal(v))
#define CV_FLOAT(DC, dsfx, scat, v) ((DC)(SREAL_##scat(v)))
#define CV_COMPLEX(DC, dsfx, scat, v) ((DC)(v))
#define CV_BOOL(DC, dsfx, scat, v) ((DC)((v) != 0))
#define CV_SINT(DC, dsfx, scat, v) ((DC)(TOINT_##scat(dsfx, v)))
#define CV_UINT(DC, dsfx, scat, v) ((DC)(TOINT_##scat(dsfx, v)))

#define CAST_DST(X, ssfx, SC, scat)                                           \
  X(ssfx, SC, scat, f16, float, FLOAT)                                        \
  X(ssfx, SC, scat, f32, float, FLOAT)                                        \
  X(ssfx, SC, scat, f64, double, FLOAT)                                       \
  X(ssfx, SC, scat, bf16, float, FLOAT)                                       \
  X(ssfx, SC, scat, f8e4m3, float, FLOAT)                                     \
  X(ssfx, SC, scat, f8e5m2, float, FLOAT)                                     \
  X(ssfx, SC, scat, i8, int64_t, SINT)                                        \
  X(ssfx, SC, scat, u8, int64_t, UINT)                                        \
  X(ssfx, SC, scat, i16, int64_t, SINT)                                       \
  X(ssfx, SC, scat, u16, int64_t, UINT)                                       \
  X(ssfx, SC, scat, i32, int64_t, SINT)                                       \
  X(ssfx, SC, scat, u32, uint64_t, UINT)                                      \
  X(ssfx, SC, scat, i64, int64_t, SINT)                                       \
  X(ssfx, SC, scat, u64, uint64_t, UINT)                                      \
  X(ssfx, SC, scat, c32, c32_t, COMPLEX)                                      \
  X(ssfx, SC, scat, c64, c64_t, COMPLEX)                                      \
  X(ssfx, SC, scat, bool_, uint8_t, BOOL)
#define CAST_K(ssfx, SC, scat, dsfx, DC, dcat)                                \
  static void cast_##ssfx##_to_##dsfx(char *const *p, const int64_t *s,       \
                                      int64_t n) {                            \
    for (int64_t i = 0; i < n; i++) {                                         \
      SC vs = ld_##ssfx(p[1] + i * s[1]);                                     \
      st_##dsfx(p[0] + i * s[0], CV_##dcat(DC, dsfx, scat, vs));              \
    }                                                                         \
  }
#define CAST_SRC(tag, sfx, S, C, LD, ST, cat) CAST_DST(CAST_K, sfx, C, cat)
NXO_TABLE(CAST_SRC)
#define CAST_TE(ssfx, SC, scat, dsfx, DC, dcat) cast_##ssfx##_to_##dsfx,
/* dst order of CAST_DST -> dtype tags */
static const int cast_dst_tags[17] = {
    NXH_F16, NXH_F32, NXH_F64, NXH_BF16, NXH_F8E4M3, NXH_F8E5M2, NXH_I8, NXH_U8,
    NXH_I16, NXH_U16, NXH_I32, NXH_U32,  NXH_I64,    NXH_U64,    NXH_C32, NXH_C64,
    NXH_BOOL};
#define CAST_SRCROW(tag, sfx, S, C, LD, ST, cat) \
  [tag] = {CAST_DST(CAST_TE, sfx, C, cat)},
static map_fn *const cast_rows[NXH_DTYPE_COUNT][17] = {NXO_TABLE(CAST_SRCROW)};
static map_fn *cast_lookup(int src, int dst) {
  for (int j = 0; j < 17; j++)
    if (cast_dst_tags[j] == dst) return cast_rows[src][j];
  return NULL;
}

/* ── thread policy (nx_c_engine.c:480-520): bandwidth-class work stays serial
   below 16 Mi elements and otherwise uses bytes/32 MiB threads; compute-class
   work uses elems/64 Ki threads; both capped by the core count. */
static int ncores(void) {
#ifdef _OPENMP
  int n = omp_get_num_procs();
  return n > 64 ? 64 : (n < 1 ? 1 : n);
#else
  return 1;
#endif
}
static int g_force_threads = 0; /* 0 = policy */
NXO_EXPORT void nxo_set_threads(int n) { g_force_threads = n; }
static int g_last_threads = 1;
NXO_EXPORT int nxo_last_threads(void) { return g_last_threads; }
NXO_EXPORT int nxo_ncores(void) { return ncores(); }
enum { COST_BANDWIDTH, COST_COMPUTE, COST_HEAVY };
static int threads_for(int cls, int64_t runs, int64_t run_len, int64_t bytes) {
  int cores = ncores();
  if (g_force_threads > 0) return g_force_threads < cores ? g_force_threads : cores;
  int64_t elems = runs * run_len;
  int64_t want = 1;
  if (cls == COST_BANDWIDTH) {
    if (elems < ((int64_t)16 << 20)) return 1;
    want = bytes / ((int64_t)32 << 20);
  } else if (cls == COST_COMPUTE) {
    want = elems / ((int64_t)64 << 10);
  } else {
    want = runs;
  }
  if (want > cores) want = cores;
  if (want < 1) want = 1;
  return (int)want;
}

/* ── coalescing + map driver (nx_c_engine.c:542-590, 780-869) ───────────── */
#define MAXOP 4
typedef struct {
  int nop, ndim;
  int64_t shape[NXH_MAX_NDIM];
  int64_t bstride[MAXOP][NXH_MAX_NDIM];
  char *base[MAXOP];
  int64_t total;
} plan_t;

static void coalesce(const nxh_tensor *const *ops, int nop, const int64_t *es,
                     plan_t *p) {
  int ndim = ops[0]->ndim;
  p->nop = nop;
  p->total = 1;
  for (int i = 0; i < ndim; i++) p->total *= ops[0]->shape[i];
  for (int k = 0; k < nop; k++)
    p->base[k] = (char *)ops[k]->data + ops[k]->offset * es[k];
  int nd = 0;
  int64_t cst[MAXOP][NXH_MAX_NDIM];
  for (int i = 0; i < ndim; i++) {
    int64_t s = ops[0]->shape[i];
    if (s == 1) continue;
    bool merge = nd > 0;
    for (int k = 0; merge && k < nop; k++)
      if (cst[k][nd - 1] != ops[k]->strides[i] * s) merge = false;
    if (merge) {
      p->shape[nd - 1] *= s;
      for (int k = 0; k < nop; k++) cst[k][nd - 1] = ops[k]->strides[i];
    } else {
      p->shape[nd] = s;
      for (int k = 0; k < nop; k++) cst[k][nd] = ops[k]->strides[i];
      nd++;
    }
  }
  if (nd == 0) {
    p->shape[0] = 1;
    for (int k = 0; k < nop; k++) cst[k][0] = 0;
    nd = 1;
  }
  p->ndim = nd;
  for (int i = 0; i < nd; i++)
    for (int k = 0; k < nop; k++) p->bstride[k][i] = cst[k][i] * es[k];
}

#define ERR_OUT_ALIASED "output has a broadcast (zero) stride"
#define ERR_UNSUPPORTED "dtype not supported for this operation"
#define ERR_PACKED "packed dtype not supported for this operation"
#define ERR_SHAPE "shape mismatch"

static void run_range(const plan_t *p, map_fn *k, int64_t lo, int64_t hi) {
  /* [lo,hi) indexes runs of the innermost dim (or elements when rank 1) */
  if (p->ndim == 1) {
    char *ptr[MAXOP];
    int64_t st[MAXOP];
    for (int j = 0; j < p->nop; j++) {
      st[j] = p->bstride[j][0];
      ptr[j] = p->base[j] + lo * st[j];
    }
    k(ptr, st, hi - lo);
    return;
  }
  int od = p->ndim - 1;
  int64_t coord[NXH_MAX_NDIM];
  char *ptr[MAXOP];
  int64_t st[MAXOP];
  int64_t rem = lo;
  for (int j = 0; j < p->nop; j++) {
    ptr[j] = p->base[j];
    st[j] = p->bstride[j][od];
  }
  for (int d = od - 1; d >= 0; d--) {
    int64_t c = rem % p->shape[d];
    rem /= p->shape[d];
    coord[d] = c;
    for (int j = 0; j < p->nop; j++) ptr[j] += c * p->bstride[j][d];
  }
  for (int64_t it = lo; it < hi; it++) {
    char *rp[MAXOP];
    for (int j = 0; j < p->nop; j++) rp[j] = ptr[j];
    k(rp, st, p->shape[od]);
    for (int d = od - 1; d >= 0; d--) {
      if (++coord[d] < p->shape[d]) {
        for (int j = 0; j < p->nop; j++) ptr[j] += p->bstride[j][d];
        break;
      }
      coord[d] = 0;
      for (int j = 0; j < p->nop; j++) ptr[j] -= (p->shape[d] - 1) * p->bstride[j][d];
    }
  }
}

static int map_run(map_fn *k, int dt_for_err, int nin, const nxh_tensor *const *ops,
                   const int64_t *es, int cls) {
  if (k == NULL)
    return fail(NXH_FAILURE, is_packed(dt_for_err) ? ERR_PACKED : ERR_UNSUPPORTED);
  plan_t p;
  coalesce(ops, nin + 1, es, &p);
  if (p.total == 0) return NXH_OK;
  for (int i = 0; i < p.ndim; i++)
    if (p.shape[i] > 1 && p.bstride[0][i] == 0)
      return fail(NXH_INVALID_ARGUMENT, ERR_OUT_ALIASED);
  int64_t bytes = 0;
  for (int j = 0; j <= nin; j++) bytes += p.total * es[j];
  int64_t units, run_len;
  if (p.ndim == 1) {
    units = p.total;
    run_len = 1;
  } else {
    units = p.total / p.shape[p.ndim - 1];
    run_len = p.shape[p.ndim - 1];
  }
  int nth = p.ndim == 1 ? threads_for(cls, 1, p.total, bytes)
                        : threads_for(cls, units, run_len, bytes);
  if (nth > units) nth = (int)units;
  g_last_threads = nth;
  if (nth <= 1) {
    run_range(&p, k, 0, units);
  } else {
#pragma omp parallel for num_threads(nth) schedule(static)
    for (int t = 0; t < nth; t++) {
      int64_t lo = units * t / nth, hi = units * (t + 1) / nth;
      if (hi > lo) run_range(&p, k, lo, hi);
    }
  }
  return NXH_OK;
}

static int check_same_shape(const nxh_tensor *a, const nxh_tensor *b) {
  if (a->ndim != b->ndim) return 0;
  for (int i = 0; i < a->ndim; i++)
    if (a->shape[i] != b->shape[i]) return 0;
  return 1;
}

static const int unary_cost[NXH_UNARY_COUNT] = {
    [NXH_SQRT] = COST_COMPUTE, [NXH_EXP] = COST_COMPUTE,  [NXH_LOG] = COST_COMPUTE,
    [NXH_SIN] = COST_COMPUTE,  [NXH_COS] = COST_COMPUTE,  [NXH_TAN] = COST_COMPUTE,
    [NXH_ASIN] = COST_COMPUTE, [NXH_ACOS] = COST_COMPUTE, [NXH_ATAN] = COST_COMPUTE,
    [NXH_SINH] = COST_COMPUTE, [NXH_COSH] = COST_COMPUTE, [NXH_TANH] = COST_COMPUTE,
    [NXH_ERF] = COST_COMPUTE};
static const int binary_cost[NXH_BINARY_COUNT] = {
    [NXH_IDIV] = COST_COMPUTE, [NXH_FDIV] = COST_COMPUTE, [NXH_MOD] = COST_COMPUTE,
    [NXH_POW] = COST_COMPUTE,  [NXH_ATAN2] = COST_COMPUTE};

/* caml_nx_c_<unary> (nx_c_map.c:1184-1204) through nx_c_map_funnel
   (nx_c_engine.c:1362-1384): dispatch on the output dtype. */
NXO_EXPORT int nxo_unary(int op, const nxh_tensor *out, const nxh_tensor *x) {
  if ((unsigned)op >= NXH_UNARY_COUNT) return fail(NXH_FAILURE, "bad op");
  (void)unary_names;
  if (!check_same_shape(out, x)) return fail(NXH_INVALID_ARGUMENT, ERR_SHAPE);
  const nxh_tensor *ops[2] = {out, x};
  int64_t es[2] = {nxo_elem_size(out->dtype), nxo_elem_size(x->dtype)};
  if (es[0] == 0 || es[1] == 0) return fail(NXH_FAILURE, ERR_PACKED);
  return map_run(unary_tables[op]->fn[out->dtype], out->dtype, 1, ops, es,
                 unary_cost[op]);
}
NXO_EXPORT int nxo_binary(int op, const nxh_tensor *out, const nxh_tensor *x,
                          const nxh_tensor *y) {
  if ((unsigned)op >= NXH_BINARY_COUNT) return fail(NXH_FAILURE, "bad op");
  (void)binary_names;
  if (!check_same_shape(out, x) || !check_same_shape(out, y))
    return fail(NXH_INVALID_ARGUMENT, ERR_SHAPE);
  const nxh_tensor *ops[3] = {out, x, y};
  int64_t es[3] = {nxo_elem_size(out->dtype), nxo_elem_size(x->dtype),
                   nxo_elem_size(y->dtype)};
  if (es[0] == 0 || es[1] == 0 || es[2] == 0) return fail(NXH_FAILURE, ERR_PACKED);
  return map_run(binary_tables[op]->fn[out->dtype], out->dtype, 2, ops, es,
                 binary_cost[op]);
}
/* nx_c_map.c:1231-1245: dispatch on the INPUT dtype. */
NXO_EXPORT int nxo_compare(int op, const nxh_tensor *out, const nxh_tensor *x,
                           const nxh_tensor *y) {
  if ((unsigned)op >= NXH_COMPARE_COUNT) return fail(NXH_FAILURE, "bad op");
  (void)compare_names;
  if (!check_same_shape(out, x) || !check_same_shape(out, y))
    return fail(NXH_INVALID_ARGUMENT, ERR_SHAPE);
  const nxh_tensor *ops[3] = {out, x, y};
  int64_t es[3] = {nxo_elem_size(out->dtype), nxo_elem_size(x->dtype),
                   nxo_elem_size(x->dtype)};
  return map_run(compare_tables[op]->fn[x->dtype], x->dtype, 2, ops, es,
                 COST_BANDWIDTH);
}
NXO_EXPORT int nxo_where(const nxh_tensor *out, const nxh_tensor *cond,
                         const nxh_tensor *a, const nxh_tensor *b) {
  if (!check_same_shape(out, cond) || !check_same_shape(out, a) ||
      !check_same_shape(out, b))
    return fail(NXH_INVALID_ARGUMENT, ERR_SHAPE);
  const nxh_tensor *ops[4] = {out, cond, a, b};
  int64_t es[4] = {nxo_elem_size(out->dtype), 1, nxo_elem_size(a->dtype),
                   nxo_elem_size(b->dtype)};
  if (es[0] == 0) return fail(NXH_FAILURE, ERR_PACKED);
  return map_run(t_where.fn[out->dtype], out->dtype, 3, ops, es, COST_BANDWIDTH);
}
static bool dense_off0(const nxh_tensor *a) {
  if (a->offset != 0) return false;
  int64_t e = 1;
  for (int i = a->ndim - 1; i >= 0; i--) {
    if (a->shape[i] == 1) continue;
    if (a->strides[i] != e) return false;
    e *= a->shape[i];
  }
  return true;
}
/* caml_nx_c_copy (nx_c_move.c:191-201); packed dtypes: whole contiguous
   offset-0 buffers only, the odd trailing nibble merged (nx_c_move.c:143-189) */
NXO_EXPORT int nxo_copy(const nxh_tensor *out, const nxh_tensor *x) {
  if (is_packed(out->dtype)) {
    int64_t n = 1, nx = 1;
    for (int i = 0; i < out->ndim; i++) n *= out->shape[i];
    for (int i = 0; i < x->ndim; i++) nx *= x->shape[i];
    if (n != nx || !dense_off0(out) || !dense_off0(x)) return fail(NXH_FAILURE, ERR_PACKED);
    memcpy(out->data, x->data, (size_t)(n / 2));
    if (n & 1) {
      uint8_t *d = (uint8_t *)out->data + n / 2;
      const uint8_t *sp = (const uint8_t *)x->data + n / 2;
      *d = (uint8_t)((*d & 0xF0) | (*sp & 0x0F));
    }
    return NXH_OK;
  }
  if (!check_same_shape(out, x)) return fail(NXH_INVALID_ARGUMENT, ERR_SHAPE);
  const nxh_tensor *ops[2] = {out, x};
  int64_t es[2] = {nxo_elem_size(out->dtype), nxo_elem_size(x->dtype)};
  if (es[0] == 0) return fail(NXH_FAILURE, ERR_PACKED);
  return map_run(t_copy.fn[out->dtype], out->dtype, 1, ops, es, COST_BANDWIDTH);
}

/* packed int4/uint4 casts (nx_c_map.c:1046-1177): dense layouts only */
static bool dense(const nxh_tensor *a) {
  int64_t e = 1;
  for (int i = a->ndim - 1; i >= 0; i--) {
    if (a->shape[i] == 1) continue;
    if (a->strides[i] != e) return false;
    e *= a->shape[i];
  }
  return true;
}
static int f2i4_s(double v) {
  if (isnan(v)) return 0;
  if (v <= -8.0) return -8;
  if (v >= 7.0) return 7;
  return (int)v;
}
static int f2i4_u(double v) {
  if (isnan(v)) return 0;
  if (v <= 0.0) return 0;
  if (v >= 15.0) return 15;
  return (int)v;
}
static int cast_packed(const nxh_tensor *out, const nxh_tensor *x) {
  if (!dense(out) || !dense(x)) return fail(NXH_FAILURE, ERR_PACKED);
  int64_t n = 1;
  for (int i = 0; i < out->ndim; i++) n *= out->shape[i];
  int src = x->dtype, dst = out->dtype;
  bool sp = is_packed(src), dp = is_packed(dst);
  for (int64_t i = 0; i < n; i++) {
    /* value of source element i as (int64 | double | is_float) */
    int64_t iv = 0;
    double fv = 0;
    bool isf = false;
    if (sp) {
      int64_t si = x->offset + i;
      uint8_t by = ((const uint8_t *)x->data)[si >> 1];
      if (src == NXH_I4)
        iv = (si & 1) ? ((int8_t)by >> 4) : ((int8_t)((by & 0x0f) << 4) >> 4);
      else
        iv = (si & 1) ? (by >> 4) : (by & 0x0f);
      if (dp) iv &= 0x0f;
    } else {
      const char *sp_ = (const char *)x->data + (x->offset + i) * nxo_elem_size(src);
      switch (src) {
#define RD_SINT(sfx) iv = (int64_t)ld_##sfx(sp_);
#define RD_UINT(sfx) iv = (int64_t)ld_##sfx(sp_);
#define RD_BOOL(sfx) iv = (int64_t)ld_##sfx(sp_);
#define RD_FLOAT(sfx) \
  fv = (double)ld_##sfx(sp_); \
  isf = true;
#define RD_COMPLEX(sfx) \
  fv = (double)creal(ld_##sfx(sp_)); \
  isf = true;
#define RD_ROW(tag, sfx, S, C, LD, ST, cat) \
  case tag: {                               \
    RD_##cat(sfx)                           \
  } break;
        NXO_TABLE(RD_ROW)
        default:
          return fail(NXH_FAILURE, ERR_UNSUPPORTED);
      }
    }
    if (dp) {
      int nibv = isf ? (dst == NXH_I4 ? f2i4_s(fv) : f2i4_u(fv)) : (int)iv;
      uint8_t nib = (uint8_t)nibv & 0x0f;
      int64_t di = out->offset + i;
      uint8_t *bp = &((uint8_t *)out->data)[di >> 1];
      *bp = (di & 1) ? (uint8_t)((*bp & 0x0f) | (nib << 4)) : (uint8_t)((*bp & 0xf0) | nib);
    } else {
      /* packed src -> compute dst: the nibble is a small signed/unsigned int */
      char *dp_ = (char *)out->data + (out->offset + i) * nxo_elem_size(dst);
      switch (dst) {
#define WR_ROW(tag, sfx, S, C, LD, ST, cat)                    \
  case tag:                                                    \
    st_##sfx(dp_, CV_##cat(C, sfx, SINT, iv));                 \
    break;
        NXO_TABLE(WR_ROW)
        default:
          return fail(NXH_FAILURE, ERR_UNSUPPORTED);
      }
    }
  }
  return NXH_OK;
}

/* caml_nx_c_cast (nx_c_map.c:1261-1280) */
NXO_EXPORT int nxo_cast(const nxh_tensor *out, const nxh_tensor *x) {
  if (!check_same_shape(out, x)) return fail(NXH_INVALID_ARGUMENT, ERR_SHAPE);
  if ((unsigned)out->dtype >= NXH_DTYPE_COUNT || (unsigned)x->dtype >= NXH_DTYPE_COUNT)
    return fail(NXH_FAILURE, "unsupported bigarray kind");
  if (is_packed(out->dtype) || is_packed(x->dtype)) return cast_packed(out, x);
  const nxh_tensor *ops[2] = {out, x};
  int64_t es[2] = {nxo_elem_size(out->dtype), nxo_elem_size(x->dtype)};
  return map_run(cast_lookup(x->dtype, out->dtype), out->dtype, 1, ops, es,
                 COST_BANDWIDTH);
}

/* full: Nx_buffer.fill on a fresh contiguous tensor (nx_backend.ml:61-64) */
NXO_EXPORT int nxo_fill(const nxh_tensor *out, const void *value) {
  int64_t es = nxo_elem_size(out->dtype);
  if (es == 0) return fail(NXH_FAILURE, ERR_PACKED);
  nxh_tensor src = *out;
  src.data = (void *)value;
  src.offset = 0;
  for (int i = 0; i < src.ndim; i++) src.strides[i] = 0;
  return nxo_copy(out, &src);
}

/* ── fold family (nx_c_fold.c, driver nx_c_engine.c:893-1170) ────────────── */
typedef union {
  int64_t i;
  uint64_t u;
  float f;
  double d;
  c32_t c32;
  c64_t c64;
} acc_t;
#define ACCF_float f
#define ACCF_double d
#define ACCF_int64_t i
#define ACCF_uint64_t u
#define ACCF_uint8_t i
#define ACCF_c32_t c32
#define ACCF_c64_t c64
#define ACC_(C) ACCF_##C
#define ACC(a, C) ((a)->ACC_(C))

typedef void fold_init(acc_t *);
typedef void fold_step(acc_t *, const char *in, int64_t step, int64_t n);
typedef void fold_fini(char *out, const acc_t *);
typedef void fold_stream(void *accs, const char *in, int64_t step, int64_t n, int first);
typedef void fold_scatter(char *out, int64_t step, const void *accs, int64_t n);

/* combine rules (nx_c_fold.c:63-91) */
#define CMB_SUM(M, V) (M) += (V)
#define CMB_PROD(M, V) (M) *= (V)
#define CMB_SUMW(M, V) (M) = (int64_t)((uint64_t)(M) + (uint64_t)(V))
#define CMB_PRODW(M, V) (M) = (int64_t)((uint64_t)(M) * (uint64_t)(V))
#define CMB_MAXI(M, V) \
  if ((V) > (M)) (M) = (V)
#define CMB_MINI(M, V) \
  if ((V) < (M)) (M) = (V)
#define CMB_MAXF(M, V) \
  if ((V) > (M))       \
    (M) = (V);         \
  else if ((V) != (V)) \
  (M) = (V)
#define CMB_MINF(M, V) \
  if ((V) < (M))       \
    (M) = (V);         \
  else if ((V) != (V)) \
  (M) = (V)
#define CMB_MAXB(M, V) (M) |= (V)
#define CMB_MINB(M, V) (M) &= (V)

/* single accumulator step (nx_c_fold.c:110-129) and stream step (:207-233) */
#define RSTEP(op, sfx, C, CMB)                                                 \
  static void op##_step_##sfx(acc_t *a, const char *in, int64_t st, int64_t n) { \
    C m = ACC(a, C);                                                           \
    for (int64_t k = 0; k < n; k++) {                                          \
      C v = ld_##sfx(in + k * st);                                             \
      CMB(m, v);                                                               \
    }                                                                          \
    ACC(a, C) = m;                                                             \
  }                                                                            \
  static void op##_stream_##sfx(void *accs, const char *in, int64_t st,        \
                                int64_t n, int first) {                        \
    C *a = (C *)accs;                                                          \
    if (first) {                                                               \
      for (int64_t j = 0; j < n; j++) a[j] = ld_##sfx(in + j * st);            \
    } else {                                                                   \
      for (int64_t j = 0; j < n; j++) {                                        \
        C v = ld_##sfx(in + j * st);                                           \
        CMB(a[j], v);                                                          \
      }                                                                        \
    }                                                                          \
  }
/* float sum: 16 partials on a unit-stride run, fixed balanced tree
   (nx_c_fold.c:139-159); its stream form is the single per-lane accumulator */
#define FSUM(sfx, S, C)                                                        \
  static void sum_step_##sfx(acc_t *a, const char *in, int64_t st, int64_t n) { \
    C s[16];                                                                   \
    for (int i = 0; i < 16; i++) s[i] = 0;                                     \
    int64_t k = 0;                                                             \
    if (st == (int64_t)sizeof(S)) {                                            \
      const S *p = (const S *)in;                                              \
      for (; k + 16 <= n; k += 16)                                             \
        for (int i = 0; i < 16; i++) s[i] += ld_##sfx(&p[k + i]);              \
      for (; k < n; k++) s[0] += ld_##sfx(&p[k]);                              \
    } else {                                                                   \
      for (; k < n; k++) s[0] += ld_##sfx(in + k * st);                        \
    }                                                                          \
    C lo = ((s[0] + s[1]) + (s[2] + s[3])) + ((s[4] + s[5]) + (s[6] + s[7]));  \
    C hi = ((s[8] + s[9]) + (s[10] + s[11])) + ((s[12] + s[13]) + (s[14] + s[15])); \
    ACC(a, C) += lo + hi;                                                      \
  }                                                                            \
  static void sum_stream_##sfx(void *accs, const char *in, int64_t st,         \
                               int64_t n, int first) {                         \
    C *a = (C *)accs;                                                          \
    if (first) {                                                               \
      for (int64_t j = 0; j < n; j++) a[j] = ld_##sfx(in + j * st);            \
    } else {                                                                   \
      for (int64_t j = 0; j < n; j++) a[j] += ld_##sfx(in + j * st);           \
    }                                                                          \
  }

#define SUM_FLOAT(sfx, S, C) FSUM(sfx, S, C)
#define SUM_SINT(sfx, S, C) RSTEP(sum, sfx, C, CMB_SUMW)
#define SUM_UINT(sfx, S, C) RSTEP(sum, sfx, C, CMB_SUM)
#define SUM_COMPLEX(sfx, S, C) RSTEP(sum, sfx, C, CMB_SUM)
#define SUM_BOOL(sfx, S, C)
#define SUM_ROW(tag, sfx, S, C, LD, ST, cat) SUM_##cat(sfx, S, C)
NXO_TABLE(SUM_ROW)
#define PROD_FLOAT(sfx, S, C) RSTEP(prod, sfx, C, CMB_PROD)
#define PROD_SINT(sfx, S, C) RSTEP(prod, sfx, C, CMB_PRODW)
#define PROD_UINT(sfx, S, C) RSTEP(prod, sfx, C, CMB_PROD)
#define PROD_COMPLEX(sfx, S, C) RSTEP(prod, sfx, C, CMB_PROD)
#define PROD_BOOL(sfx, S, C)
#define PROD_ROW(tag, sfx, S, C, LD, ST, cat) PROD_##cat(sfx, S, C)
NXO_TABLE(PROD_ROW)
#define RMAX_FLOAT(sfx, S, C) RSTEP(rmax, sfx, C, CMB_MAXF)
#define RMAX_SINT(sfx, S, C) RSTEP(rmax, sfx, C, CMB_MAXI)
#define RMAX_UINT(sfx, S, C) RSTEP(rmax, sfx, C, CMB_MAXI)
#define RMAX_BOOL(sfx, S, C) RSTEP(rmax, sfx, C, CMB_MAXB)
#define RMAX_COMPLEX(sfx, S, C)
#define RMAX_ROW(tag, sfx, S, C, LD, ST, cat) RMAX_##cat(sfx, S, C)
NXO_TABLE(RMAX_ROW)
#define RMIN_FLOAT(sfx, S, C) RSTEP(rmin, sfx, C, CMB_MINF)
#define RMIN_SINT(sfx, S, C) RSTEP(rmin, sfx, C, CMB_MINI)
#define RMIN_UINT(sfx, S, C) RSTEP(rmin, sfx, C, CMB_MINI)
#define RMIN_BOOL(sfx, S, C) RSTEP(rmin, sfx, C, CMB_MINB)
#define RMIN_COMPLEX(sfx, S, C)
#define RMIN_ROW(tag, sfx, S, C, LD, ST, cat) RMIN_##cat(sfx, S, C)
NXO_TABLE(RMIN_ROW)

/* init (nx_c_fold.c:262-314) with the sentinels of :54-61, fini/scatter (:240-258) */
#define MAXSENT_float (-INFINITY)
#define MAXSENT_double (-INFINITY)
#define MAXSENT_int64_t INT64_MIN
#define MAXSENT_uint64_t 0
#define MAXSENT_uint8_t 0
#define MINSENT_float INFINITY
#define MINSENT_double INFINITY
#define MINSENT_int64_t INT64_MAX
#define MINSENT_uint64_t UINT64_MAX
#define MINSENT_uint8_t 1
#define MAXSENT_c32_t 0
#define MAXSENT_c64_t 0
#define MINSENT_c32_t 0
#define MINSENT_c64_t 0
#define INITS(tag, sfx, S, C, LD, ST, cat)                                     \
  static void init0_##sfx(acc_t *a) { ACC(a, C) = 0; }                         \
  static void init1_##sfx(acc_t *a) { ACC(a, C) = 1; }                         \
  static void initmax_##sfx(acc_t *a) { ACC(a, C) = MAXSENT_##C; }             \
  static void initmin_##sfx(acc_t *a) { ACC(a, C) = MINSENT_##C; }             \
  static void fini_##sfx(char *out, const acc_t *a) { st_##sfx(out, (C)ACC(a, C)); } \
  static void scatter_##sfx(char *out, int64_t st, const void *accs, int64_t n) { \
    const C *a = (const C *)accs;                                              \
    for (int64_t j = 0; j < n; j++) st_##sfx(out + j * st, a[j]);              \
  }
NXO_TABLE(INITS)

typedef struct {
  fold_init *init[NXH_DTYPE_COUNT];
  fold_step *step[NXH_DTYPE_COUNT];
  fold_fini *fini[NXH_DTYPE_COUNT];
  fold_stream *stream[NXH_DTYPE_COUNT];
  fold_scatter *scatter[NXH_DTYPE_COUNT];
  int64_t acc_size[NXH_DTYPE_COUNT];
} fold_table;

#define AR_ON_SINT 1
#define AR_ON_UINT 1
#define AR_ON_FLOAT 1
#define AR_ON_COMPLEX 1
#define AR_ON_BOOL 0
#define OR_ON_SINT 1
#define OR_ON_UINT 1
#define OR_ON_FLOAT 1
#define OR_ON_COMPLEX 0
#define OR_ON_BOOL 1
#define SLOT_0(f, tag, v)
#define SLOT_1(f, tag, v) .f[tag] = v,
#define SLOT_P(on, f, tag, v) SLOT_P2(on, f, tag, v)
#define SLOT_P2(on, f, tag, v) SLOT_##on(f, tag, v)
#define FT_ROW(SUP, INIT, OP, tag, sfx, C, cat)                                \
  SLOT_P(SUP##_##cat, init, tag, INIT##_##sfx)                                 \
  SLOT_P(SUP##_##cat, step, tag, OP##_step_##sfx)                              \
  SLOT_P(SUP##_##cat, fini, tag, fini_##sfx)                                   \
  SLOT_P(SUP##_##cat, stream, tag, OP##_stream_##sfx)                          \
  SLOT_P(SUP##_##cat, scatter, tag, scatter_##sfx)                             \
  SLOT_P(SUP##_##cat, acc_size, tag, (int64_t)sizeof(C))
#define FT_SUM(tag, sfx, S, C, LD, ST, cat) FT_ROW(AR_ON, init0, sum, tag, sfx, C, cat)
#define FT_PROD(tag, sfx, S, C, LD, ST, cat) FT_ROW(AR_ON, init1, prod, tag, sfx, C, cat)
#define FT_MAX(tag, sfx, S, C, LD, ST, cat) FT_ROW(OR_ON, initmax, rmax, tag, sfx, C, cat)
#define FT_MIN(tag, sfx, S, C, LD, ST, cat) FT_ROW(OR_ON, initmin, rmin, tag, sfx, C, cat)
static const fold_table ft_sum = {NXO_TABLE(FT_SUM)};
static const fold_table ft_prod = {NXO_TABLE(FT_PROD)};
static const fold_table ft_max = {NXO_TABLE(FT_MAX)};
static const fold_table ft_min = {NXO_TABLE(FT_MIN)};
static const fold_table *const fold_tables[NXH_REDUCE_COUNT] = {&ft_sum, &ft_prod,
                                                                &ft_max, &ft_min};

typedef struct {
  int nk, nr;
  int64_t kshape[NXH_MAX_NDIM], kin[NXH_MAX_NDIM], kout[NXH_MAX_NDIM];
  int64_t rshape[NXH_MAX_NDIM], rin[NXH_MAX_NDIM];
  char *in_base, *out_base;
} fold_geom;

static void seek2(int nk, const int64_t *shape, const int64_t *si, const int64_t *so,
                  int64_t idx, int64_t *coord, char *ib, char *ob, char **ip,
                  char **op) {
  for (int d = nk - 1; d >= 0; d--) {
    int64_t c = idx % shape[d];
    idx /= shape[d];
    coord[d] = c;
    ib += c * si[d];
    ob += c * so[d];
  }
  *ip = ib;
  *op = ob;
}
static void next2(int nk, const int64_t *shape, const int64_t *si, const int64_t *so,
                  int64_t *coord, char **ip, char **op) {
  for (int d = nk - 1; d >= 0; d--) {
    if (++coord[d] < shape[d]) {
      *ip += si[d];
      *op += so[d];
      return;
    }
    coord[d] = 0;
    *ip -= (shape[d] - 1) * si[d];
    *op -= (shape[d] - 1) * so[d];
  }
}

/* one output element (nx_c_engine.c:893-920) */
static void reduce_one(const fold_geom *g, const fold_table *t, int dt, char *ip,
                       char *op) {
  acc_t acc;
  t->init[dt](&acc);
  if (g->nr == 0) {
    t->step[dt](&acc, ip, 0, 1);
  } else {
    int rod = g->nr - 1;
    int64_t outer = 1;
    for (int d = 0; d < rod; d++) outer *= g->rshape[d];
    int64_t rc[NXH_MAX_NDIM] = {0};
    char *rp = ip;
    for (int64_t o = 0; o < outer; o++) {
      t->step[dt](&acc, rp, g->rin[rod], g->rshape[rod]);
      for (int d = rod - 1; d >= 0; d--) {
        if (++rc[d] < g->rshape[d]) {
          rp += g->rin[d];
          break;
        }
        rc[d] = 0;
        rp -= (g->rshape[d] - 1) * g->rin[d];
      }
    }
  }
  t->fini[dt](op, &acc);
}

#define ERR_AXES "reduce axes must be strictly increasing and in range"
#define ERR_OUT_RANK "output rank inconsistent with the operation"
#define ERR_AXIS "axis out of range"
#define ERR_EMPTY "reduction over empty axis has no identity"

/* nx_c_engine.c:1392-1420 */
static int squeeze_out(const nxh_tensor *in, const nxh_tensor *out, const int32_t *axes,
                       int nred, nxh_tensor *sq) {
  if (nred < 0 || nred > in->ndim) return fail(NXH_INVALID_ARGUMENT, ERR_AXES);
  bool red[NXH_MAX_NDIM] = {false};
  for (int i = 0; i < nred; i++) {
    int a = axes[i];
    if (a < 0 || a >= in->ndim || red[a]) return fail(NXH_INVALID_ARGUMENT, ERR_AXES);
    red[a] = true;
  }
  int kept = in->ndim - nred;
  *sq = *out;
  if (out->ndim == kept) return NXH_OK;
  if (out->ndim != in->ndim) return fail(NXH_INVALID_ARGUMENT, ERR_OUT_RANK);
  sq->ndim = kept;
  int j = 0;
  for (int a = 0; a < in->ndim; a++)
    if (!red[a]) {
      sq->shape[j] = out->shape[a];
      sq->strides[j] = out->strides[a];
      j++;
    }
  return NXH_OK;
}

/* caml_nx_c_reduce_* (nx_c_fold.c:824-831) -> nx_c_fold_run
   (nx_c_engine.c:1052-1170) */
NXO_EXPORT int nxo_reduce(int op, const nxh_tensor *out_full, const nxh_tensor *in,
                          const int32_t *axes, int nred) {
  if ((unsigned)op >= NXH_REDUCE_COUNT) return fail(NXH_FAILURE, "bad op");
  const fold_table *t = fold_tables[op];
  int dt = in->dtype;
  if ((unsigned)dt >= NXH_DTYPE_COUNT) return fail(NXH_FAILURE, "unsupported bigarray kind");
  nxh_tensor out;
  int rc = squeeze_out(in, out_full, axes, nred, &out);
  if (rc) return rc;
  if (t->init[dt] == NULL)
    return fail(NXH_FAILURE, is_packed(dt) ? ERR_PACKED : ERR_UNSUPPORTED);
  int64_t ie = nxo_elem_size(dt), oe = nxo_elem_size(out.dtype);
  fold_geom g;
  g.in_base = (char *)in->data + in->offset * ie;
  g.out_base = (char *)out.data + out.offset * oe;
  g.nk = g.nr = 0;
  int ra = 0;
  for (int a = 0; a < in->ndim; a++) {
    if (ra < nred && axes[ra] == a) {
      g.rshape[g.nr] = in->shape[a];
      g.rin[g.nr++] = in->strides[a] * ie;
      ra++;
    } else {
      g.kshape[g.nk] = in->shape[a];
      g.kin[g.nk++] = in->strides[a] * ie;
    }
  }
  if (ra != nred) return fail(NXH_INVALID_ARGUMENT, ERR_AXES);
  if (out.ndim != g.nk) return fail(NXH_INVALID_ARGUMENT, ERR_OUT_RANK);
  for (int j = 0; j < g.nk; j++) g.kout[j] = out.strides[j] * oe;
  int64_t out_total = 1, rlen = 1;
  for (int d = 0; d < g.nk; d++) out_total *= g.kshape[d];
  if (out_total == 0) return NXH_OK;
  for (int d = 0; d < g.nr; d++) rlen *= g.rshape[d];
  bool no_identity = (op == NXH_RMAX || op == NXH_RMIN);
  if (no_identity && rlen == 0) return fail(NXH_INVALID_ARGUMENT, ERR_EMPTY);
  int64_t bytes = out_total * rlen * ie;

  /* streaming decision (nx_c_engine.c:1116-1149) */
  if (g.nk >= 1 && g.nr >= 1 && rlen >= 1) {
    int lane = -1;
    for (int j = 0; j < g.nk; j++) {
      if (g.kshape[j] <= 1) continue;
      if (lane < 0 || llabs(g.kin[j]) < llabs(g.kin[lane])) lane = j;
    }
    if (lane >= 0) {
      int64_t rs = llabs(g.rin[0]);
      for (int d = 1; d < g.nr; d++)
        if (llabs(g.rin[d]) < rs) rs = llabs(g.rin[d]);
      if (llabs(g.kin[lane]) < rs) {
        int64_t lane_len = g.kshape[lane], panels = out_total / lane_len;
        int nth = threads_for(COST_BANDWIDTH, panels, lane_len * rlen, bytes);
        if (nth > panels) nth = (int)panels;
        if (nth < 1) nth = 1;
        int64_t scratch = (int64_t)nth * lane_len * (int64_t)sizeof(acc_t);
        if (scratch <= ((int64_t)64 << 20)) {
          int np = 0;
          int64_t ps[NXH_MAX_NDIM], pin[NXH_MAX_NDIM], pout[NXH_MAX_NDIM];
          for (int j = 0; j < g.nk; j++) {
            if (j == lane) continue;
            ps[np] = g.kshape[j];
            pin[np] = g.kin[j];
            pout[np++] = g.kout[j];
          }
          g_last_threads = nth;
          char *all = malloc((size_t)scratch);
          if (!all) return fail(NXH_FAILURE, "out of memory");
#pragma omp parallel for num_threads(nth) schedule(static)
          for (int w = 0; w < nth; w++) {
            int64_t lo = panels * w / nth, hi = panels * (w + 1) / nth;
            void *accs = all + (int64_t)w * lane_len * (int64_t)sizeof(acc_t);
            int64_t coord[NXH_MAX_NDIM];
            char *ip, *op_;
            seek2(np, ps, pin, pout, lo, coord, g.in_base, g.out_base, &ip, &op_);
            for (int64_t it = lo; it < hi; it++) {
              int64_t rcd[NXH_MAX_NDIM] = {0};
              char *rp = ip;
              for (int64_t r = 0; r < rlen; r++) {
                t->stream[dt](accs, rp, g.kin[lane], lane_len, r == 0);
                for (int d = g.nr - 1; d >= 0; d--) {
                  if (++rcd[d] < g.rshape[d]) {
                    rp += g.rin[d];
                    break;
                  }
                  rcd[d] = 0;
                  rp -= (g.rshape[d] - 1) * g.rin[d];
                }
              }
              t->scatter[dt](op_, g.kout[lane], accs, lane_len);
              next2(np, ps, pin, pout, coord, &ip, &op_);
            }
          }
          free(all);
          return NXH_OK;
        }
      }
    }
  }
  /* per-output path: smallest-|stride| reduced axis becomes the run
     (nx_c_engine.c:1151-1169) */
  if (g.nr > 1) {
    int best = 0;
    for (int r = 1; r < g.nr; r++)
      if (llabs(g.rin[r]) < llabs(g.rin[best])) best = r;
    int last = g.nr - 1;
    int64_t ts = g.rshape[best];
    g.rshape[best] = g.rshape[last];
    g.rshape[last] = ts;
    ts = g.rin[best];
    g.rin[best] = g.rin[last];
    g.rin[last] = ts;
  }
  int nth = threads_for(COST_BANDWIDTH, out_total, rlen, bytes);
  if (nth > out_total) nth = (int)out_total;
  g_last_threads = nth;
#pragma omp parallel for num_threads(nth) schedule(static)
  for (int w = 0; w < nth; w++) {
    int64_t lo = out_total * w / nth, hi = out_total * (w + 1) / nth;
    int64_t coord[NXH_MAX_NDIM];
    char *ip, *op_;
    seek2(g.nk, g.kshape, g.kin, g.kout, lo, coord, g.in_base, g.out_base, &ip, &op_);
    for (int64_t it = lo; it < hi; it++) {
      reduce_one(&g, t, dt, ip, op_);
      next2(g.nk, g.kshape, g.kin, g.kout, coord, &ip, &op_);
    }
  }
  return NXH_OK;
}

/* argmax/argmin step (nx_c_fold.c:93-101, 180-198): strict compare keeps the
   earliest index; the first NaN wins */
#define ACMP_MAXI(V, B) ((V) > (B))
#define ACMP_MINI(V, B) ((V) < (B))
#define ACMP_MAXF(V, B) (((V) > (B)) || (((V) != (V)) && !((B) != (B))))
#define ACMP_MINF(V, B) (((V) < (B)) || (((V) != (V)) && !((B) != (B))))
typedef int64_t arg_fn(const char *in, int64_t st, int64_t n);
#define ARGK(op, sfx, C, ACMP)                                                 \
  static int64_t op##_##sfx(const char *in, int64_t st, int64_t n) {           \
    int64_t idx = -1;                                                          \
    C best = 0;                                                                \
    for (int64_t k = 0; k < n; k++) {                                          \
      C v = ld_##sfx(in + k * st);                                             \
      if (idx < 0 || ACMP(v, best)) {                                          \
        best = v;                                                              \
        idx = k;                                                               \
      }                                                                        \
    }                                                                          \
    return idx;                                                                \
  }
#define AMAX_FLOAT(sfx, C) ARGK(argmax, sfx, C, ACMP_MAXF)
#define AMAX_SINT(sfx, C) ARGK(argmax, sfx, C, ACMP_MAXI)
#define AMAX_UINT(sfx, C) ARGK(argmax, sfx, C, ACMP_MAXI)
#define AMAX_BOOL(sfx, C) ARGK(argmax, sfx, C, ACMP_MAXI)
#define AMAX_COMPLEX(sfx, C)
#define AMAX_ROW(tag, sfx, S, C, LD, ST, cat) AMAX_##cat(sfx, C)
NXO_TABLE(AMAX_ROW)
#define AMIN_FLOAT(sfx, C) ARGK(argmin, sfx, C, ACMP_MINF)
#define AMIN_SINT(sfx, C) ARGK(argmin, sfx, C, ACMP_MINI)
#define AMIN_UINT(sfx, C) ARGK(argmin, sfx, C, ACMP_MINI)
#define AMIN_BOOL(sfx, C) ARGK(argmin, sfx, C, ACMP_MINI)
#define AMIN_COMPLEX(sfx, C)
#define AMIN_ROW(tag, sfx, S, C, LD, ST, cat) AMIN_##cat(sfx, C)
NXO_TABLE(AMIN_ROW)
#define AT_ROW_MAX(tag, sfx, S, C, LD, ST, cat) SLOT_P(OR_ON_##cat, fn, tag, argmax_##sfx)
#define AT_ROW_MIN(tag, sfx, S, C, LD, ST, cat) SLOT_P(OR_ON_##cat, fn, tag, argmin_##sfx)
typedef struct {
  arg_fn *fn[NXH_DTYPE_COUNT];
} arg_table;
static const arg_table at_max = {NXO_TABLE(AT_ROW_MAX)};
static const arg_table at_min = {NXO_TABLE(AT_ROW_MIN)};

/* caml_nx_c_arg{max,min} -> nx_c_argreduce_run (nx_c_engine.c:1177-1254) */
NXO_EXPORT int nxo_argreduce(int is_min, const nxh_tensor *out_full,
                             const nxh_tensor *in, int axis) {
  int dt = in->dtype;
  if ((unsigned)dt >= NXH_DTYPE_COUNT) return fail(NXH_FAILURE, "unsupported bigarray kind");
  nxh_tensor out;
  int32_t ax32 = axis;
  int rc = squeeze_out(in, out_full, &ax32, 1, &out);
  if (rc) return rc;
  arg_fn *fn = (is_min ? at_min : at_max).fn[dt];
  if (!fn) return fail(NXH_FAILURE, is_packed(dt) ? ERR_PACKED : ERR_UNSUPPORTED);
  if (axis < 0 || axis >= in->ndim) return fail(NXH_INVALID_ARGUMENT, ERR_AXIS);
  if (out.ndim != in->ndim - 1) return fail(NXH_INVALID_ARGUMENT, ERR_OUT_RANK);
  int64_t alen = in->shape[axis];
  if (alen == 0) return fail(NXH_INVALID_ARGUMENT, ERR_EMPTY);
  if (alen > INT32_MAX) return fail(NXH_FAILURE, "argreduce axis length exceeds INT32_MAX");
  int64_t ie = nxo_elem_size(dt);
  int nk = 0;
  int64_t ks[NXH_MAX_NDIM], kin[NXH_MAX_NDIM], kout[NXH_MAX_NDIM];
  for (int a = 0; a < in->ndim; a++) {
    if (a == axis) continue;
    ks[nk] = in->shape[a];
    kin[nk] = in->strides[a] * ie;
    kout[nk] = out.strides[nk] * 4;
    nk++;
  }
  int64_t total = 1;
  for (int d = 0; d < nk; d++) total *= ks[d];
  if (total == 0) return NXH_OK;
  int64_t bytes = total * alen * ie;
  int nth = threads_for(COST_BANDWIDTH, total, alen, bytes);
  if (nth > total) nth = (int)total;
  g_last_threads = nth;
  char *ib = (char *)in->data + in->offset * ie;
  char *ob = (char *)out.data + out.offset * 4;
  int64_t ast = in->strides[axis] * ie;
#pragma omp parallel for num_threads(nth) schedule(static)
  for (int w = 0; w < nth; w++) {
    int64_t lo = total * w / nth, hi = total * (w + 1) / nth;
    int64_t coord[NXH_MAX_NDIM];
    char *ip, *op_;
    seek2(nk, ks, kin, kout, lo, coord, ib, ob, &ip, &op_);
    for (int64_t it = lo; it < hi; it++) {
      *(int32_t *)op_ = (int32_t)fn(ip, ast, alen);
      next2(nk, ks, kin, kout, coord, &ip, &op_);
    }
  }
  return NXH_OK;
}

/* ── matmul (nx_c_matmul.c:874-1108; arithmetic :197-209, 347-361, 424-440):
   every output element is the k-ordered sum of products in the compute type,
   stored once. For k > 2048 the reference sums 512-deep blocks separately and
   adds the partial tiles (nx_c_matmul.c:79-101), which this restates. */
#define MM_KC 512
#define MM_KC_FULLK_MAX 2048
#define MAC_SINT(acc, x, y) (acc) = (int64_t)((uint64_t)(acc) + (uint64_t)(x) * (uint64_t)(y))
#define MAC_UINT(acc, x, y) (acc) += (x) * (y)
#define MAC_FLOAT(acc, x, y) (acc) += (x) * (y)
#define MAC_COMPLEX(acc, x, y) (acc) += (x) * (y)
#define ADDC_SINT(a, b) ((int64_t)((uint64_t)(a) + (uint64_t)(b)))
#define ADDC_UINT(a, b) ((a) + (b))
#define ADDC_FLOAT(a, b) ((a) + (b))
#define ADDC_COMPLEX(a, b) ((a) + (b))
typedef void mm_fn(const char *a, int64_t ars, int64_t acs, const char *b, int64_t brs,
                   int64_t bcs, char *c, int64_t crs, int64_t ccs, int64_t m,
                   int64_t n, int64_t k, int blocked);
#define MMK(cat, sfx, S, C)                                                    \
  static void mm_##sfx(const char *a, int64_t ars, int64_t acs, const char *b, \
                       int64_t brs, int64_t bcs, char *c, int64_t crs,         \
                       int64_t ccs, int64_t m, int64_t n, int64_t k,           \
                       int blocked) {                                          \
    const int64_t es = (int64_t)sizeof(S);                                     \
    _Pragma("omp parallel for schedule(static)") for (int64_t i = 0; i < m; i++) { \
      C *row = malloc(sizeof(C) * (size_t)(n > 0 ? n : 1));                    \
      C *part = malloc(sizeof(C) * (size_t)(n > 0 ? n : 1));                   \
      for (int64_t j = 0; j < n; j++) row[j] = (C)0;                           \
      int64_t kc = (blocked && k > MM_KC_FULLK_MAX) ? MM_KC : (k > 0 ? k : 1); \
      for (int64_t p0 = 0; p0 < k; p0 += kc) {                                 \
        int64_t p1 = p0 + kc < k ? p0 + kc : k;                                \
        for (int64_t j = 0; j < n; j++) part[j] = (C)0;                        \
        for (int64_t p = p0; p < p1; p++) {                                    \
          C av = ld_##sfx(a + (i * ars + p * acs) * es);                       \
          for (int64_t j = 0; j < n; j++) {                                    \
            C bv = ld_##sfx(b + (p * brs + j * bcs) * es);                     \
            MAC_##cat(part[j], av, bv);                                        \
          }                                                                    \
        }                                                                      \
        if (p0 == 0 && p1 == k) {                                              \
          for (int64_t j = 0; j < n; j++) row[j] = part[j];                    \
        } else {                                                               \
          for (int64_t j = 0; j < n; j++) row[j] = (C)ADDC_##cat(row[j], part[j]); \
        }                                                                      \
      }                                                                        \
      for (int64_t j = 0; j < n; j++) st_##sfx(c + (i * crs + j * ccs) * es, row[j]); \
      free(row);                                                               \
      free(part);                                                              \
    }                                                                          \
  }
#define MM_SINT_(sfx, S, C) MMK(SINT, sfx, S, C)
#define MM_UINT_(sfx, S, C) MMK(UINT, sfx, S, C)
#define MM_FLOAT_(sfx, S, C) MMK(FLOAT, sfx, S, C)
#define MM_COMPLEX_(sfx, S, C) MMK(COMPLEX, sfx, S, C)
#define MM_BOOL_(sfx, S, C)
#define MM_ROW(tag, sfx, S, C, LD, ST, cat) MM_##cat##_(sfx, S, C)
NXO_TABLE(MM_ROW)
typedef struct {
  mm_fn *fn[NXH_DTYPE_COUNT];
} mm_table;
#define MMT_ROW(tag, sfx, S, C, LD, ST, cat) SLOT_P(AR_ON_##cat, fn, tag, mm_##sfx)
static const mm_table mmt = {NXO_TABLE(MMT_ROW)};

NXO_EXPORT int nxo_matmul(const nxh_tensor *C, const nxh_tensor *A, const nxh_tensor *B) {
  if (A->dtype != B->dtype || A->dtype != C->dtype)
    return fail(NXH_FAILURE, "matmul operands must share one dtype");
  int dt = A->dtype;
  if ((unsigned)dt >= NXH_DTYPE_COUNT) return fail(NXH_FAILURE, "unsupported bigarray kind");
  mm_fn *fn = mmt.fn[dt];
  if (!fn) return fail(NXH_FAILURE, is_packed(dt) ? ERR_PACKED : ERR_UNSUPPORTED);
  if (A->ndim < 2 || B->ndim < 2) return fail(NXH_INVALID_ARGUMENT, ERR_SHAPE);
  int nd = A->ndim > B->ndim ? A->ndim : B->ndim;
  if (C->ndim != nd) return fail(NXH_INVALID_ARGUMENT, ERR_SHAPE);
  int64_t m = A->shape[A->ndim - 2], k = A->shape[A->ndim - 1];
  int64_t kk = B->shape[B->ndim - 2], n = B->shape[B->ndim - 1];
  if (k != kk || C->shape[nd - 2] != m || C->shape[nd - 1] != n)
    return fail(NXH_INVALID_ARGUMENT, ERR_SHAPE);
  int bnd = nd - 2;
  int64_t bs[NXH_MAX_NDIM], as_[NXH_MAX_NDIM], bs_[NXH_MAX_NDIM], cs_[NXH_MAX_NDIM];
  int abo = nd - A->ndim, bbo = nd - B->ndim;
  int64_t nbatch = 1;
  for (int i = 0; i < bnd; i++) {
    int64_t sa = 1, sb = 1, sta = 0, stb = 0;
    if (i >= abo) {
      sa = A->shape[i - abo];
      sta = A->strides[i - abo];
    }
    if (i >= bbo) {
      sb = B->shape[i - bbo];
      stb = B->strides[i - bbo];
    }
    if (sa != sb && sa != 1 && sb != 1) return fail(NXH_INVALID_ARGUMENT, ERR_SHAPE);
    int64_t s = sa > sb ? sa : sb;
    if (C->shape[i] != s) return fail(NXH_INVALID_ARGUMENT, ERR_SHAPE);
    bs[i] = s;
    as_[i] = sa == 1 ? 0 : sta;
    bs_[i] = sb == 1 ? 0 : stb;
    cs_[i] = C->strides[i];
    if (s > 1 && cs_[i] == 0) return fail(NXH_INVALID_ARGUMENT, ERR_OUT_ALIASED);
    nbatch *= s;
  }
  if (m == 0 || n == 0 || nbatch == 0) return NXH_OK;
  int64_t ars = A->strides[A->ndim - 2], acs = A->strides[A->ndim - 1];
  int64_t brs = B->strides[B->ndim - 2], bcs = B->strides[B->ndim - 1];
  int64_t crs = C->strides[nd - 2], ccs = C->strides[nd - 1];
  if ((m > 1 && crs == 0) || (n > 1 && ccs == 0))
    return fail(NXH_INVALID_ARGUMENT, ERR_OUT_ALIASED);
  int64_t es = nxo_elem_size(dt);
  /* the direct triple loop never KC-blocks (nx_c_matmul.c:412-440, 964-965):
     MR = 8, NR = 12 (f32 family) / 4 (f64) / 8 (int, complex) */
  int NR = (dt == NXH_F64) ? 4
           : (dt == NXH_F16 || dt == NXH_F32 || dt == NXH_BF16 || dt == NXH_F8E4M3 ||
              dt == NXH_F8E5M2)
               ? 12
               : 8;
  int direct = (m < 8) || (n < NR) || (m * n * k < 48 * 48 * 48);
  g_last_threads = ncores();
  for (int64_t bi = 0; bi < nbatch; bi++) {
    int64_t rem = bi, ao = A->offset, bo = B->offset, co = C->offset;
    for (int d = bnd - 1; d >= 0; d--) {
      int64_t c = rem % bs[d];
      rem /= bs[d];
      ao += c * as_[d];
      bo += c * bs_[d];
      co += c * cs_[d];
    }
    fn((const char *)A->data + ao * es, ars, acs, (const char *)B->data + bo * es, brs,
       bcs, (char *)C->data + co * es, crs, ccs, m, n, k, !direct);
  }
  return NXH_OK;
}

/* ── gather (nx_c_move.c:342-458) ────────────────────────────────────────── */
NXO_EXPORT int nxo_gather(const nxh_tensor *out, const nxh_tensor *data,
                          const nxh_tensor *idx, int axis) {
  int dt = out->dtype;
  if ((unsigned)dt >= NXH_DTYPE_COUNT) return fail(NXH_FAILURE, "unsupported bigarray kind");
  if (is_packed(dt)) return fail(NXH_FAILURE, ERR_PACKED);
  if (axis < 0 || axis >= data->ndim) return fail(NXH_INVALID_ARGUMENT, ERR_AXIS);
  if (data->ndim != idx->ndim || data->ndim != out->ndim)
    return fail(NXH_INVALID_ARGUMENT, ERR_SHAPE);
  for (int d = 0; d < out->ndim; d++)
    if (out->shape[d] != idx->shape[d]) return fail(NXH_INVALID_ARGUMENT, ERR_SHAPE);
  int64_t total = 1;
  for (int d = 0; d < out->ndim; d++) total *= out->shape[d];
  if (total == 0) return NXH_OK;
  int64_t es = nxo_elem_size(dt), alen = data->shape[axis];
  int nd = out->ndim;
  int oob = 0;
  for (int64_t it = 0; it < total; it++) {
    int64_t coord[NXH_MAX_NDIM], rem = it;
    for (int d = nd - 1; d >= 0; d--) {
      coord[d] = rem % out->shape[d];
      rem /= out->shape[d];
    }
    int64_t io = idx->offset, oo = out->offset, doff = data->offset;
    for (int d = 0; d < nd; d++) {
      io += coord[d] * idx->strides[d];
      oo += coord[d] * out->strides[d];
    }
    int64_t index = ((const int32_t *)idx->data)[io];
    if (index < 0) index += alen;
    if (index < 0 || index >= alen) {
      oob = 1;
      break;
    }
    for (int d = 0; d < nd; d++)
      doff += (d == axis ? index : coord[d]) * data->strides[d];
    memcpy((char *)out->data + oo * es, (const char *)data->data + doff * es, (size_t)es);
  }
  if (oob)
    return fail(NXH_FAILURE, "index out of bounds for the gathered/scattered axis");
  return NXH_OK;
}

/* ── pad (nx_c_move.c:203-276) ───────────────────────────────────────────────
   Border slabs filled by broadcasting the fill scalar through copy, then the
   interior copied; every output element is written once. `fill` is one
   storage element of out's dtype. */
static int pad_fill(const nxh_tensor *slab, const void *fill) {
  for (int d = 0; d < slab->ndim; d++)
    if (slab->shape[d] == 0) return NXH_OK;
  return nxo_fill(slab, fill);
}
NXO_EXPORT int nxo_pad(const nxh_tensor *out, const nxh_tensor *in, const void *fill,
                       const int64_t *pad_before) {
  if ((unsigned)out->dtype >= NXH_DTYPE_COUNT) return fail(NXH_FAILURE, "unsupported bigarray kind");
  if (out->ndim != in->ndim) return fail(NXH_INVALID_ARGUMENT, ERR_SHAPE);
  if (is_packed(out->dtype)) return fail(NXH_FAILURE, ERR_PACKED);
  nxh_tensor slab = *out;
  for (int d = 0; d < out->ndim; d++) {
    int64_t before = pad_before[d];
    int64_t after = out->shape[d] - in->shape[d] - before;
    if (before < 0 || after < 0) return fail(NXH_INVALID_ARGUMENT, ERR_SHAPE);
    if (before > 0) {
      slab.shape[d] = before;
      int rc = pad_fill(&slab, fill);
      if (rc) return rc;
    }
    if (after > 0) {
      slab.shape[d] = after;
      slab.offset += (before + in->shape[d]) * out->strides[d];
      int rc = pad_fill(&slab, fill);
      if (rc) return rc;
      slab.offset -= (before + in->shape[d]) * out->strides[d];
    }
    slab.shape[d] = in->shape[d];
    slab.offset += before * out->strides[d];
  }
  return nxo_copy(&slab, in);
}

/* ── cat (nx_c_move.c:278-312) ───────────────────────────────────────────────
   One strided copy per member into successive slices of the output. */
NXO_EXPORT int nxo_cat(const nxh_tensor *out, const nxh_tensor *const *inputs, int n,
                       int axis) {
  if ((unsigned)out->dtype >= NXH_DTYPE_COUNT) return fail(NXH_FAILURE, "unsupported bigarray kind");
  if (axis < 0 || axis >= out->ndim) return fail(NXH_INVALID_ARGUMENT, ERR_AXIS);
  int64_t pos = 0;
  for (int m = 0; m < n; m++) {
    const nxh_tensor *in = inputs[m];
    if (in->ndim != out->ndim) return fail(NXH_INVALID_ARGUMENT, ERR_SHAPE);
    nxh_tensor slice = *out;
    slice.offset = out->offset + pos * out->strides[axis];
    for (int d = 0; d < out->ndim; d++) slice.shape[d] = in->shape[d];
    int rc = nxo_copy(&slice, in);
    if (rc) return rc;
    pos += in->shape[axis];
  }
  return NXH_OK;
}

/* ── inclusive scan (nx_c_fold.c:161-176, driver nx_c_engine.c:1257-1331) ────
   Sequential within a slice: the running value lives in the compute type and a
   rounded copy is stored per element. One element at a time through the fold
   step is exactly the reference's CMB(s, v); st(out, s). */
NXO_EXPORT int nxo_scan(int op, const nxh_tensor *out, const nxh_tensor *in, int axis) {
  if ((unsigned)op >= NXH_REDUCE_COUNT) return fail(NXH_INVALID_ARGUMENT, "unknown op");
  const fold_table *t = fold_tables[op];
  int dt = in->dtype;
  if ((unsigned)dt >= NXH_DTYPE_COUNT) return fail(NXH_FAILURE, "unsupported bigarray kind");
  if (!t->init[dt] || !t->step[dt])
    return fail(NXH_FAILURE, is_packed(dt) ? ERR_PACKED : ERR_UNSUPPORTED);
  if (axis < 0 || axis >= in->ndim) return fail(NXH_INVALID_ARGUMENT, ERR_AXIS);
  if (out->ndim != in->ndim) return fail(NXH_INVALID_ARGUMENT, "output rank mismatch");
  int64_t es = nxo_elem_size(dt), oes = nxo_elem_size(out->dtype);
  int64_t slices = 1, alen = in->shape[axis];
  for (int a = 0; a < in->ndim; a++)
    if (a != axis) slices *= in->shape[a];
  if (slices == 0 || alen == 0) return NXH_OK;
  for (int64_t it = 0; it < slices; it++) {
    int64_t rem = it, io = in->offset, oo = out->offset;
    for (int a = in->ndim - 1; a >= 0; a--) {
      if (a == axis) continue;
      int64_t c = rem % in->shape[a];
      rem /= in->shape[a];
      io += c * in->strides[a];
      oo += c * out->strides[a];
    }
    acc_t acc;
    t->init[dt](&acc);
    for (int64_t k = 0; k < alen; k++) {
      t->step[dt](&acc, (const char *)in->data + (io + k * in->strides[axis]) * es, es, 1);
      t->fini[dt]((char *)out->data + (oo + k * out->strides[axis]) * oes, &acc);
    }
  }
  return NXH_OK;
}

/* ── threefry2x32-20 (nx_c_random.c:36-133) ──────────────────────────────── */
static inline uint32_t rotl32(uint32_t x, int r) { return (uint32_t)((x << r) | (x >> (32 - r))); }
static void threefry2x32(uint32_t k0, uint32_t k1, uint32_t c0, uint32_t c1, uint32_t *o0,
                         uint32_t *o1) {
  static const int rots[8] = {13, 15, 26, 6, 17, 29, 16, 24};
  uint32_t ks[3] = {k0, k1, (uint32_t)0x1BD11BDA ^ k0 ^ k1};
  uint32_t x0 = c0 + k0, x1 = c1 + k1;
  for (int r = 0; r < 20; r++) {
    x0 += x1;
    x1 = rotl32(x1, rots[r % 8]);
    x1 ^= x0;
    if ((r + 1) % 4 == 0) {
      int s = (r + 1) / 4;
      x0 += ks[s % 3];
      x1 += ks[(s + 1) % 3] + (uint32_t)s;
    }
  }
  *o0 = x0;
  *o1 = x1;
}
NXO_EXPORT int nxo_threefry(const nxh_tensor *out, const nxh_tensor *key, const nxh_tensor *ctr) {
  if (out->dtype != NXH_I32 || key->dtype != NXH_I32 || ctr->dtype != NXH_I32)
    return fail(NXH_FAILURE, ERR_UNSUPPORTED);
  const char *bad = "threefry: last axis must have extent 2";
  if (key->ndim < 1 || key->ndim != ctr->ndim || key->ndim != out->ndim)
    return fail(NXH_INVALID_ARGUMENT, bad);
  int last = key->ndim - 1;
  for (int d = 0; d < key->ndim; d++)
    if (key->shape[d] != ctr->shape[d] || key->shape[d] != out->shape[d])
      return fail(NXH_INVALID_ARGUMENT, bad);
  if (key->shape[last] != 2) return fail(NXH_INVALID_ARGUMENT, bad);
  int64_t vectors = 1;
  for (int d = 0; d < last; d++) vectors *= key->shape[d];
  const int32_t *kd = key->data, *cd = ctr->data;
  int32_t *od = out->data;
  for (int64_t it = 0; it < vectors; it++) {
    int64_t rem = it, kb = key->offset, cb = ctr->offset, ob = out->offset;
    for (int d = last - 1; d >= 0; d--) {
      int64_t c = rem % key->shape[d];
      rem /= key->shape[d];
      kb += c * key->strides[d];
      cb += c * ctr->strides[d];
      ob += c * out->strides[d];
    }
    uint32_t o0, o1;
    threefry2x32((uint32_t)kd[kb], (uint32_t)kd[kb + key->strides[last]], (uint32_t)cd[cb],
                 (uint32_t)cd[cb + ctr->strides[last]], &o0, &o1);
    od[ob] = (int32_t)o0;
    od[ob + out->strides[last]] = (int32_t)o1;
  }
  return NXH_OK;
}

/* ── scatter (nx_c_move.c:460-586) ───────────────────────────────────────────
   out already holds the template. A serial row-major walk over the index space:
   Set keeps the last write, Add accumulates in the compute type in that order. */
#define MOVE_ADD_SINT(a, b) ((int64_t)((uint64_t)(a) + (uint64_t)(b)))
#define MOVE_ADD_UINT(a, b) ((a) + (b))
#define MOVE_ADD_FLOAT(a, b) ((a) + (b))
#define MOVE_ADD_COMPLEX(a, b) ((a) + (b))
#define MOVE_ADD_BOOL(a, b) ((a) + (b))
typedef void scatter_add_fn(char *out, const char *upd);
#define SCATTER_ADD(tag, sfx, S, C, LD, ST, cat) \
  static void scatter_add_##sfx(char *out, const char *upd) { \
    st_##sfx(out, (C)MOVE_ADD_##cat(ld_##sfx(out), ld_##sfx(upd))); \
  }
NXO_TABLE(SCATTER_ADD)
#define SCATTER_ADD_ROW(tag, sfx, S, C, LD, ST, cat) [tag] = scatter_add_##sfx,
static scatter_add_fn *const scatter_add_tbl[NXH_DTYPE_COUNT] = {NXO_TABLE(SCATTER_ADD_ROW)};

NXO_EXPORT int nxo_scatter(const nxh_tensor *out, const nxh_tensor *indices,
                           const nxh_tensor *updates, int axis, int mode) {
  int dt = out->dtype;
  if ((unsigned)dt >= NXH_DTYPE_COUNT) return fail(NXH_FAILURE, "unsupported bigarray kind");
  if (is_packed(dt)) return fail(NXH_FAILURE, ERR_PACKED);
  if (axis < 0 || axis >= out->ndim) return fail(NXH_INVALID_ARGUMENT, ERR_AXIS);
  if (out->ndim != indices->ndim || out->ndim != updates->ndim)
    return fail(NXH_INVALID_ARGUMENT, ERR_SHAPE);
  for (int d = 0; d < out->ndim; d++) {
    if (indices->shape[d] != updates->shape[d]) return fail(NXH_INVALID_ARGUMENT, ERR_SHAPE);
    if (d != axis && indices->shape[d] != out->shape[d]) return fail(NXH_INVALID_ARGUMENT, ERR_SHAPE);
  }
  scatter_add_fn *add = mode == 1 ? scatter_add_tbl[dt] : NULL;
  if (mode == 1 && !add) return fail(NXH_FAILURE, ERR_UNSUPPORTED);
  int nd = indices->ndim;
  int64_t total = 1, es = nxo_elem_size(dt), alen = out->shape[axis];
  for (int d = 0; d < nd; d++) total *= indices->shape[d];
  for (int64_t it = 0; it < total; it++) {
    int64_t coord[NXH_MAX_NDIM], rem = it;
    for (int d = nd - 1; d >= 0; d--) {
      coord[d] = rem % indices->shape[d];
      rem /= indices->shape[d];
    }
    int64_t io = indices->offset, uo = updates->offset, oo = out->offset;
    for (int d = 0; d < nd; d++) {
      io += coord[d] * indices->strides[d];
      uo += coord[d] * updates->strides[d];
    }
    int64_t index = ((const int32_t *)indices->data)[io];
    if (index < 0) index += alen;
    if (index < 0 || index >= alen)
      return fail(NXH_FAILURE, "index out of bounds for the gathered/scattered axis");
    for (int d = 0; d < nd; d++) oo += (d == axis ? index : coord[d]) * out->strides[d];
    char *op = (char *)out->data + oo * es;
    const char *up = (const char *)updates->data + uo * es;
    if (add) add(op, up);
    else memcpy(op, up, (size_t)es);
  }
  return NXH_OK;
}

/* ── sort / argsort (nx_c_sort.c:46-112, 262-330; driver :366-470) ────────────
   Each slice along `axis` is gathered into the compute type, NaN-class elements
   go to the tail in both directions, and the rest is ordered by the dtype's
   total order (complex: real, then imaginary). argsort breaks ties by the
   original index in both directions (nx_c_sort.c:96-104). The value sort of the
   reference is unstable and its descending result is the reverse of the
   ascending finite prefix (:283-289): elements that compare equal are
   indistinguishable except IEEE +-0, whose order the reference leaves
   unspecified; here that order is fixed as "ascending by original index, then
   reversed for descending", i.e. what a stable ascending sort followed by the
   reference's reversal gives. NaN-class elements keep their original order.
   A stable merge sort stands in for the reference's introsort: the result is
   determined by the order relation alone. */
#define SORT_LT_SINT(a, b) ((a) < (b))
#define SORT_LT_UINT(a, b) ((a) < (b))
#define SORT_LT_BOOL(a, b) ((a) < (b))
#define SORT_LT_FLOAT(a, b) ((a) < (b))
#define SORT_LT_COMPLEX(a, b) \
  (__real__(a) < __real__(b) || (__real__(a) == __real__(b) && __imag__(a) < __imag__(b)))
#define SORT_NAN_SINT(x) (0)
#define SORT_NAN_UINT(x) (0)
#define SORT_NAN_BOOL(x) (0)
#define SORT_NAN_FLOAT(x) (isnan(x))
#define SORT_NAN_COMPLEX(x) (isnan(__real__(x)) || isnan(__imag__(x)))

typedef void sort_slice_fn(char *o, int64_t os, const char *in, int64_t is, int64_t n, int desc,
                           int is_arg);
#define SORT_SLICE(tag, sfx, S, C, LD, ST, cat)                                              \
  /* a sorts strictly before b under the ascending value order, ties by index */             \
  static int sort_before_##sfx(const C *keys, int32_t i, int32_t j, int desc) {              \
    C x = keys[i], y = keys[j];                                                              \
    if (SORT_LT_##cat(x, y)) return !desc;                                                   \
    if (SORT_LT_##cat(y, x)) return desc;                                                    \
    return i < j;                                                                            \
  }                                                                                          \
  static void sort_merge_##sfx(const C *keys, int32_t *a, int32_t *tmp, int64_t n, int desc) { \
    if (n < 2) return;                                                                       \
    int64_t h = n / 2;                                                                       \
    sort_merge_##sfx(keys, a, tmp, h, desc);                                                 \
    sort_merge_##sfx(keys, a + h, tmp, n - h, desc);                                         \
    int64_t i = 0, j = h, k = 0;                                                             \
    while (i < h && j < n) tmp[k++] = sort_before_##sfx(keys, a[j], a[i], desc) ? a[j++] : a[i++]; \
    while (i < h) tmp[k++] = a[i++];                                                         \
    while (j < n) tmp[k++] = a[j++];                                                         \
    memcpy(a, tmp, (size_t)n * sizeof(int32_t));                                             \
  }                                                                                          \
  static void sort_slice_##sfx(char *o, int64_t os, const char *in, int64_t is, int64_t n,   \
                               int desc, int is_arg) {                                       \
    C *keys = malloc((size_t)n * sizeof(C));                                                 \
    int32_t *idx = malloc((size_t)n * sizeof(int32_t)), *tmp = malloc((size_t)n * sizeof(int32_t)); \
    for (int64_t k = 0; k < n; k++) keys[k] = ld_##sfx(in + k * is);                         \
    int64_t f = 0;                                                                           \
    for (int64_t k = 0; k < n; k++)                                                          \
      if (!(SORT_NAN_##cat(keys[k]))) idx[f++] = (int32_t)k;                                 \
    int64_t tail = f;                                                                        \
    for (int64_t k = 0; k < n; k++)                                                          \
      if (SORT_NAN_##cat(keys[k])) idx[tail++] = (int32_t)k;                                 \
    if (is_arg) {                                                                            \
      sort_merge_##sfx(keys, idx, tmp, f, desc);                                             \
      for (int64_t k = 0; k < n; k++) *(int32_t *)(o + k * os) = idx[k];                     \
    } else {                                                                                 \
      sort_merge_##sfx(keys, idx, tmp, f, 0);                                                \
      if (desc)                                                                              \
        for (int64_t i = 0, j = f - 1; i < j; i++, j--) {                                    \
          int32_t t = idx[i];                                                                \
          idx[i] = idx[j];                                                                   \
          idx[j] = t;                                                                        \
        }                                                                                    \
      for (int64_t k = 0; k < n; k++) st_##sfx(o + k * os, keys[idx[k]]);                    \
    }                                                                                        \
    free(keys);                                                                              \
    free(idx);                                                                               \
    free(tmp);                                                                               \
  }
NXO_TABLE(SORT_SLICE)
#define SORT_ROW(tag, sfx, S, C, LD, ST, cat) [tag] = sort_slice_##sfx,
static sort_slice_fn *const sort_tbl[NXH_DTYPE_COUNT] = {NXO_TABLE(SORT_ROW)};

static int sort_drive(const nxh_tensor *out, const nxh_tensor *in, int axis, int desc, int is_arg) {
  int dt = in->dtype;
  if ((unsigned)dt >= NXH_DTYPE_COUNT) return fail(NXH_FAILURE, "unsupported bigarray kind");
  if (is_packed(dt)) return fail(NXH_FAILURE, ERR_PACKED);
  if (axis < 0 || axis >= in->ndim) return fail(NXH_INVALID_ARGUMENT, ERR_AXIS);
  if (out->ndim != in->ndim) return fail(NXH_INVALID_ARGUMENT, "output rank inconsistent with the operation");
  int64_t n = in->shape[axis];
  if (is_arg && n > INT32_MAX) return fail(NXH_FAILURE, "argsort axis length exceeds INT32_MAX");
  int64_t ies = nxo_elem_size(dt), oes = is_arg ? 4 : ies, nslices = 1;
  for (int d = 0; d < in->ndim; d++)
    if (d != axis) nslices *= in->shape[d];
  if (nslices == 0 || n == 0) return NXH_OK;
  for (int64_t s = 0; s < nslices; s++) {
    int64_t rem = s, io = in->offset, oo = out->offset;
    for (int d = in->ndim - 1; d >= 0; d--) {
      if (d == axis) continue;
      int64_t c = rem % in->shape[d];
      rem /= in->shape[d];
      io += c * in->strides[d];
      oo += c * out->strides[d];
    }
    sort_tbl[dt]((char *)out->data + oo * oes, out->strides[axis] * oes, (const char *)in->data + io * ies,
                 in->strides[axis] * ies, n, desc, is_arg);
  }
  return NXH_OK;
}
NXO_EXPORT int nxo_sort(const nxh_tensor *out, const nxh_tensor *in, int axis, int descending) {
  return sort_drive(out, in, axis, descending, 0);
}
NXO_EXPORT int nxo_argsort(const nxh_tensor *out, const nxh_tensor *in, int axis, int descending) {
  return sort_drive(out, in, axis, descending, 1);
}

/* ── unfold / fold (nx_c_move.c:588-870) ──────────────────────────────────────
   unfold: (leading..., spatial...) -> (leading..., prod(kernel), L); element
   (lead, tap kf, window w) reads x[lead, w*stride + k*dilation - pad_before] per
   spatial dim, or zero outside the input (:655-690). fold: the inverse, summing
   the taps that land on each output element in ascending tap order, in the
   compute type (:745-787). padding is flat [before0, after0, ...]. */
typedef struct {
  int K, ld;
  int64_t kernel[NXH_MAX_NDIM], stride[NXH_MAX_NDIM], dilation[NXH_MAX_NDIM], before[NXH_MAX_NDIM];
  int64_t win[NXH_MAX_NDIM], win_cp[NXH_MAX_NDIM], ker_cp[NXH_MAX_NDIM], kernel_prod, L;
} window_t;
static void window_counts(window_t *w, const int64_t *extent, const int64_t *padding) {
  for (int d = 0; d < w->K; d++) {
    int64_t eff = w->dilation[d] * (w->kernel[d] - 1) + 1;
    int64_t padded = extent[d] + padding[2 * d] + padding[2 * d + 1];
    int64_t win = (padded - eff) / w->stride[d] + 1;
    w->win[d] = win < 1 ? 1 : win;
    w->before[d] = padding[2 * d];
  }
  w->win_cp[w->K - 1] = 1;
  w->ker_cp[w->K - 1] = 1;
  for (int d = w->K - 2; d >= 0; d--) {
    w->win_cp[d] = w->win_cp[d + 1] * w->win[d + 1];
    w->ker_cp[d] = w->ker_cp[d + 1] * w->kernel[d + 1];
  }
}
NXO_EXPORT int nxo_unfold(const nxh_tensor *out, const nxh_tensor *in, int K, const int64_t *kernel,
                          const int64_t *stride, const int64_t *dilation, const int64_t *padding) {
  int dt = out->dtype;
  if ((unsigned)dt >= NXH_DTYPE_COUNT) return fail(NXH_FAILURE, "unsupported bigarray kind");
  if (is_packed(dt)) return fail(NXH_FAILURE, ERR_PACKED);
  if (K < 1 || K > NXH_MAX_NDIM || in->ndim < K) return fail(NXH_INVALID_ARGUMENT, ERR_SHAPE);
  window_t w;
  w.K = K;
  w.ld = in->ndim - K;
  for (int d = 0; d < K; d++) w.kernel[d] = kernel[d], w.stride[d] = stride[d], w.dilation[d] = dilation[d];
  w.kernel_prod = out->shape[w.ld];
  w.L = out->shape[w.ld + 1];
  window_counts(&w, &in->shape[w.ld], padding);
  int64_t lead = 1, es = nxo_elem_size(dt);
  for (int d = 0; d < w.ld; d++) lead *= in->shape[d];
  int64_t total = lead * w.kernel_prod * w.L;
  for (int64_t it = 0; it < total; it++) {
    int64_t wf = it % w.L, rem = it / w.L, kf = rem % w.kernel_prod, l = rem / w.kernel_prod;
    int64_t oo = out->offset + kf * out->strides[w.ld] + wf * out->strides[w.ld + 1], io = in->offset;
    for (int d = w.ld - 1; d >= 0; d--) {
      int64_t c = l % in->shape[d];
      l /= in->shape[d];
      oo += c * out->strides[d];
      io += c * in->strides[d];
    }
    bool valid = true;
    for (int d = 0; d < K && valid; d++) {
      int64_t wc = (wf / w.win_cp[d]) % w.win[d], kc = (kf / w.ker_cp[d]) % w.kernel[d];
      int64_t sp = wc * w.stride[d] + kc * w.dilation[d] - w.before[d];
      if (sp < 0 || sp >= in->shape[w.ld + d]) valid = false;
      else io += sp * in->strides[w.ld + d];
    }
    char *dst = (char *)out->data + oo * es;
    if (valid) memcpy(dst, (const char *)in->data + io * es, (size_t)es);
    else memset(dst, 0, (size_t)es);
  }
  return NXH_OK;
}

typedef void fold_sum_fn(char *out, const char *const *taps, int ntaps);
#define FOLD_SUM(tag, sfx, S, C, LD, ST, cat)                                   \
  static void fold_sum_##sfx(char *out, const char *const *taps, int ntaps) {   \
    C acc = (C)0;                                                               \
    for (int i = 0; i < ntaps; i++) acc = (C)MOVE_ADD_##cat(acc, ld_##sfx(taps[i])); \
    st_##sfx(out, acc);                                                         \
  }
NXO_TABLE(FOLD_SUM)
#define FOLD_SUM_ROW(tag, sfx, S, C, LD, ST, cat) [tag] = fold_sum_##sfx,
static fold_sum_fn *const fold_sum_tbl[NXH_DTYPE_COUNT] = {NXO_TABLE(FOLD_SUM_ROW)};

NXO_EXPORT int nxo_fold(const nxh_tensor *out, const nxh_tensor *in, int K, const int64_t *output_size,
                        const int64_t *kernel, const int64_t *stride, const int64_t *dilation,
                        const int64_t *padding) {
  int dt = out->dtype;
  if ((unsigned)dt >= NXH_DTYPE_COUNT) return fail(NXH_FAILURE, "unsupported bigarray kind");
  if (is_packed(dt)) return fail(NXH_FAILURE, ERR_PACKED);
  if (K < 1 || K > NXH_MAX_NDIM || in->ndim < 2) return fail(NXH_INVALID_ARGUMENT, ERR_SHAPE);
  window_t w;
  w.K = K;
  w.ld = in->ndim - 2;
  for (int d = 0; d < K; d++) w.kernel[d] = kernel[d], w.stride[d] = stride[d], w.dilation[d] = dilation[d];
  w.kernel_prod = in->shape[w.ld];
  w.L = in->shape[w.ld + 1];
  window_counts(&w, output_size, padding);
  int64_t lead = 1, spatial = 1, es = nxo_elem_size(dt);
  for (int d = 0; d < w.ld; d++) lead *= in->shape[d];
  for (int d = 0; d < K; d++) spatial *= output_size[d];
  const char **taps = malloc((size_t)(w.kernel_prod > 0 ? w.kernel_prod : 1) * sizeof(char *));
  for (int64_t it = 0; it < lead * spatial; it++) {
    int64_t ol = it % spatial, l = it / spatial, oc[NXH_MAX_NDIM];
    for (int d = K - 1; d >= 0; d--) {
      oc[d] = ol % output_size[d];
      ol /= output_size[d];
    }
    int64_t oo = out->offset, il = in->offset;
    for (int d = w.ld - 1; d >= 0; d--) {
      int64_t c = l % out->shape[d];
      l /= out->shape[d];
      oo += c * out->strides[d];
      il += c * in->strides[d];
    }
    for (int d = 0; d < K; d++) oo += oc[d] * out->strides[w.ld + d];
    int ntaps = 0;
    for (int64_t kf = 0; kf < w.kernel_prod; kf++) {
      bool valid = true;
      int64_t wf = 0;
      for (int d = 0; d < K && valid; d++) {
        int64_t kc = (kf / w.ker_cp[d]) % w.kernel[d];
        int64_t num = oc[d] + w.before[d] - kc * w.dilation[d];
        if (num < 0 || num % w.stride[d] != 0 || num / w.stride[d] >= w.win[d]) valid = false;
        else wf += (num / w.stride[d]) * w.win_cp[d];
      }
      if (valid)
        taps[ntaps++] = (const char *)in->data + (il + kf * in->strides[w.ld] + wf * in->strides[w.ld + 1]) * es;
    }
    fold_sum_tbl[dt]((char *)out->data + oo * es, taps, ntaps);
  }
  free(taps);
  return NXH_OK;
}
