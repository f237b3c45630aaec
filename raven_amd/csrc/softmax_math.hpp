// softmax_math.hpp — the exponential and the quotient of the fused softmax
// kernels whose result is rounded to a 16-bit dtype right behind them
// (attention.hip; softmax_rows with a 16-bit output in rowfuse.hip).
#pragma once

// e^x for x <= 0, -inf or NaN. The library's expf costs about thirteen
// instructions and bounded those kernels. Six do: 2^(x log2 e) by the hardware
// exponential on the rounded product p, times e^d for what the rounding of p
// dropped, d = x - p ln 2 in two fused steps, e^d = 1 + d to 2^-39. Within 2 ulp
// of the exact value (the primitive's expf is within 1), far inside the
// reference's tolerance for f32 transcendentals (rel 1e-4,
// backend_contract.ml:179-188). x = -inf has p = -inf, r = 0 and
// d = inf - inf = NaN: the maximum drops that NaN (a true d is tiny), so the
// result is 0; a NaN x gives NaN through r. Results below 2^-126 are flushed
// to zero.
__device__ __forceinline__ float exp_nonpositive(float x) {
  const float p = x * 0x1.715476p+0f;
  const float r = __builtin_amdgcn_exp2f(p);
  float d = __builtin_fmaf(p, -0x1.62e400p-1f, x);  // ln 2 in two parts (0.693145751953125 + 1.4286068e-6)
  d = __builtin_fmaf(p, -0x1.7f7d1cp-20f, d);
  return __builtin_fmaf(r, __builtin_fmaxf(d, -1.0f), r);
}

// e / l with 1 / l at hand: one Newton step on the quotient (Markstein), which is
// the correctly rounded e / l whenever rl is the correctly rounded reciprocal and
// the quotient is a normal number; three instructions against the ten of a division.
__device__ __forceinline__ float div_by_reciprocal(float e, float l, float rl) {
  const float q = e * rl;
  return __builtin_fmaf(__builtin_fmaf(-q, l, e), rl, q);
}

