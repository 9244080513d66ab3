// Device-side scalar math for the activation kernels.  Short straight-line
// sequences built on v_exp_f32 / v_rcp_f32 and FMAs: at HBM roofline an MI355X
// retires roughly one fp32 element per 40-50 lane instructions, so libm calls
// (branches, table lookups) would turn these memory-bound ops compute-bound.
#pragma once

#include <hip/hip_runtime.h>

namespace twg {

constexpr float kLog2eHi = 0x1.715476p+0f;    // float(log2(e))
constexpr float kLog2eLo = 0x1.4ae0c0p-26f;   // log2(e) - float(log2(e))
constexpr float kLn2 = 0x1.62e430p-1f;

__device__ __forceinline__ float hw_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float hw_rcp(float x) { return __builtin_amdgcn_rcpf(x); }

// max(0, x) as PyTorch's CPU kernel evaluates it: NaN stays NaN, -0.0 stays
// -0.0, every negative value (and -inf) becomes +0.0.
// Reference formula: csrc/ops/unary.cpp:91  "max(0.0, x)".
__device__ __forceinline__ float relu_f32(float x) { return x < 0.0f ? 0.0f : x; }

// exp(-m) for m >= 0 as 2^(-m*log2e), with the rounding error of the product
// -m*log2e (and of the constant) folded back in to first order.  Without this
// the relative error grows like |m| * 2^-24, which is 5e-6 at m = 80.
// v_exp_f32 flushes subnormal results, so below 2^-96 the exponential is taken
// 64 binades up and `tiny` tells the caller to scale its product back by 2^-64.
// Returns e = exp(-m) (times 2^64 if tiny) to about 2 ulp.
__device__ __forceinline__ float exp_neg(float m, bool &tiny) {
  m = fminf(m, 150.0f);  // exp(-150) is 0 in binary32; also keeps inf - inf out of u_lo
  const float u_hi = __fmul_rn(-m, kLog2eHi);
  float u_lo = __fmaf_rn(-m, kLog2eHi, -u_hi);
  u_lo = __fmaf_rn(-m, kLog2eLo, u_lo);
  tiny = u_hi < -96.0f;
  const float e = hw_exp2(u_hi + (tiny ? 64.0f : 0.0f));
  return __fmaf_rn(e, kLn2 * u_lo, e);
}

// x * sigmoid(w) where w has the sign of x (or is x itself).
//   w >= 0:  x / (1 + e^-w);   w < 0:  x * e^w / (1 + e^w)
// Both branches share e = exp(-|w|) in (0, 1], so nothing overflows.  When e is
// tiny, 1 + e rounds to 1 whether or not e carries the 2^64 factor.
__device__ __forceinline__ float x_sigmoid(float x, float w) {
  bool tiny;
  const float e = exp_neg(fabsf(w), tiny);
  const float r = hw_rcp(1.0f + e);
  const float xs = tiny ? x * 0x1p-64f : x;
  const float num = (w >= 0.0f) ? x : xs * e;
  return num * r;
}

// SiLU.  Reference formula: csrc/ops/unary.cpp:97  "x * (1 / (1 + exp(-1 * x)))".
__device__ __forceinline__ float silu_f32(float x) { return x_sigmoid(x, x); }

// GeLU, tanh form.  Reference formula: csrc/ops/unary.cpp:94
//   0.5*x*(1 + tanh(sqrt(2/pi) * (x + 0.044715*x^3)))
// evaluated through the identity 0.5*(1 + tanh(u)) = sigmoid(2u), which has no
// cancellation for negative x.  x^3 is x*x*x (WGSL pow(x, 3) is undefined for
// x < 0).
__device__ __forceinline__ float gelu_tanh_f32(float x) {
  constexpr float k2 = 2.0f * 0.7978845608028654f;  // 2*sqrt(2/pi)
  const float x2 = x * x;
  const float w = (k2 * x) * __fmaf_rn(0.044715f, x2, 1.0f);
  return x_sigmoid(x, w);
}

// GeLU, exact form x * Phi(x) (ATen approximate='none').
//
// With a = |x|:  Phi(-a) = exp(-a^2/2) * G(a),  G(a) = erfcx(a/sqrt 2)/2.
// G is smooth and positive; G(a) = t * P8(t), t = 1/(1 + 0.35 a), is a weighted
// least-squares fit on a in [0, 15] with relative error 3.7e-8.  a^2/2 is
// formed as a rounded product plus its exact FMA residual, and the exponent is
// split the same way, so the result keeps about 4e-7 relative error down into
// the far negative tail where x*Phi(x) is ~1e-38 (plain 0.5*x*(1+erf(x/sqrt 2))
// has lost every digit by x = -6).  The exponential is evaluated 64 binades up and
// the result scaled back at the end, so subnormal results are rounded once.
//   x > 0:  x * (1 - Phi(-a)) = x * (1 - q);     x <= 0:  x * q.
// gelu(+-0) = +-0, gelu(NaN) = NaN, gelu(+inf) = +inf, gelu(x <= -14.2) = -0 for finite x
// (the argument of Phi is clamped at 15, so -inf comes back as -inf).
__device__ __forceinline__ float gelu_erf_f32(float x) {
  const float a = fminf(fabsf(x), 15.0f);
  const float t = hw_rcp(__fmaf_rn(0.35f, a, 1.0f));
  float p = -0.02949463550446831f;
  p = __fmaf_rn(p, t, 0.14561740209021237f);
  p = __fmaf_rn(p, t, -0.2589950403025755f);
  p = __fmaf_rn(p, t, 0.1627681203503808f);
  p = __fmaf_rn(p, t, -0.02546558414936332f);
  p = __fmaf_rn(p, t, 0.10644964114479509f);
  p = __fmaf_rn(p, t, 0.11960979643938191f);
  p = __fmaf_rn(p, t, 0.13989037693051265f);
  p = __fmaf_rn(p, t, 0.139619904786415f);
  const float g = t * p;

  const float h = 0.5f * a;
  const float s_hi = __fmul_rn(h, a);
  const float s_lo = __fmaf_rn(h, a, -s_hi);
  const float u_hi = __fmul_rn(-s_hi, kLog2eHi);
  float u_lo = __fmaf_rn(-s_hi, kLog2eHi, -u_hi);
  u_lo = __fmaf_rn(-s_hi, kLog2eLo, u_lo);
  // The exponential is always taken 64 binades up (u_hi >= -163 because a <= 15, so the
  // argument stays above v_exp_f32's flush threshold of -126) and the factor 2^-64 is
  // applied last: results that are subnormal are then rounded exactly once.
  const float e = hw_exp2(u_hi + 64.0f);
  const float eg = e * g;
  const float q = __fmaf_rn(eg, __fmaf_rn(kLn2, u_lo, -s_lo), eg);  // Phi(-a) * 2^64
  // x > 0 (not >=) so that -0.0 takes the product branch and keeps its sign;
  // x * (1 - Phi(-a)) rather than x - x*Phi(-a) so that +inf stays +inf.
  return (x > 0.0f) ? x * __fmaf_rn(q, -0x1p-64f, 1.0f) : (x * q) * 0x1p-64f;
}

}  // namespace twg
