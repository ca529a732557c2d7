// Correctly rounded fp32 division, reciprocal and square root for operands in the layer's working range,
// cheaper than the compiler's general IEEE expansions.
//
// The compiler expands a / b into div_scale, rcp, four fused refinement steps, div_fmas and div_fixup (one
// refinement of the reciprocal, two corrections of the quotient); the scale / fixup instructions only matter for
// operands near the ends of the exponent range, denormals, zeros and infinities in the denominator.  The sequences
// below drop that range handling AND the second correction of the quotient:
//   r = rcp(d) refined once        is the correctly rounded 1 / d for every float d in [2^-40, 2^40],
//   q = n r corrected once         (q + fma(-d, q, n) r) is the correctly rounded n / d for ALL 2^46 pairs of mantissas
//                                  (n, d in [1, 2)), hence for every pair of ordinary operands: the three operations are
//                                  exact up to a common power of two as long as nothing underflows.
// Both facts hold for this GPU's v_rcp_f32 and are checked exhaustively on the device against the compiler's `/`
// (inpaint_selftest_rsqrt for the reciprocal, inpaint_selftest_division_pairs for the quotient: 7.0e13 pairs, about
// 40 s).  They return the compiler's bits whenever the operands are ordinary:
//   denominators here are >= 0.02 (1 + c, max(1, .), a triangle norm above delta) and finite,
//   numerators are zero or of ordinary magnitude.
// The reciprocal is a separate step so that several numerators can share one denominator.
// x / c for the two Huber thresholds c = 0.1f, 0.2f needs no reciprocal instruction at all: with R = RN(1 / c)
// (10.0f and 5.0f; |c R - 1| = 2^-26) one correction of x R is within 2^-26 ulp of x / c, and a quotient by a
// 24-bit c is never closer than 2^-25 ulp to a rounding boundary (checked exhaustively as well).
// exact_sqrt is v_rsq_f32 (1 ulp) turned into the root and corrected once; inputs below 2^-96 would need the
// compiler's pre-scaling to stay exact and callers do not need them exact (a triangle norm that small is far below the
// Huber threshold).
//
// inpaint_selftest_math() (C ABI) compares them against the compiler's `/` and sqrtf on the GPU:
// exhaustively where the domain is one float, on structured + random pairs over a wide range of exponents otherwise.
#pragma once

#include <hip/hip_runtime.h>

namespace inpaint {

// reciprocal of d, refined once: the correctly rounded 1 / d
__device__ __forceinline__ float rcp_refined(float d) {
  float r = __builtin_amdgcn_rcpf(d);
  const float e = __builtin_fmaf(-d, r, 1.0f);
  return __builtin_fmaf(e, r, r);
}
__device__ __forceinline__ float exact_rcp(float d) { return rcp_refined(d); }

// n / d given r = rcp_refined(d)
__device__ __forceinline__ float div_by(float n, float d, float r) {
  const float q = n * r;
  const float e = __builtin_fmaf(-d, q, n);
  return __builtin_fmaf(e, r, q);
}

__device__ __forceinline__ float exact_div(float n, float d) { return div_by(n, d, rcp_refined(d)); }

// x / 0.1f and x / 0.2f (the Huber thresholds)
__device__ __forceinline__ float div_by_tenth(float x) { return div_by(x, 0.1f, 10.0f); }
__device__ __forceinline__ float div_by_fifth(float x) { return div_by(x, 0.2f, 5.0f); }

// sqrt(x), correctly rounded, for x = 0 and every finite x >= 2^-96: v_rsq_f32 (1 ulp) gives the root x * y and half its
// reciprocal y / 2, and one Newton correction with the exact fma residual lands on the correctly rounded value for every
// such x (checked exhaustively).  The clamp keeps y finite at x = 0, where the root and the residual are 0.  +inf is not
// in the domain (the product inf * 0 is NaN); smaller positive x may be one ulp off, denormals more.
__device__ __forceinline__ float exact_sqrt(float x) {
  const float y = __builtin_amdgcn_rsqf(fmaxf(x, 1.17549435e-38f));
  const float s = x * y;
  const float e = __builtin_fmaf(-s, s, x);
  return __builtin_fmaf(e, 0.5f * y, s);
}

// Values of lanes outside the image read as +0: inside(v) is v where `ok` held and +0 elsewhere, bit for bit what
// `ok ? v : 0.f` gives.  The loaded bits are ANDed with an all-ones / all-zeros word whose origin the empty asm hides
// from the optimizer; written as a conditional, a group of such values is compiled into a branch that zeroes all of
// them and then copies all of them.
struct LaneMask {
  unsigned keep;
  __device__ __forceinline__ explicit LaneMask(bool ok) : keep(ok ? 0xffffffffu : 0u) { asm("" : "+v"(keep)); }
  __device__ __forceinline__ float operator()(float v) const { return __uint_as_float(__float_as_uint(v) & keep); }
};
// The same values from the plain conditional, for the kernels in which the AND form costs registers they do not have.
struct LaneSelect {
  bool ok;
  __device__ __forceinline__ explicit LaneSelect(bool ok_) : ok(ok_) {}
  __device__ __forceinline__ float operator()(float v) const { return ok ? v : 0.f; }
};

}  // namespace inpaint
