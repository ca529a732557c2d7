// Correctly rounded fp32 division and square root for operands in the layer's working range,
// cheaper than the compiler's general IEEE expansions.
//
// The compiler expands a / b into div_scale, rcp, four fused refinement steps, div_fmas and
// div_fixup; the scale / fixup instructions only matter for operands near the ends of the exponent
// range, denormals, zeros and infinities in the denominator.  The sequences below are the same
// Newton-Raphson core (reciprocal refined once, quotient corrected twice with exact fma residuals)
// without that range handling, so they return the same bits whenever the operands are ordinary:
//   denominators here are >= 0.02 (1 + c, max(1, .), a triangle norm above delta) and finite,
//   numerators are zero or of ordinary magnitude.
// The reciprocal is a separate step so that several numerators can share one denominator.
// exact_sqrt is v_sqrt_f32 (1 ulp) plus the one-ulp-up / one-ulp-down residual test; inputs below
// 2^-96 would need the compiler's pre-scaling to stay exact and callers do not need them exact
// (a triangle norm that small is far below the Huber threshold).
//
// inpaint_selftest_math() (C ABI) compares all three against the compiler's `/` and sqrtf on the
// GPU: exhaustively where the domain is one float, on structured + random pairs otherwise.
#pragma once

#include <hip/hip_runtime.h>

namespace inpaint {

// reciprocal of d, refined: |r - 1/d| is far below half an ulp except in rare last-bit cases
__device__ __forceinline__ float rcp_refined(float d) {
  float r = __builtin_amdgcn_rcpf(d);
  const float e = __builtin_fmaf(-d, r, 1.0f);
  return __builtin_fmaf(e, r, r);
}

// n / d given r = rcp_refined(d)
__device__ __forceinline__ float div_by(float n, float d, float r) {
  float q = n * r;
  float e = __builtin_fmaf(-d, q, n);
  q = __builtin_fmaf(e, r, q);
  e = __builtin_fmaf(-d, q, n);
  return __builtin_fmaf(e, r, q);
}

__device__ __forceinline__ float exact_div(float n, float d) { return div_by(n, d, rcp_refined(d)); }

__device__ __forceinline__ float exact_sqrt(float x) {
  const float s = __builtin_amdgcn_sqrtf(x);
  const float s_dn = __int_as_float(__float_as_int(s) - 1);
  const float s_up = __int_as_float(__float_as_int(s) + 1);
  const float r_dn = __builtin_fmaf(-s_dn, s, x);
  const float r_up = __builtin_fmaf(-s_up, s, x);
  // x = 0 and x = +inf need no case of their own: their residuals are 0 or NaN, both tests fail and s itself
  // (0 or +inf) is returned
  float out = (r_dn <= 0.0f) ? s_dn : s;
  out = (r_up > 0.0f) ? s_up : out;
  return out;
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
