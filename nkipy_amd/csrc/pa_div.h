// x / s for many x and one s, in three instructions per x instead of the ten-odd of a division, with the
// bits of the correctly rounded float32 quotient.
//
// r = pa_refine_rcp(s, r0) is one Newton step on a reciprocal estimate r0 of s; pa_div_by(x, s, r) is the
// product x r corrected once by its exact residual (Markstein's scheme).  For every x with at most 8
// significant bits (a bf16 value) and every float32 s whose mantissa field is not all ones the result
// equals x / s rounded to nearest even, for any estimate r0 within 4 ulp of 1 / s: checked over all
// 2^7 x 2^23 mantissa pairs and the nine estimates by tests/test_div_by_scale.py, which compiles this very
// file for the CPU.  (With all ones, x a power of two gives 2^k where x / s rounds to 2^k (1 + 2^-23).)
// Scaling x or s by a power of two scales every intermediate exactly as long as none of them leaves the
// normal range: callers keep s within [2^-40, 2^40] and take an ordinary division otherwise.  The sign is
// taken from x at the end (x = -0 would come out as +0).
//
// The includer defines PA_HD, the qualifiers of the functions (`__device__ __forceinline__` in the kernels,
// `static inline` in the CPU check).
#ifndef PA_HD
#error "define PA_HD (the function qualifiers) before including pa_div.h"
#endif

PA_HD float pa_refine_rcp(float s, float r0) {
  const float e = fmaf(-s, r0, 1.f);
  return fmaf(e, r0, r0);
}

PA_HD float pa_div_by(float x, float s, float r) {
  const float q = x * r;
  const float e = fmaf(-s, q, x);
  return copysignf(fmaf(e, r, q), x);
}

// s for which pa_div_by may stand in for a division
PA_HD int pa_div_by_ok(float s, unsigned s_bits) {
  return s >= 0x1p-40f && s <= 0x1p40f && (s_bits & 0x7fffffu) != 0x7fffffu;
}
