/* Exhaustive CPU check of nkipy_amd/csrc/pa_div.h, the quotient the fp8 KV write forms from a reciprocal.
 * For every float32 scale mantissa (step argv[1], default 1), every reciprocal estimate within 4 ulp of
 * 1 / s and every 8-bit significand of x: pa_div_by == x / s bit for bit, except where the mantissa field of
 * s is all ones (which pa_div_by_ok must refuse).  Also walks exponents of s at the ends of the accepted range
 * and the signs and zeros of x.  Prints one line; exit status 0 when nothing differs. */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#define PA_HD static inline
#include "pa_div.h"

static inline float f_of(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t u_of(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

int main(int argc, char** argv) {
  const int step = argc > 1 ? atoi(argv[1]) : 1;
  long bad = 0, refused_wrongly = 0, n = 0;
#pragma omp parallel for reduction(+ : bad, refused_wrongly, n) schedule(static)
  for (uint32_t ms = 0; ms < (1u << 23); ms += step) {
    const float s = f_of(0x3f800000u | ms);
    const int ok = pa_div_by_ok(s, u_of(s));
    if (ok != (ms != 0x7fffffu)) ++refused_wrongly;
    if (!ok) continue;
    const float rn = 1.0f / s;
    for (int d = -4; d <= 4; ++d) {
      const float r = pa_refine_rcp(s, f_of(u_of(rn) + d));
      for (uint32_t mx = 0; mx < 128; ++mx) {
        const float x = f_of(0x3f800000u | (mx << 16));
        if (u_of(pa_div_by(x, s, r)) != u_of(x / s)) ++bad;
        ++n;
      }
    }
  }
  /* exponents: s at both ends of the accepted range and around one, x over the whole bf16 range (every
   * exponent, a few significands, both signs, zeros); results that matter to an fp8 code (|q| >= 2^-12) must be
   * exact, smaller ones must keep the sign and stay small */
  const uint32_t s_bits[] = {0x2b800000u /* 2^-40 */, 0x2b9e3779u, 0x3f7ffffeu, 0x3f800001u, 0x53000000u /* 2^39 */, 0x537ffffeu, 0x53800000u /* 2^40 */};
  for (unsigned si = 0; si < sizeof s_bits / sizeof *s_bits; ++si) {
    const float s = f_of(s_bits[si]);
    if (!pa_div_by_ok(s, s_bits[si])) { ++refused_wrongly; continue; }
    const float r = pa_refine_rcp(s, 1.0f / s);
    for (uint32_t hi = 0; hi < 0x10000u; ++hi) {
      if ((hi & 0x7f80u) == 0x7f80u) continue;           /* inf / nan rows never reach the quotient's fast form */
      const float x = f_of(hi << 16), want = x / s, got = pa_div_by(x, s, r);
      if (fabsf(want) > 500.f) continue;                  /* x <= 448 s in the kernel */
      ++n;
      if (fabsf(want) >= 0x1p-12f) { if (u_of(got) != u_of(want)) ++bad; }
      else if (signbit(got) != signbit(want) || !(fabsf(got) < 0x1p-11f)) ++bad;
    }
  }
  if (pa_div_by_ok(0x1p-41f, u_of(0x1p-41f)) || pa_div_by_ok(0x1.8p40f, u_of(0x1.8p40f)) || pa_div_by_ok(INFINITY, u_of(INFINITY)) ||
      pa_div_by_ok(NAN, u_of(NAN)) || pa_div_by_ok(0.f, 0u))
    ++refused_wrongly;
  printf("cases %ld  wrong quotients %ld  wrong acceptance %ld\n", n, bad, refused_wrongly);
  return bad || refused_wrongly ? 1 : 0;
}
