// v / q in fp32, correctly rounded, for a divisor q that is fixed for a whole launch: five multiply-adds with the
// correctly rounded reciprocal r = RN(1/q) instead of the hardware's division sequence (ten instructions):
//    y0 = RN(v r)                       within 2 ulp of v / q
//    y1 = RN(y0 + RN(v - q y0) r)       within 1 ulp (a faithful rounding: one of the two neighbours of v / q)
//    y  = RN(y1 + (v - q y1) r)         v - q y1 is exact in a fused multiply-add; by Markstein's theorem a faithful
//                                       quotient corrected once more with a reciprocal of relative error below 2^-24 is
//                                       the correctly rounded one.  RN(1/q) has that accuracy unless the significand of q
//                                       is all ones.
// This holds while nothing overflows or goes subnormal on the way; quotient_plan() admits only divisors and operand
// ranges for which that is certain wherever the result matters to a caller that rounds it to an 8-bit integer
// (|v / q| >= 1/4; below that every approximation within a few ulp rounds to 0 like the exact quotient).
#pragma once
#include <cmath>
#include <cstdint>
#include <cstring>

#if defined(__HIPCC__)
#define SOFIE_QUOTIENT_FN __host__ __device__ inline
#else
#define SOFIE_QUOTIENT_FN inline
#endif

namespace sofie_hip {

SOFIE_QUOTIENT_FN float quotient_by_reciprocal(float v, float q, float r)
{
   const float y0 = v * r;
   const float e0 = __builtin_fmaf(-y0, q, v);
   const float y1 = __builtin_fmaf(e0, r, y0);
   const float e1 = __builtin_fmaf(-y1, q, v);
   return __builtin_fmaf(e1, r, y1);
}

// RN(1/q) for a finite non-zero q: the candidate from double arithmetic, checked against its two neighbours with the exact
// residual 1 - q r (a 48-bit product and a difference of nearby numbers: both exact in double).
inline float reciprocal_rn(float q)
{
   float best = (float)(1.0 / (double)q);
   double err = std::fabs(1.0 - (double)q * (double)best);
   const float cand[2] = {std::nextafterf(best, INFINITY), std::nextafterf(best, -INFINITY)};
   for (float c : cand) {
      const double e = std::fabs(1.0 - (double)q * (double)c);
      if (e < err) {
         err = e;
         best = c;
      }
   }
   return best;
}

// Whether quotient_by_reciprocal may stand in for the division of v = float(acc) * s by q, acc any int32: s zero or
// 2^-40 <= |s| <= 2^30, 2^-30 <= |q| <= 2^40 (no overflow: |v / q| <= 2^91; no subnormal residual where |v / q| >= 1/4),
// and the significand of q not all ones.  Sets r = RN(1/q).
inline bool quotient_plan(float s, float q, float &r)
{
   r = 0.0f;
   if (!std::isfinite(s) || !std::isfinite(q) || q == 0.0f)
      return false;
   const float as = std::fabs(s), aq = std::fabs(q);
   if (as != 0.0f && (as < 0x1p-40f || as > 0x1p30f))
      return false;
   if (aq < 0x1p-30f || aq > 0x1p40f)
      return false;
   uint32_t bits;
   std::memcpy(&bits, &q, 4);
   if ((bits & 0x7fffffu) == 0x7fffffu)
      return false;
   r = reciprocal_rn(q);
   return true;
}

} // namespace sofie_hip
