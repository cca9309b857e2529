// CPU check of sofie_amd/csrc/exact_quotient.hpp: the five multiply-adds with the rounded reciprocal against the
// processor's IEEE division.  Prints one line per divisor: "<q> <values tried> <mismatches>", then "reciprocals <tried> <wrong>".
//   quotient_check <seed>
#include "exact_quotient.hpp"
#include <cstdio>
#include <cstdlib>
#include <vector>

using sofie_hip::quotient_by_reciprocal;
using sofie_hip::quotient_plan;
using sofie_hip::reciprocal_rn;

static float from_bits(uint32_t b)
{
   float f;
   std::memcpy(&f, &b, 4);
   return f;
}
static uint32_t bits_of(float f)
{
   uint32_t b;
   std::memcpy(&b, &f, 4);
   return b;
}
static uint64_t rng_state = 1;
static uint32_t rng()
{
   rng_state = rng_state * 6364136223846793005ull + 1442695040888963407ull;
   return (uint32_t)(rng_state >> 32);
}

int main(int argc, char **argv)
{
   rng_state = argc > 1 ? strtoull(argv[1], nullptr, 0) : 1;
   std::vector<float> qs = {1.0f, 2.0f, 3.0f, 10.0f, 0.601829112f, 16.3691254f, -7.25f, 0x1p-30f, 0x1p40f, 0.1f, 1.9999996f /* significand 0x7ffffd */,
                            from_bits(0x3f800001u), 127.0f, 1.0f / 127.0f};
   for (int i = 0; i < 6; ++i)
      qs.push_back(from_bits(((97u + rng() % 70u) << 23) | (rng() & 0x7fffffu) | ((rng() & 1u) << 31))); // 2^-30 .. 2^39
   int status = 0;
   for (float q : qs) {
      float r;
      if (!quotient_plan(1.0f, q, r)) {
         std::printf("%.9g refused\n", q);
         status = 1;
         continue;
      }
      unsigned long long tried = 0, bad = 0;
      // every v with 2^-4 <= |v / q| < 2^10, roughly: the 15 binades of v around those of q, both signs
      const int eq = (int)((bits_of(q) >> 23) & 0xff);
      for (int e = eq - 5; e <= eq + 10; ++e) {
         if (e < 1 || e > 254)
            continue;
         for (uint32_t sign = 0; sign < 2; ++sign)
            for (uint32_t m = 0; m < (1u << 23); ++m) {
               const float v = from_bits((sign << 31) | ((uint32_t)e << 23) | m);
               const float want = v / q, got = quotient_by_reciprocal(v, q, r);
               ++tried;
               if (bits_of(want) != bits_of(got))
                  ++bad;
            }
      }
      // random v over the whole admitted range |v| in [2^-40, 2^61]: exact where |v / q| >= 1/4, below 1/2 in magnitude otherwise
      for (int i = 0; i < 4000000; ++i) {
         const float v = from_bits(((87u + rng() % 102u) << 23) | (rng() & 0x7fffffu) | ((rng() & 1u) << 31));
         const float want = v / q, got = quotient_by_reciprocal(v, q, r);
         ++tried;
         if (std::fabs(want) >= 0.25f ? bits_of(want) != bits_of(got) : !(std::fabs(got) < 0.5f))
            ++bad;
      }
      const float zero = quotient_by_reciprocal(0.0f, q, r);
      if (zero != 0.0f)
         ++bad;
      std::printf("%.9g %llu %llu\n", q, tried, bad);
      if (bad)
         status = 1;
   }
   // the reciprocal against quad precision
   unsigned long long rtried = 0, rbad = 0;
   for (int i = 0; i < 2000000; ++i) {
      const float q = from_bits(((97u + rng() % 70u) << 23) | (rng() & 0x7fffffu) | ((rng() & 1u) << 31));
      const float want = (float)((__float128)1 / (__float128)q);
      ++rtried;
      if (bits_of(want) != bits_of(reciprocal_rn(q)))
         ++rbad;
   }
   std::printf("reciprocals %llu %llu\n", rtried, rbad);
   // divisors that must be refused
   float r;
   const float refused[] = {0.0f, INFINITY, NAN, 0x1p-31f, 0x1p41f, from_bits(0x3fffffffu)};
   for (float q : refused)
      if (quotient_plan(1.0f, q, r)) {
         std::printf("%.9g admitted\n", q);
         status = 1;
      }
   const float bad_scales[] = {INFINITY, NAN, 0x1p-41f, 0x1p31f};
   for (float s : bad_scales)
      if (quotient_plan(s, 3.0f, r)) {
         std::printf("scale %.9g admitted\n", s);
         status = 1;
      }
   if (!quotient_plan(0.0f, 3.0f, r)) {
      std::printf("scale 0 refused\n");
      status = 1;
   }
   return status | (rbad ? 1 : 0);
}
