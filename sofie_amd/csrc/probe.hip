// Register-only int8 MFMA loop: what the matrix cores of this board sustain with no memory traffic at
// all.  With operands that toggle every instruction the board clocks down under its power limit, so
// this, and not the data-sheet figure, is the ceiling a GEMM on random int8 data can approach.
#include "mfma8_common.hpp"

namespace sofie_hip {

__device__ __forceinline__ unsigned probe_hash(unsigned x)
{
   x ^= x >> 16;
   x *= 0x7feb352dU;
   x ^= x >> 15;
   x *= 0x846ca68bU;
   x ^= x >> 16;
   return x;
}

template <int RANDOM>
__global__ __launch_bounds__(256) void mfma_i8_probe_kernel(int *out, int iters, int seed)
{
   v16i acc[8];
#pragma unroll
   for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v)
         acc[i][v] = 0;
   v4i a[8], b[8];
#pragma unroll
   for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
         a[i][j] = RANDOM ? (int)probe_hash(seed * 977 + threadIdx.x * 131 + i * 17 + j) : 0x01010101;
         b[i][j] = RANDOM ? (int)probe_hash(seed * 31 + threadIdx.x * 7 + i * 29 + j + 1000) : 0x01010101;
      }
   for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
         acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b[(i + 3) & 7], acc[i], 0, 0, 0);
#pragma unroll
      for (int i = 0; i < 8; ++i)
         acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[(i + 5) & 7], b[i], acc[i], 0, 0, 0);
   }
   int s = 0;
#pragma unroll
   for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v)
         s += acc[i][v];
   out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

} // namespace sofie_hip

using namespace sofie_hip;

extern "C" int sofie_hip_mfma_i8_probe(sofie_hip_ctx *ctx, void *scratch, size_t scratch_bytes, int32_t iters, int32_t random_operands,
                                       double *ops_per_second)
{
   SOFIE_HIP_REQUIRE(ctx && scratch && ops_per_second, "sofie_hip_mfma_i8_probe: NULL argument");
   SOFIE_HIP_REQUIRE(iters > 0 && iters <= 1000000, "sofie_hip_mfma_i8_probe: iters out of range");
   hipDeviceProp_t prop;
   SOFIE_HIP_CHECK(hipGetDeviceProperties(&prop, ctx->device));
   const int wgs = prop.multiProcessorCount; // one workgroup of 4 waves per CU: one wave per SIMD
   SOFIE_HIP_REQUIRE(scratch_bytes >= (size_t)wgs * 256 * 4, "sofie_hip_mfma_i8_probe: scratch of %zu bytes needed", (size_t)wgs * 256 * 4);
   float best = 0.0f;
   for (int rep = 0; rep < 3; ++rep) {
      SOFIE_HIP_CHECK(hipEventRecord(ctx->ev0, ctx->stream));
      if (random_operands)
         hipLaunchKernelGGL(mfma_i8_probe_kernel<1>, dim3(wgs), dim3(256), 0, ctx->stream, (int *)scratch, iters, rep + 1);
      else
         hipLaunchKernelGGL(mfma_i8_probe_kernel<0>, dim3(wgs), dim3(256), 0, ctx->stream, (int *)scratch, iters, rep + 1);
      SOFIE_HIP_CHECK(hipEventRecord(ctx->ev1, ctx->stream));
      SOFIE_HIP_CHECK(hipEventSynchronize(ctx->ev1));
      float ms = 0.0f;
      SOFIE_HIP_CHECK(hipEventElapsedTime(&ms, ctx->ev0, ctx->ev1));
      if (rep == 0 || ms < best)
         best = ms;
   }
   const double ops = 2.0 * (double)wgs * 4 * (double)iters * 16 * 32768.0;
   *ops_per_second = ops / ((double)best * 1e-3);
   return SOFIE_HIP_OK;
}
