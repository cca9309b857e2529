// FP8 (OCP e4m3fn) GEMM on the gfx950 matrix cores (v_mfma_f32_32x32x64_f8f6f4, fp32 accumulate) with
// scale + bias + activation + bf16 conversion fused into the store, and the fp32 -> e4m3fn quantiser.
#include "mfma8_dispatch.hpp"

namespace sofie_hip {

// fp32 -> bf16 bits, round to nearest even; NaN stays NaN.
__device__ __forceinline__ uint16_t f32_to_bf16_rne(float x)
{
   uint32_t u = __float_as_uint(x);
   if ((u & 0x7fffffffu) > 0x7f800000u)
      return (uint16_t)((u >> 16) | 0x40);
   u += 0x7fffu + ((u >> 16) & 1u);
   return (uint16_t)(u >> 16);
}

// Two fp32 -> two bf16 in one dword (round to nearest even, NaN stays a quiet NaN): one v_cvt_pk_bf16_f32.
__device__ __forceinline__ uint32_t pack_bf16_rne(float lo, float hi)
{
   typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
   typedef float f32x2 __attribute__((ext_vector_type(2)));
   const f32x2 v = {lo, hi};
   return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}

// fp32 -> e4m3fn code, round to nearest even, saturating at +-448 (also +-inf); NaN -> 0x7f.
__device__ __forceinline__ uint8_t f32_to_e4m3_rne_sat(float x)
{
   uint32_t u = __float_as_uint(x);
   uint8_t sign = (uint8_t)((u >> 24) & 0x80);
   if ((u & 0x7fffffffu) > 0x7f800000u)
      return 0x7f;
   float a = fabsf(x);
   if (a >= 448.0f)
      return sign | 0x7e;
   int e = (int)((u >> 23) & 0xff) - 127; // exponent of the leading bit (denormal fp32 -> far below range)
   if (e < -6)
      e = -6;
   float q = __builtin_rintf(ldexpf(a, 3 - e)); // a / 2^(e-3), exact; ties to even
   float r = ldexpf(q, e - 3);
   if (r < 0.015625f) // 2^-6: subnormal codes, quantum 2^-9
      return sign | (uint8_t)(int)ldexpf(r, 9);
   uint32_t ur = __float_as_uint(r);
   int er = (int)((ur >> 23) & 0xff) - 127;
   return sign | (uint8_t)((er + 7) << 3) | (uint8_t)((ur >> 20) & 7);
}

__global__ __launch_bounds__(256) void quantize_fp8_kernel(uint8_t *__restrict__ dst, const float *__restrict__ src, size_t n,
                                                            float scale)
{
   const size_t stride = (size_t)gridDim.x * blockDim.x;
   for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += stride)
      dst[i] = f32_to_e4m3_rne_sat(__fdiv_rn(src[i], scale));
}

// GELU (erf form) for the FP8 store, v Phi(v) with Phi from the rational approximation 7.1.26 of Abramowitz & Stegun,
//   erfc(z) = (a1 t + ... + a5 t^5) exp(-z^2),  t = 1/(1 + p z),  z = |v| / sqrt 2 >= 0,   |error| <= 1.5e-7,
// one exponential and one reciprocal per element instead of the library erff (the tile store of a 256 x 256 tile evaluates
// it 256 times per lane, which with erff costs half as much as the whole K loop).  Written in v directly: the factor 1/2 of
// Phi(-|v|) = erfc(z) / 2 sits in the coefficients, p / sqrt 2 in the reciprocal's argument, and exp(-z^2) is
// 2^-(v sqrt(log2(e) / 2))^2, the hardware's own exponential.  The reciprocal is the hardware's too (v_rcp_f32, one ulp): the
// correctly rounded one is a division sequence of ten instructions.  Sixteen plain instructions and the two transcendental
// ones; the absolute error of the result, <= 5e-7 |v|, is far inside the FP8 GEMM's stated bound.
__device__ __forceinline__ float gelu_erf_fast(float v)
{
   const float t = __builtin_amdgcn_rcpf(__fmaf_rn(0.23164189f, fabsf(v), 1.0f));
   float poly = __fmaf_rn(t, 0.5306527145f, -0.7265760135f);
   poly = __fmaf_rn(t, poly, 0.7107068705f);
   poly = __fmaf_rn(t, poly, -0.142248368f);
   poly = __fmaf_rn(t, poly, 0.127414796f);
   poly = __fmul_rn(poly, t);
   const float u = __fmul_rn(v, 0.8493218003f);
   const float h = __fmul_rn(poly, __builtin_amdgcn_exp2f(-__fmul_rn(u, u))); // Phi(-|v|)
   const float phi = (v < 0.0f) ? h : (1.0f - h);
   return __fmul_rn(v, phi);
}

// GELU (erf form) for the bf16 store: v * Phi(v) with Phi(v) - 1/2 an odd polynomial of degree 15 in v clamped to [-4, 4]
// (minimax for |v * error|; beyond the clamp Phi is taken as Phi(+-4), 3e-5 off).  Eleven plain instructions, no exponential, no
// reciprocal: |error| <= 8e-5 |v|, a fiftieth of the half ulp of a bf16 result, where the fp32 store above keeps 1e-6 |v|.
__device__ __forceinline__ float gelu_erf_for_bf16(float v)
{
   const float c = __builtin_amdgcn_fmed3f(v, -4.0f, 4.0f);
   const float s = __fmul_rn(c, c);
   float q = __fmaf_rn(s, -1.3012979351e-09f, 1.0419626164e-07f);
   q = __fmaf_rn(s, q, -3.6571383814e-06f);
   q = __fmaf_rn(s, q, 7.4855119269e-05f);
   q = __fmaf_rn(s, q, -1.0064909419e-03f);
   q = __fmaf_rn(s, q, 9.5054004836e-03f);
   q = __fmaf_rn(s, q, -6.5887847274e-02f);
   q = __fmaf_rn(s, q, 3.9867339703e-01f);
   return __fmul_rn(v, __fmaf_rn(c, q, 0.5f));
}

struct F8Epilogue {
   static constexpr bool kConvertInRegisters = false; // activation (erf, tanh, exp) + bf16 rounding per element: keep the code once
   const float *bias;
   float scale;
   int act, out;
   void *Y;
   int ldy;
   int stage_ok;
   int N;

   // The store is compiled once per (output type, activation class): MODE = out | class << 1, class 0 = none, 1 = relu,
   // 2 = gelu (erf form), 3 = any other activation, chosen per element at run time.  With the activation a compile-time
   // constant the conversion of one element is a few instructions (about 25 for gelu); with the run-time switch every
   // element of an unrolled tile store carries the code of all of them, and the store of a 256 x 256 tile took 26 us.
   static constexpr int kClassNone = 0, kClassRelu = 1, kClassGelu = 2, kClassAny = 3;
   template <class F>
   __device__ __forceinline__ void dispatch(F f) const
   {
      const int cls = act == SOFIE_ACT_NONE ? kClassNone : act == SOFIE_ACT_RELU ? kClassRelu : act == SOFIE_ACT_GELU ? kClassGelu : kClassAny;
      switch ((out == SOFIE_F8OUT_F32 ? 1 : 0) | (cls << 1)) {
      case 0: f(std::integral_constant<int, 0>{}); break;
      case 1: f(std::integral_constant<int, 1>{}); break;
      case 2: f(std::integral_constant<int, 2>{}); break;
      case 3: f(std::integral_constant<int, 3>{}); break;
      case 4: f(std::integral_constant<int, 4>{}); break;
      case 5: f(std::integral_constant<int, 5>{}); break;
      case 6: f(std::integral_constant<int, 6>{}); break;
      default: f(std::integral_constant<int, 7>{}); break;
      }
   }
   // the names the pipelined and the persistent kernel call (the int8 store has one more mode in each)
   template <class F>
   __device__ __forceinline__ void dispatch_for_registers(F f) const
   {
      dispatch(f);
   }
   template <class F>
   __device__ __forceinline__ void dispatch_with_reciprocal(F f) const
   {
      dispatch(f);
   }
   template <int MODE>
   static constexpr int out_bytes()
   {
      return (MODE & 1) ? 4 : 2;
   }
   __device__ __forceinline__ bool rows_vectorizable() const { return stage_ok != 0; }
   __device__ __forceinline__ char *out_base() const { return (char *)Y; }
   __device__ __forceinline__ size_t out_index(int m, int n) const { return (size_t)m * (size_t)ldy + n; }
   __device__ __forceinline__ size_t out_index_of_plain_rows(int m, int n) const { return out_index(m, n); }
   template <int C>
   struct col_params {
      float b[C];
   };
   template <int C>
   __device__ __forceinline__ void load_params(int n, col_params<C> &p) const
   {
#pragma unroll
      for (int i = 0; i < C; ++i)
         p.b[i] = bias ? bias[n + i < N ? n + i : N - 1] : -0.0f; // -0: the neutral element of the addition
   }
   // the constants of one column as 32-bit words (what the register tile store hands from lane to lane): the bias
   static constexpr int kColWords = 1;
   static constexpr bool kBiasInAccumulator = false; // floating-point sums: the bias is added to the finished sum, as the definition has it
   static constexpr int kBiasWord = 0;
   __device__ __forceinline__ void load_column(int n, uint32_t (&w)[kColWords]) const { w[0] = __float_as_uint(bias ? bias[n] : -0.0f); }
   __device__ __forceinline__ void load_column_for_registers(int n, uint32_t (&w)[kColWords]) const { load_column(n, w); }
   template <int C>
   static __device__ __forceinline__ void set_column(col_params<C> &p, int i, const uint32_t (&w)[kColWords])
   {
      p.b[i] = __uint_as_float(w[0]);
   }
   // row-major output with 16-byte aligned rows (what the register tile store handles)
   bool stores_plain_rows() const { return stage_ok != 0; }
   int elements_per_16_bytes() const { return out == SOFIE_F8OUT_F32 ? 4 : 8; }
   // v = acc*scale + bias[n]; activation in fp32; then fp32 or bf16 (round to nearest even)
   template <int MODE, int C>
   __device__ __forceinline__ void pack4(const col_params<C> &p, int q, float a0, float a1, float a2, float a3, uint32_t *w) const
   {
      constexpr int cls = MODE >> 1;
      const float a[4] = {a0, a1, a2, a3};
      float v[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
         v[i] = mul_nofma(a[i], scale) + p.b[4 * q + i]; // without a bias the constant is -0, which leaves every v as it is
         if constexpr (cls == kClassRelu)
            v[i] = apply_activation(v[i], SOFIE_ACT_RELU, 0.0f);
         else if constexpr (cls == kClassGelu)
            v[i] = (MODE & 1) ? gelu_erf_fast(v[i]) : gelu_erf_for_bf16(v[i]);
         else if constexpr (cls == kClassAny)
            v[i] = apply_activation(v[i], act, 0.0f);
      }
      if constexpr (MODE & 1) {
#pragma unroll
         for (int i = 0; i < 4; ++i)
            w[i] = __float_as_uint(v[i]);
      } else {
         w[0] = pack_bf16_rne(v[0], v[1]);
         w[1] = pack_bf16_rne(v[2], v[3]);
      }
   }
};

} // namespace sofie_hip

using namespace sofie_hip;

extern "C" {

int sofie_hip_quantize_fp8(sofie_hip_ctx *ctx, uint8_t *dst, const float *src, size_t n, float scale)
{
   SOFIE_HIP_REQUIRE(ctx != nullptr, "sofie_hip_quantize_fp8: ctx is NULL");
   if (n == 0)
      return SOFIE_HIP_OK;
   SOFIE_HIP_REQUIRE(dst && src, "sofie_hip_quantize_fp8: NULL pointer");
   SOFIE_HIP_REQUIRE(scale > 0.0f, "sofie_hip_quantize_fp8: scale must be positive");
   size_t blocks = (n + 255) / 256;
   if (blocks > 8192)
      blocks = 8192;
   hipLaunchKernelGGL(quantize_fp8_kernel, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, dst, src, n, scale);
   return launch_status("quantize_fp8_kernel");
}

int sofie_hip_gemm_fp8(sofie_hip_ctx *ctx, const sofie_gemm_fp8_desc *d)
{
   SOFIE_HIP_REQUIRE(ctx && d, "sofie_hip_gemm_fp8: NULL argument");
   SOFIE_HIP_REQUIRE(d->M >= 0 && d->N >= 0 && d->K >= 0, "sofie_hip_gemm_fp8: negative dimension");
   SOFIE_HIP_REQUIRE(d->out == SOFIE_F8OUT_BF16 || d->out == SOFIE_F8OUT_F32, "sofie_hip_gemm_fp8: unknown output kind %d", d->out);
   SOFIE_HIP_REQUIRE(d->act >= SOFIE_ACT_NONE && d->act <= SOFIE_ACT_TANH && d->act != SOFIE_ACT_LEAKYRELU,
                     "sofie_hip_gemm_fp8: unsupported activation %d", d->act);
   if (d->M == 0 || d->N == 0)
      return SOFIE_HIP_OK;
   SOFIE_HIP_REQUIRE(d->Y != nullptr, "sofie_hip_gemm_fp8: Y is NULL");
   SOFIE_HIP_REQUIRE(d->K == 0 || (d->A && d->B), "sofie_hip_gemm_fp8: A or B is NULL");
   const int M = d->M, N = d->N, K = d->K;
   int lda = d->lda ? d->lda : K;
   int ldb = d->ldb ? d->ldb : (d->transB ? K : N);
   int ldy = d->ldy ? d->ldy : N;
   SOFIE_HIP_REQUIRE(lda >= K && ldb >= (d->transB ? K : N) && ldy >= N, "sofie_hip_gemm_fp8: leading dimension too small");
   const int8_t *A = (const int8_t *)d->A, *Bt = (const int8_t *)d->B;
   if (K > 0 && !d->transB) {
      size_t need = (((size_t)K * (size_t)N) + 255) & ~(size_t)255;
      SOFIE_HIP_REQUIRE(d->workspace != nullptr && d->workspace_bytes >= need,
                        "sofie_hip_gemm_fp8: B is [K,N]; a workspace of %zu bytes is needed to re-lay it out", need);
      SOFIE_HIP_REQUIRE(((uintptr_t)d->workspace & 255) == 0, "sofie_hip_gemm_fp8: workspace must be 256-byte aligned");
      int st = transpose_i8(ctx->stream, (int8_t *)d->workspace, (const int8_t *)d->B, K, N, ldb, K);
      if (st)
         return st;
      Bt = (const int8_t *)d->workspace;
      ldb = K;
   }
   F8Epilogue ep;
   ep.bias = d->bias;
   ep.scale = d->scale;
   ep.act = d->act;
   ep.out = d->out;
   ep.Y = d->Y;
   ep.ldy = ldy;
   ep.N = N;
   const size_t esz = d->out == SOFIE_F8OUT_F32 ? 4 : 2;
   ep.stage_ok = (((size_t)ldy * esz) % 16 == 0) && (((uintptr_t)d->Y & 15) == 0);
   if (K == 0) {
      A = (const int8_t *)d->Y;
      Bt = (const int8_t *)d->Y;
      lda = ldb = 16;
   }
   return launch_mfma8_best<MfmaF8, F8Epilogue>(launch_cfg_f8(ctx), A, Bt, M, N, K, lda, ldb, ep);
}

} // extern "C"
