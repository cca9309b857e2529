// Store stage of the int8 GEMM and of the int8 convolution: bias, requantisation or dequantisation,
// optional relu, and the output addressing (row-major [M,N], or NCHW when the GEMM rows are the
// output pixels of a convolution).
#pragma once
#include "mfma8_gemm.hpp"

namespace sofie_hip {

struct I8Epilogue {
   const int32_t *bias;
   const float *scale;
   float scale_scalar;
   float q_scale;
   int relu_acc, relu_out, out;
   void *Y;
   int ldy;
   int vec_store; // Y/ldy alignment allows vector stores of 4 consecutive columns
   int N;         // number of valid columns
   int nchw_ohw;  // 0: Y[m*ldy + n]; else m = (img, pix) and Y[(img*ldy + n)*nchw_ohw + pix], ldy = Cout
   int n_offset;  // added to n for bias/scale/Y addressing (grouped convolution)

   __device__ __forceinline__ void store_one(size_t idx, int acc, float s) const
   {
      switch (out) {
      case SOFIE_I8OUT_I32: ((int32_t *)Y)[idx] = acc; break;
      case SOFIE_I8OUT_F32: {
         float v = mul_nofma((float)acc, s);
         if (relu_out)
            v = v > 0.0f ? v : 0.0f;
         ((float *)Y)[idx] = v;
      } break;
      case SOFIE_I8OUT_I8: {
         int q = quantize_rne_sat8(mul_nofma((float)acc, s));
         if (relu_out)
            q = q > 0 ? q : 0;
         ((int8_t *)Y)[idx] = (int8_t)q;
      } break;
      default: ((int8_t *)Y)[idx] = (int8_t)quantize_rne_sat8(__fdiv_rn(mul_nofma((float)acc, s), q_scale)); break;
      }
   }

   // 4 consecutive columns n..n+3 of row m; `a*` hold the exact int32 dot products.
   __device__ __forceinline__ void store4(int m, int n, int a0, int a1, int a2, int a3) const
   {
      int acc[4] = {a0, a1, a2, a3};
      float s[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
         int nn = (n + i < N ? n + i : N - 1) + n_offset;
         int b = bias ? bias[nn] : 0;
         s[i] = scale ? scale[nn] : scale_scalar;
         acc[i] += b;
         if (relu_acc)
            acc[i] = acc[i] > 0 ? acc[i] : 0;
      }
      if (nchw_ohw) {
         const int img = m / nchw_ohw, pix = m - img * nchw_ohw;
#pragma unroll
         for (int i = 0; i < 4; ++i)
            if (n + i < N)
               store_one(((size_t)img * ldy + (n + i + n_offset)) * nchw_ohw + pix, acc[i], s[i]);
         return;
      }
      const size_t row = (size_t)m * (size_t)ldy + n + n_offset;
      if (!((n + 3 < N) && vec_store)) {
#pragma unroll
         for (int i = 0; i < 4; ++i)
            if (n + i < N)
               store_one(row + i, acc[i], s[i]);
         return;
      }
      switch (out) {
      case SOFIE_I8OUT_I32: *(v4i *)((int32_t *)Y + row) = v4i{acc[0], acc[1], acc[2], acc[3]}; break;
      case SOFIE_I8OUT_F32: {
         float v[4];
#pragma unroll
         for (int i = 0; i < 4; ++i) {
            v[i] = mul_nofma((float)acc[i], s[i]);
            if (relu_out)
               v[i] = v[i] > 0.0f ? v[i] : 0.0f;
         }
         *(float4 *)((float *)Y + row) = make_float4(v[0], v[1], v[2], v[3]);
      } break;
      default: {
         int q[4];
#pragma unroll
         for (int i = 0; i < 4; ++i) {
            if (out == SOFIE_I8OUT_I8) {
               q[i] = quantize_rne_sat8(mul_nofma((float)acc[i], s[i]));
               if (relu_out)
                  q[i] = q[i] > 0 ? q[i] : 0;
            } else {
               q[i] = quantize_rne_sat8(__fdiv_rn(mul_nofma((float)acc[i], s[i]), q_scale));
            }
         }
         *(uint32_t *)((int8_t *)Y + row) = (uint32_t)(q[0] & 0xff) | ((uint32_t)(q[1] & 0xff) << 8) |
                                            ((uint32_t)(q[2] & 0xff) << 16) | ((uint32_t)(q[3] & 0xff) << 24);
      } break;
      }
   }
};

// Y = epilogue(A[M,K] * Bt[N,K]^T); fills ep.vec_store and ep.N.  force_tile 0 = heuristic.
int gemm_i8_nt(hipStream_t stream, const int8_t *A, const int8_t *Bt, int M, int N, int K, int lda, int ldb, I8Epilogue ep,
               int force_tile);
int forced_i8_tile();

} // namespace sofie_hip
