// fp32 Gemm / MatMul and fp32 convolution (implicit GEMM) with the bias + activation epilogue fused
// into the store.  These are the small-batch, HBM/latency-bound operators of the fp32 path: tiles of
// 64x64 outputs, K walked in slabs of 16 staged through LDS, 4x4 outputs per lane, fp32 FMA.
// The operand fetch is a functor, so the same tile loop serves a strided/transposed Gemm and a
// convolution whose column matrix is gathered on the fly (no materialised im2col).
#include "common.hpp"
#include <cstdlib>

namespace sofie_hip {

constexpr int F32_BM = 64, F32_BN = 64, F32_BK = 16;

struct GemmOperandA {
   const float *p;
   long long sm, sk; // element strides of op(A)[m,k]
   __device__ __forceinline__ float operator()(int m, int k) const { return p[m * sm + k * sk]; }
};
struct GemmOperandB {
   const float *p;
   long long sk, sn; // element strides of op(B)[k,n]
   __device__ __forceinline__ float operator()(int k, int n) const { return p[k * sk + n * sn]; }
};

struct F32Epilogue {
   float alpha, beta;
   const float *C;
   int bias_mode;
   long long ldc;
   PostChain chain; // the activation, then the caller's chain of one-to-one operators
   const float *R;  // tensor of Y's shape added before the activation, or nullptr
   long long ldr;
};

__device__ __forceinline__ float f32_epilogue(const F32Epilogue &ep, float acc, int m, int n)
{
   float v = ep.alpha * acc;
   switch (ep.bias_mode) {
   case SOFIE_BIAS_ROW: v += ep.C[n]; break;
   case SOFIE_BIAS_COL: v += ep.C[m]; break;
   case SOFIE_BIAS_SCALAR: v += ep.C[0]; break;
   case SOFIE_BIAS_FULL: v += ep.beta * ep.C[m * ep.ldc + n]; break;
   default: break;
   }
   if (ep.R)
      v += ep.R[m * ep.ldr + n];
   return apply_chain(v, ep.chain);
}

// The tile loop: acc[4][4] per lane over a 64x64 tile.  LA(m,k), LB(k,n) return 0-safe values only for
// in-range indices; the loop bounds-checks before calling them.
template <class LA, class LB>
__device__ __forceinline__ void f32_tile_loop(const LA &la, const LB &lb, int M, int N, int K, int m0, int n0,
                                              float (&acc)[4][4])
{
   __shared__ float sA[F32_BK][F32_BM + 4];
   __shared__ float sB[F32_BK][F32_BN + 4];
   const int t = threadIdx.x;
   const int tx = t & 15, ty = t >> 4; // 16x16 lanes, each 4x4 outputs
#pragma unroll
   for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
         acc[i][j] = 0.0f;

   for (int k0 = 0; k0 < K; k0 += F32_BK) {
      // 64x16 elements of each operand, 256 threads -> 4 each
#pragma unroll
      for (int i = 0; i < 4; ++i) {
         int id = t + i * 256;
         int kk = id & 15, mm = id >> 4; // k fastest for A: consecutive lanes walk k
         int m = m0 + mm, k = k0 + kk;
         sA[kk][mm] = (m < M && k < K) ? la(m, k) : 0.0f;
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
         int id = t + i * 256;
         int nn = id & 63, kk = id >> 6; // n fastest for B
         int n = n0 + nn, k = k0 + kk;
         sB[kk][nn] = (n < N && k < K) ? lb(k, n) : 0.0f;
      }
      __syncthreads();
#pragma unroll
      for (int kk = 0; kk < F32_BK; ++kk) {
         float a[4], b[4];
#pragma unroll
         for (int i = 0; i < 4; ++i)
            a[i] = sA[kk][ty * 4 + i];
#pragma unroll
         for (int j = 0; j < 4; ++j)
            b[j] = sB[kk][tx * 4 + j];
#pragma unroll
         for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
               acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
      }
      __syncthreads();
   }
}

__global__ __launch_bounds__(256) void gemm_f32_kernel(GemmOperandA la, GemmOperandB lb, int M, int N, int K, float *Y,
                                                        long long ldy, F32Epilogue ep, long long strideA, long long strideB,
                                                        long long strideC, long long strideY)
{
   const int b = blockIdx.z;
   la.p += b * strideA;
   lb.p += b * strideB;
   if (ep.C)
      ep.C += b * strideC;
   if (ep.R)
      ep.R += b * strideY;
   Y += b * strideY;
   const int m0 = blockIdx.x * F32_BM, n0 = blockIdx.y * F32_BN;
   float acc[4][4];
   f32_tile_loop(la, lb, M, N, K, m0, n0, acc);
   const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
#pragma unroll
   for (int i = 0; i < 4; ++i) {
      int m = m0 + ty * 4 + i;
      if (m >= M)
         continue;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
         int n = n0 + tx * 4 + j;
         if (n < N)
            Y[m * ldy + n] = f32_epilogue(ep, acc[i][j], m, n);
      }
   }
}

// Small products (the fp32 MLP at batch 64 has 64x128, 64x64 and 64x10 outputs): the 64x64 tiles above would
// occupy a handful of CUs and spend their time waiting for one 16-wide K slab after another.  Here a
// workgroup is ONE wave that owns an 8x8 tile, one output per lane, so even these products spread over
// more than a hundred CUs.  K is walked in chunks of 256: the 8 rows of op(A) and the 8 columns of op(B)
// are staged in LDS with K contiguous (row pitch 260 floats: the 8 rows a wave reads at once fall into
// different banks), the next chunk's loads are issued before the current chunk is consumed, and a lane
// reads 4 K values of its row and its column per step into four partial sums (k mod 4), added at the end.
constexpr int SK_T = 8, SK_KC = 256, SK_PITCH = SK_KC + 4;

template <bool VEC_A, bool VEC_B>
__global__ __launch_bounds__(64) void gemm_f32_skinny_kernel(GemmOperandA la, GemmOperandB lb, int M, int N, int K, float *Y,
                                                              long long ldy, F32Epilogue ep, long long strideA, long long strideB,
                                                              long long strideC, long long strideY)
{
   __shared__ __attribute__((aligned(16))) float sA[2][SK_T][SK_PITCH];
   __shared__ __attribute__((aligned(16))) float sB[2][SK_T][SK_PITCH];
   const int b = blockIdx.z;
   la.p += b * strideA;
   lb.p += b * strideB;
   if (ep.C)
      ep.C += b * strideC;
   if (ep.R)
      ep.R += b * strideY;
   Y += b * strideY;
   const int lane = threadIdx.x;
   const int tm = lane >> 3, tn = lane & 7;
   const int m0 = blockIdx.x * SK_T, n0 = blockIdx.y * SK_T;

   // staging registers of one chunk: row i of the tile, K values 4*lane..4*lane+3 (vector form), or
   // element lane + 64*j of the 8x256 block (scalar form, any strides)
   float4 ra[SK_T], rb[SK_T];
   float qa[VEC_A ? 1 : 32], qb[VEC_B ? 1 : 32];
   auto fetch = [&](int k0) {
      if (VEC_A) {
#pragma unroll
         for (int i = 0; i < SK_T; ++i) {
            const int m = m0 + i, k = k0 + lane * 4;
            ra[i] = (m < M && k < K) ? *(const float4 *)(la.p + m * la.sm + k) : make_float4(0.f, 0.f, 0.f, 0.f);
         }
      } else {
#pragma unroll
         for (int j = 0; j < 32; ++j) {
            const int id = lane + 64 * j, row = id & 7, kk = id >> 3; // rows fastest: a transposed operand is contiguous there
            const int m = m0 + row, k = k0 + kk;
            qa[j] = (m < M && k < K) ? la(m, k) : 0.0f;
         }
      }
      if (VEC_B) {
#pragma unroll
         for (int i = 0; i < SK_T; ++i) {
            const int n = n0 + i, k = k0 + lane * 4;
            rb[i] = (n < N && k < K) ? *(const float4 *)(lb.p + n * lb.sn + k) : make_float4(0.f, 0.f, 0.f, 0.f);
         }
      } else {
#pragma unroll
         for (int j = 0; j < 32; ++j) {
            const int id = lane + 64 * j, row = id & 7, kk = id >> 3;
            const int n = n0 + row, k = k0 + kk;
            qb[j] = (n < N && k < K) ? lb(k, n) : 0.0f;
         }
      }
   };
   auto stage = [&](int buf) {
      if (VEC_A) {
#pragma unroll
         for (int i = 0; i < SK_T; ++i)
            *(float4 *)&sA[buf][i][lane * 4] = ra[i];
      } else {
#pragma unroll
         for (int j = 0; j < 32; ++j) {
            const int id = lane + 64 * j;
            sA[buf][id & 7][id >> 3] = qa[j];
         }
      }
      if (VEC_B) {
#pragma unroll
         for (int i = 0; i < SK_T; ++i)
            *(float4 *)&sB[buf][i][lane * 4] = rb[i];
      } else {
#pragma unroll
         for (int j = 0; j < 32; ++j) {
            const int id = lane + 64 * j;
            sB[buf][id & 7][id >> 3] = qb[j];
         }
      }
   };

   float acc4[4] = {0.0f, 0.0f, 0.0f, 0.0f}; // k = 0,1,2,3 (mod 4): four independent FMA chains, added at the end
   fetch(0);
   int buf = 0;
   for (int k0 = 0; k0 < K; k0 += SK_KC) {
      stage(buf);
      if (k0 + SK_KC < K)
         fetch(k0 + SK_KC); // in flight while this chunk is consumed
      __builtin_amdgcn_wave_barrier();
      const int kc = (K - k0) < SK_KC ? (K - k0) : SK_KC;
#pragma unroll 4
      for (int kk = 0; kk < kc; kk += 4) {
         const float4 a = *(const float4 *)&sA[buf][tm][kk];
         const float4 c = *(const float4 *)&sB[buf][tn][kk];
         acc4[0] = fmaf(a.x, c.x, acc4[0]);
         acc4[1] = fmaf(a.y, c.y, acc4[1]);
         acc4[2] = fmaf(a.z, c.z, acc4[2]);
         acc4[3] = fmaf(a.w, c.w, acc4[3]);
      }
      buf ^= 1;
   }
   const float acc = (acc4[0] + acc4[1]) + (acc4[2] + acc4[3]);
   const int m = m0 + tm, n = n0 + tn;
   if (m < M && n < N)
      Y[m * ldy + n] = f32_epilogue(ep, acc, m, n);
}

// Column-matrix element (row m = (image, oh, ow), column k = (ci, kh, kw)) gathered from NCHW input;
// the same index arithmetic as the reference's Im2col, zero outside the image.
struct ConvOperandA {
   const float *X;
   int C, H, W, kh, kw, OH, OW, pad_h0, pad_w0, stride_h, stride_w, dil_h, dil_w;
   int c_first; // first input channel of this group
   __device__ __forceinline__ float operator()(int m, int k) const
   {
      int ow = m % OW, t = m / OW;
      int oh = t % OH, img = t / OH;
      int kx = k % kw, t2 = k / kw;
      int ky = t2 % kh, ci = t2 / kh;
      int ih = oh * stride_h - pad_h0 + ky * dil_h;
      int iw = ow * stride_w - pad_w0 + kx * dil_w;
      if ((unsigned)ih >= (unsigned)H || (unsigned)iw >= (unsigned)W)
         return 0.0f;
      return X[(((size_t)img * C + c_first + ci) * H + ih) * W + iw];
   }
};
// The same for three spatial dimensions (the reference's Im2col_3d): row m = (image, od, oh, ow), column k = (ci, kd, kh, kw).
struct Conv3dOperandA {
   const float *X;
   int C, D, H, W, kd, kh, kw, OD, OH, OW, pad_d0, pad_h0, pad_w0, stride_d, stride_h, stride_w, dil_d, dil_h, dil_w;
   int c_first;
   __device__ __forceinline__ float operator()(int m, int k) const
   {
      int ow = m % OW, t = m / OW;
      int oh = t % OH;
      t /= OH;
      int od = t % OD, img = t / OD;
      int kx = k % kw, t2 = k / kw;
      int ky = t2 % kh;
      t2 /= kh;
      int kz = t2 % kd, ci = t2 / kd;
      int id = od * stride_d - pad_d0 + kz * dil_d;
      int ih = oh * stride_h - pad_h0 + ky * dil_h;
      int iw = ow * stride_w - pad_w0 + kx * dil_w;
      if ((unsigned)id >= (unsigned)D || (unsigned)ih >= (unsigned)H || (unsigned)iw >= (unsigned)W)
         return 0.0f;
      return X[((((size_t)img * C + c_first + ci) * D + id) * H + ih) * W + iw];
   }
};
struct ConvOperandB {
   const float *Wt; // [Cout_g][Kg] rows of this group
   int Kg;
   __device__ __forceinline__ float operator()(int k, int n) const { return Wt[(size_t)n * Kg + k]; }
};

template <class LA>
__global__ __launch_bounds__(256) void conv_f32_kernel(LA la, const float *Wt, const float *bias, float *Y, int M,
                                                        int Cout_g, int Kg, int Cg, int Cout, int OHW, PostChain chain, const float *R)
{
   const int g = blockIdx.z;
   la.c_first = g * Cg;
   ConvOperandB lb{Wt + (size_t)g * Cout_g * Kg, Kg};
   const int m0 = blockIdx.x * F32_BM, n0 = blockIdx.y * F32_BN;
   float acc[4][4];
   f32_tile_loop(la, lb, M, Cout_g, Kg, m0, n0, acc);
   const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
#pragma unroll
   for (int i = 0; i < 4; ++i) {
      int m = m0 + ty * 4 + i;
      if (m >= M)
         continue;
      int img = m / OHW, pix = m % OHW;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
         int n = n0 + tx * 4 + j;
         if (n < Cout_g) {
            int co = g * Cout_g + n;
            float v = acc[i][j];
            if (bias)
               v += bias[co];
            const size_t at = ((size_t)img * Cout + co) * OHW + pix;
            if (R)
               v += R[at];
            Y[at] = apply_chain(v, chain);
         }
      }
   }
}

} // namespace sofie_hip

namespace sofie_hip {

// ---- a chain of small products in one launch -----------------------------------------------------------------
// Layer l+1 reads what layer l wrote (an MLP at small batch): per layer launches cost more than the arithmetic, so one
// workgroup takes RB rows through every layer, the rows of activations staying in LDS between layers (each layer's
// output is also written to its Y, as separate launches would).  The weights stream from L2 once per workgroup:
//   transB (W stored [N][K], the ONNX export of a Linear layer): a wave takes 4 outputs at a time, its lanes stride over k
//     (coalesced 256-byte reads of each weight row), then the 64 partial sums are folded with shuffles;
//   else (W stored [K][N]): a thread owns output n and walks k (lanes read consecutive n of one weight row).
struct ChainLayerArgs {
   const float *B;
   long long ldb;
   int transB, N, K;
   float *Y;
   long long ldy;
   F32Epilogue ep;
};
struct ChainArgs {
   int count, M;
   const float *A;
   long long lda;
   ChainLayerArgs layer[SOFIE_MAX_GEMM_CHAIN];
};

// 16 waves per workgroup: what a layer costs is the round trips to L2 for its weights, and the waves' loads overlap
constexpr int CHAIN_THREADS = 1024;

template <int RB>
__global__ __launch_bounds__(CHAIN_THREADS) void gemm_chain_f32_kernel(ChainArgs a, int width)
{
   extern __shared__ float chain_lds[]; // two buffers of RB rows x width
   const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
   const int m0 = blockIdx.x * RB;
   const int rows = (a.M - m0) < RB ? (a.M - m0) : RB;
   float *in = chain_lds, *out = chain_lds + RB * width;
   // rows beyond the matrix are kept at zero so that the loops below need no row test
   if (rows < RB) {
      for (int i = t; i < 2 * RB * width; i += CHAIN_THREADS)
         chain_lds[i] = 0.0f;
      __syncthreads();
   }
   const int K0 = a.layer[0].K;
   for (int r = 0; r < rows; ++r)
      for (int k = t; k < K0; k += CHAIN_THREADS)
         in[r * width + k] = a.A[(long long)(m0 + r) * a.lda + k];
   __syncthreads();
   for (int l = 0; l < a.count; ++l) {
      const ChainLayerArgs &L = a.layer[l];
      const int N = L.N, K = L.K;
      const float *__restrict__ B = L.B;
      if (L.transB) {
         for (int n0 = wave * 4; n0 < N; n0 += CHAIN_THREADS / 16) {
            float acc[4][RB];
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
               for (int r = 0; r < RB; ++r)
                  acc[j][r] = 0.0f;
            // rows of W past N are read as row N-1 and their sums dropped
            const float *w0 = B + (long long)(n0 + 0 < N ? n0 + 0 : N - 1) * L.ldb;
            const float *w1 = B + (long long)(n0 + 1 < N ? n0 + 1 : N - 1) * L.ldb;
            const float *w2 = B + (long long)(n0 + 2 < N ? n0 + 2 : N - 1) * L.ldb;
            const float *w3 = B + (long long)(n0 + 3 < N ? n0 + 3 : N - 1) * L.ldb;
            // (issuing the loads of eight guarded k-positions at once instead, with no remainder loop, measured slower)
#pragma unroll 8
            for (int k = lane; k < K; k += 64) {
               const float w[4] = {w0[k], w1[k], w2[k], w3[k]};
#pragma unroll
               for (int r = 0; r < RB; ++r) {
                  const float x = in[r * width + k];
#pragma unroll
                  for (int j = 0; j < 4; ++j)
                     acc[j][r] = fmaf(w[j], x, acc[j][r]);
               }
            }
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1)
#pragma unroll
               for (int j = 0; j < 4; ++j)
#pragma unroll
                  for (int r = 0; r < RB; ++r)
                     acc[j][r] += __shfl_xor(acc[j][r], off, 64);
            // every lane now holds the 4 x RB sums: lane j finishes output n0 + j
            const int n = n0 + lane;
            if (lane < 4 && n < N) {
#pragma unroll
               for (int r = 0; r < RB; ++r) {
                  if (r < rows) {
                     const float s = lane == 0 ? acc[0][r] : lane == 1 ? acc[1][r] : lane == 2 ? acc[2][r] : acc[3][r];
                     const float v = f32_epilogue(L.ep, s, m0 + r, n);
                     out[r * width + n] = v;
                     L.Y[(long long)(m0 + r) * L.ldy + n] = v;
                  }
               }
            }
         }
      } else {
         for (int n = t; n < N; n += CHAIN_THREADS) {
            float acc[RB];
#pragma unroll
            for (int r = 0; r < RB; ++r)
               acc[r] = 0.0f;
#pragma unroll 8
            for (int k = 0; k < K; ++k) {
               const float w = B[(long long)k * L.ldb + n];
#pragma unroll
               for (int r = 0; r < RB; ++r)
                  acc[r] = fmaf(w, in[r * width + k], acc[r]);
            }
#pragma unroll
            for (int r = 0; r < RB; ++r) {
               if (r < rows) {
                  const float v = f32_epilogue(L.ep, acc[r], m0 + r, n);
                  out[r * width + n] = v;
                  L.Y[(long long)(m0 + r) * L.ldy + n] = v;
               }
            }
         }
      }
      __syncthreads();
      float *tmp = in;
      in = out;
      out = tmp;
   }
}

} // namespace sofie_hip

using namespace sofie_hip;

extern "C" {

int sofie_hip_gemm_f32(sofie_hip_ctx *ctx, const sofie_gemm_f32_desc *d)
{
   SOFIE_HIP_REQUIRE(ctx && d, "sofie_hip_gemm_f32: NULL argument");
   SOFIE_HIP_REQUIRE(d->M >= 0 && d->N >= 0 && d->K >= 0, "sofie_hip_gemm_f32: negative dimension");
   SOFIE_HIP_REQUIRE(d->batch >= 1, "sofie_hip_gemm_f32: batch must be >= 1");
   SOFIE_HIP_REQUIRE(d->bias_mode >= SOFIE_BIAS_NONE && d->bias_mode <= SOFIE_BIAS_FULL, "sofie_hip_gemm_f32: unknown bias mode %d", d->bias_mode);
   F32Epilogue ep;
   int bad = 0;
   SOFIE_HIP_REQUIRE(make_post_chain(ep.chain, d->act, d->act_alpha, d->post, bad),
                     "sofie_hip_gemm_f32: unknown activation or post operator %d (or more than %d post operators)", bad, SOFIE_MAX_POST_OPS);
   if (d->M == 0 || d->N == 0)
      return SOFIE_HIP_OK;
   SOFIE_HIP_REQUIRE(d->Y != nullptr, "sofie_hip_gemm_f32: Y is NULL");
   SOFIE_HIP_REQUIRE(d->K == 0 || (d->A && d->B), "sofie_hip_gemm_f32: A or B is NULL");
   SOFIE_HIP_REQUIRE(d->bias_mode == SOFIE_BIAS_NONE || d->C != nullptr, "sofie_hip_gemm_f32: bias mode set but C is NULL");
   const int M = d->M, N = d->N, K = d->K;
   const long long lda = d->lda ? d->lda : (d->transA ? M : K);
   const long long ldb = d->ldb ? d->ldb : (d->transB ? K : N);
   const long long ldy = d->ldy ? d->ldy : N;
   SOFIE_HIP_REQUIRE(lda >= (d->transA ? M : K) && ldb >= (d->transB ? K : N) && ldy >= N,
                     "sofie_hip_gemm_f32: leading dimension too small");
   GemmOperandA la{d->A, d->transA ? 1 : lda, d->transA ? lda : 1};
   GemmOperandB lb{d->B, d->transB ? 1 : ldb, d->transB ? ldb : 1};
   ep.alpha = d->alpha;
   ep.beta = d->beta;
   ep.C = d->bias_mode == SOFIE_BIAS_NONE ? nullptr : d->C;
   ep.bias_mode = d->bias_mode;
   ep.ldc = N;
   ep.R = d->residual;
   ep.ldr = ldy;
   const unsigned gy = (M + F32_BM - 1) / F32_BM, gx = (N + F32_BN - 1) / F32_BN;
   SOFIE_HIP_REQUIRE(gx <= 65535 && d->batch <= 65535, "sofie_hip_gemm_f32: N or batch too large for one launch");
   // few 64x64 tiles: one-wave workgroups with 8x8 tiles reach every CU (SOFIE_HIP_F32_SKINNY=0/1 overrides)
   const bool skinny = ctx->opt.f32_skinny >= 0 ? ctx->opt.f32_skinny != 0 : ((long long)gy * gx * d->batch < 192);
   if (skinny && K > 0 && (N + SK_T - 1) / SK_T <= 65535) {
      auto aligned16 = [](const void *p) { return ((uintptr_t)p & 15) == 0; };
      const bool va = !d->transA && K % 4 == 0 && lda % 4 == 0 && aligned16(d->A) && d->strideA % 4 == 0;
      const bool vb = d->transB && K % 4 == 0 && ldb % 4 == 0 && aligned16(d->B) && d->strideB % 4 == 0;
      const dim3 grid((M + SK_T - 1) / SK_T, (N + SK_T - 1) / SK_T, (unsigned)d->batch);
#define SOFIE_SKINNY(VA, VB)                                                                                              \
   hipLaunchKernelGGL((gemm_f32_skinny_kernel<VA, VB>), grid, dim3(64), 0, ctx->stream, la, lb, M, N, K, d->Y, ldy, ep,   \
                      (long long)d->strideA, (long long)d->strideB, (long long)d->strideC, (long long)d->strideY)
      if (va && vb)
         SOFIE_SKINNY(true, true);
      else if (va)
         SOFIE_SKINNY(true, false);
      else if (vb)
         SOFIE_SKINNY(false, true);
      else
         SOFIE_SKINNY(false, false);
#undef SOFIE_SKINNY
      return launch_status("gemm_f32_skinny_kernel");
   }
   hipLaunchKernelGGL(gemm_f32_kernel, dim3(gy, gx, (unsigned)d->batch), dim3(256), 0, ctx->stream, la, lb, M, N, K, d->Y, ldy, ep,
                      (long long)d->strideA, (long long)d->strideB, (long long)d->strideC, (long long)d->strideY);
   return launch_status("gemm_f32_kernel");
}

int sofie_hip_gemm_chain_f32(sofie_hip_ctx *ctx, const sofie_gemm_f32_desc *layers, int32_t count)
{
   SOFIE_HIP_REQUIRE(ctx && layers, "sofie_hip_gemm_chain_f32: NULL argument");
   SOFIE_HIP_REQUIRE(count >= 1 && count <= SOFIE_MAX_GEMM_CHAIN, "sofie_hip_gemm_chain_f32: %d layers (1..%d allowed)", count, SOFIE_MAX_GEMM_CHAIN);
   for (int l = 1; l < count; ++l)
      SOFIE_HIP_REQUIRE(layers[l].A == layers[l - 1].Y && layers[l].A != nullptr, "sofie_hip_gemm_chain_f32: layer %d does not read the output of layer %d", l, l - 1);
   // One launch when the batch is small enough that launches, not arithmetic, set the time, and the rows fit in LDS.
   const int M = layers[0].M;
   bool fused = count >= 2 && M >= 1 && (ctx->opt.f32_chain >= 0 ? ctx->opt.f32_chain != 0 : M <= 256);
   int width = layers[0].K;
   ChainArgs a;
   a.count = count;
   a.M = M;
   a.A = layers[0].A;
   a.lda = layers[0].lda ? layers[0].lda : layers[0].K;
   for (int l = 0; l < count && fused; ++l) {
      const sofie_gemm_f32_desc &d = layers[l];
      const long long ldb = d.ldb ? d.ldb : (d.transB ? d.K : d.N), ldy = d.ldy ? d.ldy : d.N;
      fused = d.M == M && d.N >= 1 && d.K >= 1 && !d.transA && d.batch == 1 && d.A && d.B && d.Y && ldb >= (d.transB ? d.K : d.N) && ldy >= d.N &&
              d.bias_mode >= SOFIE_BIAS_NONE && d.bias_mode <= SOFIE_BIAS_FULL && (d.bias_mode == SOFIE_BIAS_NONE || d.C != nullptr) &&
              (l == 0 ? a.lda >= d.K : (d.K == layers[l - 1].N && (d.lda ? d.lda : d.K) == (layers[l - 1].ldy ? layers[l - 1].ldy : layers[l - 1].N)));
      if (!fused)
         break;
      ChainLayerArgs &L = a.layer[l];
      L.B = d.B;
      L.ldb = ldb;
      L.transB = d.transB ? 1 : 0;
      L.N = d.N;
      L.K = d.K;
      L.Y = d.Y;
      L.ldy = ldy;
      int bad = 0;
      fused = make_post_chain(L.ep.chain, d.act, d.act_alpha, d.post, bad);
      L.ep.alpha = d.alpha;
      L.ep.beta = d.beta;
      L.ep.C = d.bias_mode == SOFIE_BIAS_NONE ? nullptr : d.C;
      L.ep.bias_mode = d.bias_mode;
      L.ep.ldc = d.N;
      L.ep.R = d.residual;
      L.ep.ldr = ldy;
      width = d.N > width ? d.N : width;
   }
   // In one launch a workgroup takes ITS rows through every layer, independently of the other workgroups.  Two tensors of the
   // chain may therefore share memory only row for row (same address, same pitch, same width: the ping-pong of equal layers,
   // where a row is rewritten by the workgroup that owns it); any other overlap of what a layer writes with what a layer
   // reads or writes would let one workgroup's rows land on another's.  Callers that planned the layers' tensors by
   // per-layer lifetimes get the layer-by-layer form then.
   if (fused) {
      struct Range {
         const char *lo, *hi;
         long long pitch, width;
      };
      auto range = [](const void *p, long long bytes, long long pitch, long long w) {
         return Range{(const char *)p, (const char *)p + (bytes > 0 ? bytes : 0), pitch, w};
      };
      auto overlap = [](const Range &x, const Range &y) { return x.lo < y.hi && y.lo < x.hi; };
      auto same_rows = [](const Range &x, const Range &y) { return x.lo == y.lo && x.pitch == y.pitch && x.width == y.width; };
      Range reads[2 * SOFIE_MAX_GEMM_CHAIN], writes[SOFIE_MAX_GEMM_CHAIN];
      int nr = 0;
      const Range input = range(layers[0].A, ((long long)(M - 1) * a.lda + layers[0].K) * 4, a.lda, layers[0].K);
      for (int l = 0; l < count; ++l) {
         const sofie_gemm_f32_desc &d = layers[l];
         const long long ldy = d.ldy ? d.ldy : d.N, ybytes = ((long long)(M - 1) * ldy + d.N) * 4;
         writes[l] = range(d.Y, ybytes, ldy, d.N);
         if (d.bias_mode != SOFIE_BIAS_NONE)
            reads[nr++] = range(d.C, 4LL * (d.bias_mode == SOFIE_BIAS_ROW ? d.N : d.bias_mode == SOFIE_BIAS_COL ? M : d.bias_mode == SOFIE_BIAS_FULL ? (long long)M * d.N : 1), 0, 0);
         if (d.residual)
            reads[nr++] = range(d.residual, ybytes, 0, 0);
      }
      for (int l = 0; l < count && fused; ++l) {
         if (overlap(writes[l], input) && !same_rows(writes[l], input))
            fused = false;
         for (int m = 0; m < l && fused; ++m)
            if (overlap(writes[l], writes[m]) && !same_rows(writes[l], writes[m]))
               fused = false;
         for (int r = 0; r < nr && fused; ++r)
            if (overlap(writes[l], reads[r]))
               fused = false;
      }
   }
   const int RB = M <= 64 ? 1 : M <= 128 ? 2 : 4;
   width = (width + 3) / 4 * 4;
   if (fused && (long long)RB * width <= 8192) {
      const size_t lds = (size_t)2 * RB * width * sizeof(float);
      const dim3 grid((unsigned)((M + RB - 1) / RB));
      if (RB == 1)
         hipLaunchKernelGGL(gemm_chain_f32_kernel<1>, grid, dim3(CHAIN_THREADS), lds, ctx->stream, a, width);
      else if (RB == 2)
         hipLaunchKernelGGL(gemm_chain_f32_kernel<2>, grid, dim3(CHAIN_THREADS), lds, ctx->stream, a, width);
      else
         hipLaunchKernelGGL(gemm_chain_f32_kernel<4>, grid, dim3(CHAIN_THREADS), lds, ctx->stream, a, width);
      return launch_status("gemm_chain_f32_kernel");
   }
   // anything else (and every malformed descriptor, which the single product reports): one launch per layer
   for (int l = 0; l < count; ++l)
      if (int st = sofie_hip_gemm_f32(ctx, &layers[l]))
         return st;
   return SOFIE_HIP_OK;
}

int sofie_hip_conv_f32(sofie_hip_ctx *ctx, const sofie_conv_desc *d, const float *X, const float *W, const float *bias,
                       int32_t act, float act_alpha, float *Y, const sofie_post_ops *post, const float *residual)
{
   SOFIE_HIP_REQUIRE(ctx && d, "sofie_hip_conv_f32: NULL argument");
   SOFIE_HIP_REQUIRE(d->N >= 0 && d->C > 0 && d->H > 0 && d->W > 0 && d->Cout > 0 && d->kh > 0 && d->kw > 0,
                     "sofie_hip_conv_f32: bad shape");
   SOFIE_HIP_REQUIRE(d->group > 0 && d->C % d->group == 0 && d->Cout % d->group == 0,
                     "sofie_hip_conv_f32: group %d does not divide the channels", d->group);
   SOFIE_HIP_REQUIRE(d->stride_h > 0 && d->stride_w > 0 && d->dil_h > 0 && d->dil_w > 0, "sofie_hip_conv_f32: bad stride or dilation");
   SOFIE_HIP_REQUIRE(d->pad_h0 >= 0 && d->pad_w0 >= 0 && d->pad_h1 >= 0 && d->pad_w1 >= 0, "sofie_hip_conv_f32: negative padding");
   const int eff_kh = d->dil_h * (d->kh - 1) + 1, eff_kw = d->dil_w * (d->kw - 1) + 1;
   SOFIE_HIP_REQUIRE(d->H + d->pad_h0 + d->pad_h1 >= eff_kh && d->W + d->pad_w0 + d->pad_w1 >= eff_kw,
                     "sofie_hip_conv_f32: kernel larger than the padded image");
   const int OH = (d->H + d->pad_h0 + d->pad_h1 - eff_kh) / d->stride_h + 1;
   const int OW = (d->W + d->pad_w0 + d->pad_w1 - eff_kw) / d->stride_w + 1;
   SOFIE_HIP_REQUIRE(OH == d->OH && OW == d->OW, "sofie_hip_conv_f32: output shape %dx%d does not match the descriptor's %dx%d", OH, OW,
                     d->OH, d->OW);
   PostChain chain;
   int bad = 0;
   SOFIE_HIP_REQUIRE(make_post_chain(chain, act, act_alpha, post, bad),
                     "sofie_hip_conv_f32: unknown activation or post operator %d (or more than %d post operators)", bad, SOFIE_MAX_POST_OPS);
   if (d->N == 0)
      return SOFIE_HIP_OK;
   SOFIE_HIP_REQUIRE(X && W && Y, "sofie_hip_conv_f32: NULL pointer");
   const long long M = (long long)d->N * OH * OW;
   SOFIE_HIP_REQUIRE(M < (1LL << 31), "sofie_hip_conv_f32: too many output pixels");
   const int Cg = d->C / d->group, Cout_g = d->Cout / d->group, Kg = Cg * d->kh * d->kw;
   ConvOperandA la{X, d->C, d->H, d->W, d->kh, d->kw, OH, OW, d->pad_h0, d->pad_w0, d->stride_h, d->stride_w, d->dil_h, d->dil_w, 0};
   const unsigned gy = (unsigned)((M + F32_BM - 1) / F32_BM), gx = (Cout_g + F32_BN - 1) / F32_BN;
   SOFIE_HIP_REQUIRE(gx <= 65535 && d->group <= 65535, "sofie_hip_conv_f32: too many channels or groups for one launch");
   hipLaunchKernelGGL(conv_f32_kernel<ConvOperandA>, dim3(gy, gx, (unsigned)d->group), dim3(256), 0, ctx->stream, la, W, bias, Y, (int)M, Cout_g, Kg,
                      Cg, d->Cout, OH * OW, chain, residual);
   return launch_status("conv_f32_kernel");
}

int sofie_hip_conv3d_f32(sofie_hip_ctx *ctx, const sofie_conv3d_desc *d, const float *X, const float *W, const float *bias,
                         int32_t act, float act_alpha, float *Y, const sofie_post_ops *post, const float *residual)
{
   SOFIE_HIP_REQUIRE(ctx && d, "sofie_hip_conv3d_f32: NULL argument");
   SOFIE_HIP_REQUIRE(d->N >= 0 && d->C > 0 && d->D > 0 && d->H > 0 && d->W > 0 && d->Cout > 0 && d->kd > 0 && d->kh > 0 && d->kw > 0,
                     "sofie_hip_conv3d_f32: bad shape");
   SOFIE_HIP_REQUIRE(d->group > 0 && d->C % d->group == 0 && d->Cout % d->group == 0,
                     "sofie_hip_conv3d_f32: group %d does not divide the channels", d->group);
   const int in[3] = {d->D, d->H, d->W}, kern[3] = {d->kd, d->kh, d->kw}, want[3] = {d->OD, d->OH, d->OW};
   int outd[3];
   for (int a = 0; a < 3; ++a) {
      SOFIE_HIP_REQUIRE(d->stride[a] > 0 && d->dil[a] > 0, "sofie_hip_conv3d_f32: bad stride or dilation");
      SOFIE_HIP_REQUIRE(d->pad[a] >= 0 && d->pad[a + 3] >= 0, "sofie_hip_conv3d_f32: negative padding");
      const int eff = d->dil[a] * (kern[a] - 1) + 1;
      SOFIE_HIP_REQUIRE(in[a] + d->pad[a] + d->pad[a + 3] >= eff, "sofie_hip_conv3d_f32: kernel larger than the padded volume");
      outd[a] = (in[a] + d->pad[a] + d->pad[a + 3] - eff) / d->stride[a] + 1;
      SOFIE_HIP_REQUIRE(outd[a] == want[a], "sofie_hip_conv3d_f32: output extent %d of axis %d does not match the descriptor's %d", outd[a], a, want[a]);
   }
   PostChain chain;
   int bad = 0;
   SOFIE_HIP_REQUIRE(make_post_chain(chain, act, act_alpha, post, bad),
                     "sofie_hip_conv3d_f32: unknown activation or post operator %d (or more than %d post operators)", bad, SOFIE_MAX_POST_OPS);
   if (d->N == 0)
      return SOFIE_HIP_OK;
   SOFIE_HIP_REQUIRE(X && W && Y, "sofie_hip_conv3d_f32: NULL pointer");
   const long long plane = (long long)outd[0] * outd[1] * outd[2], M = (long long)d->N * plane;
   SOFIE_HIP_REQUIRE(M < (1LL << 31) && (long long)d->C * d->D * d->H * d->W < (1LL << 31), "sofie_hip_conv3d_f32: too many output or input elements");
   const long long Kg64 = (long long)(d->C / d->group) * d->kd * d->kh * d->kw;
   SOFIE_HIP_REQUIRE(Kg64 < (1LL << 31), "sofie_hip_conv3d_f32: reduction too long");
   const int Cg = d->C / d->group, Cout_g = d->Cout / d->group, Kg = (int)Kg64;
   Conv3dOperandA la{X, d->C, d->D, d->H, d->W, d->kd, d->kh, d->kw, outd[0], outd[1], outd[2], d->pad[0], d->pad[1], d->pad[2],
                     d->stride[0], d->stride[1], d->stride[2], d->dil[0], d->dil[1], d->dil[2], 0};
   const unsigned gy = (unsigned)((M + F32_BM - 1) / F32_BM), gx = (Cout_g + F32_BN - 1) / F32_BN;
   SOFIE_HIP_REQUIRE(gx <= 65535 && d->group <= 65535, "sofie_hip_conv3d_f32: too many channels or groups for one launch");
   hipLaunchKernelGGL(conv_f32_kernel<Conv3dOperandA>, dim3(gy, gx, (unsigned)d->group), dim3(256), 0, ctx->stream, la, W, bias, Y, (int)M,
                      Cout_g, Kg, Cg, d->Cout, (int)plane, chain, residual);
   return launch_status("conv_f32_kernel (3-D)");
}

} // extern "C"
