// int8 x int8 -> int32 GEMM on the gfx950 matrix cores (v_mfma_i32_32x32x32_i8) with the
// requantisation / dequantisation epilogue fused into the store, and the int8 re-layout kernel.
#include "i8_epilogue.hpp"
#include "conv_i8_few_channels.hpp"
#include <cmath>
#include <mutex>

namespace sofie_hip {

// dst[c][r] = src[r][c] for an int8 matrix, through a 64x64 LDS tile.
__global__ __launch_bounds__(256) void transpose_i8_kernel(int8_t *__restrict__ dst, const int8_t *__restrict__ src,
                                                            int rows, int cols, int ld_src, int ld_dst)
{
   __shared__ int8_t tile[64][64 + 4];
   const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
   const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
   for (int i = ty; i < 64; i += 4) {
      int r = r0 + i, c = c0 + tx;
      tile[i][tx] = (r < rows && c < cols) ? src[(size_t)r * ld_src + c] : (int8_t)0;
   }
   __syncthreads();
   for (int i = ty; i < 64; i += 4) {
      int c = c0 + i, r = r0 + tx;
      if (c < cols && r < rows)
         dst[(size_t)c * ld_dst + r] = tile[tx][i];
   }
}


// The fields of the epilogue that follow from the others: what the stores may assume about alignment, and whether the
// quotient of SOFIE_I8OUT_I8_DQQ may be formed from the reciprocal (a per-tensor scale known here, in a safe range).
static void derive_epilogue_fields(I8Epilogue &ep, int N)
{
   const size_t esz = ep.out == SOFIE_I8OUT_I32 || ep.out == SOFIE_I8OUT_F32 ? 4 : 1;
   ep.N = N;
   ep.stage_ok = (ep.nchw_ohw == 0) && (((size_t)ep.ldy * esz) % 16 == 0) && (((size_t)ep.n_offset * esz) % 16 == 0) &&
                 (((uintptr_t)ep.Y & 15) == 0);
   ep.vec_param = (ep.n_offset % 4 == 0) && (!ep.bias || ((uintptr_t)ep.bias & 15) == 0) &&
                  (!ep.scale || ((uintptr_t)ep.scale & 15) == 0);
   ep.q_rcp = 0.0f;
   ep.q_by_rcp = ep.out == SOFIE_I8OUT_I8_DQQ && !ep.scale && quotient_plan(ep.scale_scalar, ep.q_scale, ep.q_rcp);
}

int gemm_i8_nt(const LaunchCfg &lc, const int8_t *A, const int8_t *Bt, int M, int N, int K, int lda, int ldb, I8Epilogue ep)
{
   derive_epilogue_fields(ep, N);
   return launch_mfma8_best<MfmaI8, I8Epilogue>(lc, A, Bt, M, N, K, lda, ldb, ep);
}

int conv_i8_implicit(const LaunchCfg &lc, const ConvRows &src, int Cg, const int8_t *Wp, int M, int N, int K, I8Epilogue ep)
{
   derive_epilogue_fields(ep, N);
   return launch_mfma8_conv<I8Epilogue>(lc, src, Cg, Wp, M, N, K, ep);
}

int conv_i8_gather(const LaunchCfg &lc, const GatherConvRows &src, const int8_t *Wp, int M, int N, int Kp, I8Epilogue ep)
{
   derive_epilogue_fields(ep, N);
   return launch_mfma8_gather<I8Epilogue>(lc, src, Wp, M, N, Kp, ep);
}

int conv_i8_few_channels(const LaunchCfg &lc, const FewChannelConv &src, const int8_t *Wp, int M, int N, int Kp, I8Epilogue ep, bool *taken)
{
   derive_epilogue_fields(ep, N);
   *taken = false;
   // 27 asks for it by force; any other forced tile or variant keeps it away
   if (!((lc.tile == 0 && lc.variant == 0) || lc.tile == 27))
      return SOFIE_HIP_OK;
   if (N != 64 || M % 64 != 0 || !ep.stores_plain_rows() || !conv_i8_few_channels_applies(src, Wp))
      return SOFIE_HIP_OK;
   *taken = true;
   return launch_conv_i8_few_channels<I8Epilogue>(lc, src, Wp, M, Kp, ep);
}

int transpose_i8(hipStream_t stream, int8_t *dst, const int8_t *src, int rows, int cols, int ld_src, int ld_dst)
{
   dim3 grid((cols + 63) / 64, (rows + 63) / 64);
   hipLaunchKernelGGL(transpose_i8_kernel, grid, dim3(256), 0, stream, dst, src, rows, cols, ld_src, ld_dst);
   return launch_status("transpose_i8_kernel");
}

} // namespace sofie_hip

using namespace sofie_hip;


extern "C" {

size_t sofie_hip_gemm_i8_workspace(const sofie_gemm_i8_desc *d)
{
   if (!d)
      return 0;
   size_t need = 0;
   if (!d->transB)
      need += (((size_t)d->K * (size_t)d->N) + 255) & ~(size_t)255;
   if (d->transA)
      need += (((size_t)d->K * (size_t)d->M) + 255) & ~(size_t)255;
   return need;
}

int sofie_hip_transpose_i8(sofie_hip_ctx *ctx, int8_t *dst, const int8_t *src, int32_t rows, int32_t cols, int32_t ld_src,
                           int32_t ld_dst)
{
   SOFIE_HIP_REQUIRE(ctx && dst && src, "sofie_hip_transpose_i8: NULL argument");
   SOFIE_HIP_REQUIRE(rows >= 0 && cols >= 0, "sofie_hip_transpose_i8: negative shape");
   if (rows == 0 || cols == 0)
      return SOFIE_HIP_OK;
   if (ld_src == 0)
      ld_src = cols;
   if (ld_dst == 0)
      ld_dst = rows;
   SOFIE_HIP_REQUIRE(ld_src >= cols && ld_dst >= rows, "sofie_hip_transpose_i8: leading dimension too small");
   SOFIE_HIP_REQUIRE((rows + 63) / 64 <= 65535, "sofie_hip_transpose_i8: too many rows");
   return transpose_i8(ctx->stream, dst, src, rows, cols, ld_src, ld_dst);
}

// The body of sofie_hip_gemm_i8 with the re-layout scratch given separately from the descriptor.
static int gemm_i8_with_workspace(sofie_hip_ctx *ctx, const sofie_gemm_i8_desc *d, void *workspace, size_t workspace_bytes)
{
   SOFIE_HIP_REQUIRE(ctx && d, "sofie_hip_gemm_i8: NULL argument");
   SOFIE_HIP_REQUIRE(d->M >= 0 && d->N >= 0 && d->K >= 0, "sofie_hip_gemm_i8: negative dimension");
   SOFIE_HIP_REQUIRE(d->out >= SOFIE_I8OUT_I32 && d->out <= SOFIE_I8OUT_I8_DQQ, "sofie_hip_gemm_i8: unknown output kind %d", d->out);
   if (d->M == 0 || d->N == 0)
      return SOFIE_HIP_OK;
   SOFIE_HIP_REQUIRE(d->Y != nullptr, "sofie_hip_gemm_i8: Y is NULL");
   SOFIE_HIP_REQUIRE(d->K == 0 || (d->A && d->B), "sofie_hip_gemm_i8: A or B is NULL");
   SOFIE_HIP_REQUIRE(d->out != SOFIE_I8OUT_I8_DQQ || (d->q_scale != 0.0f && std::isfinite(d->q_scale)),
                     "sofie_hip_gemm_i8: q_scale is 0 or not finite");
   const int M = d->M, N = d->N, K = d->K;
   int lda = d->lda ? d->lda : (d->transA ? M : K);
   int ldb = d->ldb ? d->ldb : (d->transB ? K : N);
   int ldy = d->ldy ? d->ldy : N;
   SOFIE_HIP_REQUIRE(lda >= (d->transA ? M : K) && ldb >= (d->transB ? K : N) && ldy >= N,
                     "sofie_hip_gemm_i8: leading dimension too small");

   const int8_t *A = d->A, *Bt = d->B;
   char *ws = (char *)workspace;
   size_t ws_left = workspace_bytes;
   if (K > 0 && !d->transB) {
      // B is [K,N]: the kernel wants [N,K]
      size_t need = (((size_t)K * (size_t)N) + 255) & ~(size_t)255;
      SOFIE_HIP_REQUIRE(ws != nullptr && ws_left >= need,
                        "sofie_hip_gemm_i8: B is [K,N]; a workspace of %zu bytes is needed to re-lay it out", need);
      SOFIE_HIP_REQUIRE(((uintptr_t)ws & 255) == 0, "sofie_hip_gemm_i8: workspace must be 256-byte aligned");
      int st = transpose_i8(ctx->stream, (int8_t *)ws, d->B, K, N, ldb, K);
      if (st)
         return st;
      Bt = (const int8_t *)ws;
      ldb = K;
      ws += need;
      ws_left -= need;
   }
   if (K > 0 && d->transA) {
      size_t need = (((size_t)K * (size_t)M) + 255) & ~(size_t)255;
      SOFIE_HIP_REQUIRE(ws != nullptr && ws_left >= need,
                        "sofie_hip_gemm_i8: A is stored [K,M]; a workspace of %zu more bytes is needed", need);
      int st = transpose_i8(ctx->stream, (int8_t *)ws, d->A, K, M, lda, K);
      if (st)
         return st;
      A = (const int8_t *)ws;
      lda = K;
   }

   I8Epilogue ep;
   ep.bias = d->bias;
   ep.scale = d->scale;
   ep.scale_scalar = d->scale_scalar;
   ep.q_scale = d->q_scale;
   ep.relu_acc = d->relu_acc;
   ep.relu_out = d->relu_out;
   ep.out = d->out;
   ep.Y = d->Y;
   ep.ldy = ldy;
   ep.stage_ok = 0;
   ep.vec_param = 0;
   ep.N = N;
   ep.nchw_ohw = 0;
   ep.n_offset = 0;
   if (K == 0) {
      // empty reduction: acc = 0 everywhere; run the kernel with K = 0 using any valid pointer
      A = (const int8_t *)d->Y;
      Bt = (const int8_t *)d->Y;
      lda = ldb = 16;
   }
   return gemm_i8_nt(launch_cfg_i8(ctx), A, Bt, M, N, K, lda, ldb, ep);
}

int sofie_hip_gemm_i8(sofie_hip_ctx *ctx, const sofie_gemm_i8_desc *d)
{
   SOFIE_HIP_REQUIRE(ctx && d, "sofie_hip_gemm_i8: NULL argument");
   return gemm_i8_with_workspace(ctx, d, d->workspace, d->workspace_bytes);
}

// ---- the entry point that allocates nothing -------------------------------------------------------------------------------
// The operand re-layout of sofie_hip_gemm_i8 (B given as [K,N], A given as [K,M]) needs scratch memory.  Here it lives in a
// static device array instead of a workspace of the caller: every GPU the library runs on holds its own copy of the array
// until the process ends.  In host code the array's name is only a stand-in; the device address comes from
// hipGetSymbolAddress, once per device, and that pointer is what the kernels are given.
static __device__ __align__(256) unsigned char scratch[SOFIE_HIP_GEMM_I8_NOALLOC_SCRATCH_BYTES];

namespace {
std::mutex g_scratch_mutex;
void *g_scratch_ptr[64] = {}; // per device: the address of `scratch` there
} // namespace

int sofie_hip_gemm_i8_noalloc(sofie_hip_ctx *ctx, const sofie_gemm_i8_desc *d)
{
   SOFIE_HIP_REQUIRE(ctx && d, "sofie_hip_gemm_i8_noalloc: NULL argument");
   SOFIE_HIP_REQUIRE(ctx->device >= 0 && ctx->device < 64, "sofie_hip_gemm_i8_noalloc: device %d out of range", ctx->device);
   const size_t need = sofie_hip_gemm_i8_workspace(d);
   SOFIE_HIP_REQUIRE(need <= (size_t)SOFIE_HIP_GEMM_I8_NOALLOC_SCRATCH_BYTES,
                     "sofie_hip_gemm_i8_noalloc: the operand re-layout needs %zu bytes of scratch, the static buffer holds %zu "
                     "(use sofie_hip_gemm_i8 with a workspace, or operands already laid out [M,K] and [N,K])",
                     need, (size_t)SOFIE_HIP_GEMM_I8_NOALLOC_SCRATCH_BYTES);
   void *ptr = nullptr;
   {
      std::lock_guard<std::mutex> lock(g_scratch_mutex);
      if (!g_scratch_ptr[ctx->device]) {
         // first call on this device: look the array's address up with that device current
         int current = -1;
         SOFIE_HIP_CHECK(hipGetDevice(&current));
         if (current != ctx->device)
            SOFIE_HIP_CHECK(hipSetDevice(ctx->device));
         void *p = nullptr;
         const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
         if (current != ctx->device)
            (void)hipSetDevice(current);
         if (e != hipSuccess || !p)
            return fail(SOFIE_HIP_ERR_RUNTIME, "sofie_hip_gemm_i8_noalloc: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
         g_scratch_ptr[ctx->device] = p;
      }
      ptr = g_scratch_ptr[ctx->device];
   }
   // the re-layout kernels overwrite every byte they later read: nothing has to start at zero
   return gemm_i8_with_workspace(ctx, d, ptr, (size_t)SOFIE_HIP_GEMM_I8_NOALLOC_SCRATCH_BYTES);
}

} // extern "C"
