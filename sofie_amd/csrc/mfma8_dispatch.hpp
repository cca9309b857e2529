// Kernel choice for the int8 / FP8 GEMM and the int8 convolution: which tile, which pipelined kernel, or the general one.
#pragma once
#include "mfma8_gemm_persist.hpp"

namespace sofie_hip {

// Chooses between the pipelined kernels (aligned operands, K a multiple of 64) and the general one.
// `variant` selects a tuning alternative of the pipelined kernel (0 = default); -1 forces the general kernel.
template <class MMA, class EPI>
static int launch_mfma8_best(hipStream_t stream, const int8_t *A, const int8_t *Bt, int M, int N, int K, int lda, int ldb,
                             const EPI &ep, int force_tile, int variant)
{
   const bool aligned = (lda % 16 == 0) && (ldb % 16 == 0) && (((uintptr_t)A & 15) == 0) && (((uintptr_t)Bt & 15) == 0);
   if (variant < 0 || !aligned || K < 64 || K % 64 != 0)
      return launch_mfma8_auto<MMA, EPI>(stream, A, Bt, M, N, K, lda, ldb, ep, force_tile);
   const int tile = pick_tile(M, N, force_tile);
   const bool k128 = (K % 128 == 0);
   if constexpr (MMA::KSTEP * 2 <= 64) {
      // Large products that divide into whole 256 x 256 tiles: the persistent kernel (512 asks for it by force)
      if ((force_tile == 512 || (!force_tile && variant == 0 && tile == 256)) && mfma8_persist_applies(A, Bt, M, N, K, lda, ldb) &&
          ep.stores_plain_rows())
         return launch_mfma8_persist<MfmaI8x16, EPI>(stream, A, Bt, M, N, K, lda, ldb, ep);
      // Short reductions over many tiles: the 256 x 128 tile with a ring of three slabs fits twice on a CU, and one
      // workgroup's prologue and store overlap the other's K loop (8192 x 4096 x 512: 829 -> 1019 TOP/s, 8192 x 1024 x 1024:
      // 1003 -> 1091; no gain from K = 2048 on).  258 asks for it by force.
      const long long tiles_256x128 = (long long)((M + 255) / 256) * ((N + 127) / 128);
      if (force_tile == 258 || (!force_tile && variant == 0 && K <= 1024 && N >= 128 && tiles_256x128 >= 512))
         return launch_mfma8_dma_src<MMA, 256, 128, 64, 2, 2, 3, EPI, 0, RowMajorRows, 2>(stream, RowMajorRows{A, lda}, Bt, M, N, K, ldb, ep);
   }
   if constexpr (MMA::KSTEP * 2 > 64) {
      // two K-steps per slab are the minimum: a 64-byte K-step needs 128-byte slabs
      if (!k128)
         return launch_mfma8_auto<MMA, EPI>(stream, A, Bt, M, N, K, lda, ldb, ep, force_tile);
      if ((force_tile == 512 || (!force_tile && variant == 0 && tile == 256)) && mfma8_persist_applies(A, Bt, M, N, K, lda, ldb) &&
          ep.stores_plain_rows())
         return launch_mfma8_persist<MMA, EPI>(stream, A, Bt, M, N, K, lda, ldb, ep);
      switch (tile) {
      case 256:
         if (variant == 1)
            return launch_mfma8_dma<MMA, 256, 128, 128, 2, 2, 3, EPI>(stream, A, Bt, M, N, K, lda, ldb, ep);
         return launch_mfma8_pair<MMA, 256, 256, 64, 2, 2, 5, EPI>(stream, A, Bt, M, N, K, lda, ldb, ep);
      case 128: return launch_mfma8_dma<MMA, 128, 128, 128, 2, 2, 3, EPI>(stream, A, Bt, M, N, K, lda, ldb, ep);
      case 64: return launch_mfma8_dma<MMA, 64, 64, 128, 2, 2, 4, EPI>(stream, A, Bt, M, N, K, lda, ldb, ep);
      default: return fail(SOFIE_HIP_ERR_INVALID, "gemm: unknown tile %d", tile);
      }
   } else {
      switch (tile) {
      case 256:
#ifdef SOFIE_HIP_TUNING
         if (variant >= 10 && variant < 18) {
            switch (variant - 10) {
            case 1: return launch_mfma8_dma<MMA, 256, 256, 64, 2, 2, 4, EPI, 1>(stream, A, Bt, M, N, K, lda, ldb, ep);
            case 2: return launch_mfma8_dma<MMA, 256, 256, 64, 2, 2, 4, EPI, 2>(stream, A, Bt, M, N, K, lda, ldb, ep);
            case 3: return launch_mfma8_dma<MMA, 256, 256, 64, 2, 2, 4, EPI, 3>(stream, A, Bt, M, N, K, lda, ldb, ep);
            case 4: return launch_mfma8_dma<MMA, 256, 256, 64, 2, 2, 4, EPI, 4>(stream, A, Bt, M, N, K, lda, ldb, ep);
            case 6: return launch_mfma8_dma<MMA, 256, 256, 64, 2, 2, 4, EPI, 6>(stream, A, Bt, M, N, K, lda, ldb, ep);
            default: break;
            }
         }
         if (variant == 21)
            return launch_mfma8_dma<MMA, 256, 128, 128, 2, 2, 3, EPI, 6>(stream, A, Bt, M, N, K, lda, ldb, ep);
         if (variant == 22)
            return launch_mfma8_dma<MMA, 256, 128, 64, 2, 2, 4, EPI, 6>(stream, A, Bt, M, N, K, lda, ldb, ep);
         if (variant == 23)
            return launch_mfma8_dma<MMA, 256, 128, 128, 2, 2, 3, EPI, 0>(stream, A, Bt, M, N, K, lda, ldb, ep);
         if (variant == 24)
            return launch_mfma8_dma<MMA, 256, 128, 64, 2, 2, 4, EPI, 0>(stream, A, Bt, M, N, K, lda, ldb, ep);
         if (variant == 31)
            return launch_mfma8_pair<MMA, 256, 256, 64, 2, 2, 5, EPI, 6>(stream, A, Bt, M, N, K, lda, ldb, ep);
         if (variant == 32)
            return launch_mfma8_pair<MMA, 256, 256, 64, 2, 2, 5, EPI, 3>(stream, A, Bt, M, N, K, lda, ldb, ep);
         if (variant == 33)
            return launch_mfma8_pair<MMA, 256, 256, 64, 2, 2, 5, EPI, 10>(stream, A, Bt, M, N, K, lda, ldb, ep);
         if (variant == 34)
            return launch_mfma8_pair<MMA, 256, 256, 64, 2, 2, 5, EPI, 2>(stream, A, Bt, M, N, K, lda, ldb, ep);
         if (variant == 35)
            return launch_mfma8_pair<MMA, 256, 256, 64, 2, 2, 5, EPI, 1>(stream, A, Bt, M, N, K, lda, ldb, ep);
         if (variant == 36)
            return launch_mfma8_pair<MMA, 256, 256, 64, 2, 2, 5, EPI, 8>(stream, A, Bt, M, N, K, lda, ldb, ep);
         if (variant == 37)
            return launch_mfma8_pair<MMA, 256, 256, 64, 2, 2, 5, EPI, 24>(stream, A, Bt, M, N, K, lda, ldb, ep);
         if (variant == 41)
            return launch_mfma8_pair<MMA, 256, 256, 64, 2, 2, 5, EPI, 64>(stream, A, Bt, M, N, K, lda, ldb, ep);
         if (variant == 42)
            return launch_mfma8_pair<MMA, 256, 256, 64, 2, 2, 5, EPI, 128>(stream, A, Bt, M, N, K, lda, ldb, ep);
         if (variant == 38)
            return launch_mfma8_pair<MMA, 256, 256, 64, 2, 2, 5, EPI, 19>(stream, A, Bt, M, N, K, lda, ldb, ep);
         if (variant == 61)
            return launch_mfma8_pair<MMA, 256, 256, 64, 2, 4, 5, EPI, 0>(stream, A, Bt, M, N, K, lda, ldb, ep);
         if (variant == 62)
            return launch_mfma8_pair<MMA, 256, 256, 64, 4, 2, 5, EPI, 0>(stream, A, Bt, M, N, K, lda, ldb, ep);
         if (variant == 63)
            return launch_mfma8_pair<MMA, 256, 256, 64, 2, 4, 5, EPI, 16>(stream, A, Bt, M, N, K, lda, ldb, ep);
#endif
         if (variant == 1 || !k128)
            return launch_mfma8_dma<MMA, 256, 256, 64, 2, 2, 4, EPI>(stream, A, Bt, M, N, K, lda, ldb, ep);
         return launch_mfma8_pair<MMA, 256, 256, 64, 2, 2, 5, EPI>(stream, A, Bt, M, N, K, lda, ldb, ep);
      case 128:
#ifdef SOFIE_HIP_TUNING
         if (variant == 51)
            return launch_mfma8_dma<MMA, 128, 128, 128, 2, 2, 4, EPI>(stream, A, Bt, M, N, K, lda, ldb, ep);
         if (variant == 52)
            return launch_mfma8_dma<MMA, 128, 128, 64, 2, 2, 8, EPI>(stream, A, Bt, M, N, K, lda, ldb, ep);
         if (variant == 53)
            return launch_mfma8_dma<MMA, 128, 128, 64, 2, 2, 6, EPI>(stream, A, Bt, M, N, K, lda, ldb, ep);
         if (variant == 54)
            return launch_mfma8_dma<MMA, 128, 128, 128, 2, 2, 3, EPI, 4>(stream, A, Bt, M, N, K, lda, ldb, ep);
         if (variant == 55)
            return launch_mfma8_dma<MMA, 128, 128, 128, 2, 2, 3, EPI, 1>(stream, A, Bt, M, N, K, lda, ldb, ep);
         if (variant == 56)
            return launch_mfma8_dma<MMA, 128, 128, 128, 2, 2, 4, EPI, 4>(stream, A, Bt, M, N, K, lda, ldb, ep);
         if (variant == 57)
            return launch_mfma8_dma<MMA, 128, 128, 128, 2, 2, 3, EPI, 7>(stream, A, Bt, M, N, K, lda, ldb, ep);
#endif
         if (variant == 1 || !k128)
            return launch_mfma8_dma<MMA, 128, 128, 64, 2, 2, 4, EPI>(stream, A, Bt, M, N, K, lda, ldb, ep);
         return launch_mfma8_dma<MMA, 128, 128, 128, 2, 2, 3, EPI>(stream, A, Bt, M, N, K, lda, ldb, ep);
      case 64:
#ifdef SOFIE_HIP_TUNING
         if (variant == 54)
            return launch_mfma8_dma<MMA, 64, 64, 128, 2, 2, 4, EPI, 4>(stream, A, Bt, M, N, K, lda, ldb, ep);
         if (variant == 55)
            return launch_mfma8_dma<MMA, 64, 64, 128, 2, 2, 4, EPI, 1>(stream, A, Bt, M, N, K, lda, ldb, ep);
         if (variant == 57)
            return launch_mfma8_dma<MMA, 64, 64, 128, 2, 2, 4, EPI, 7>(stream, A, Bt, M, N, K, lda, ldb, ep);
#endif
         if (variant == 1 || !k128)
            return launch_mfma8_dma<MMA, 64, 64, 64, 2, 2, 4, EPI>(stream, A, Bt, M, N, K, lda, ldb, ep);
         return launch_mfma8_dma<MMA, 64, 64, 128, 2, 2, 4, EPI>(stream, A, Bt, M, N, K, lda, ldb, ep);
      default: return fail(SOFIE_HIP_ERR_INVALID, "gemm: unknown tile %d", tile);
      }
   }
}

} // namespace sofie_hip

namespace sofie_hip {

// Convolution as one implicit GEMM: A is read through ConvRows (BK = 64 must divide the channels per group),
// Wp is the packed weight [N][K] with K = taps * Cg.
template <class EPI>
static int launch_mfma8_conv(hipStream_t stream, const ConvRows &a, int Cg, const int8_t *Wp, int M, int N, int K, const EPI &ep,
                             int force_tile)
{
   auto tiles = [&](int bm, int bn) { return (long long)((M + bm - 1) / bm) * ((N + bn - 1) / bn); };
   const bool pairs = (Cg % 128 == 0);
   int tile = force_tile;
   if (!tile)
      // Short reductions (a 3x3 convolution over 64 or 128 channels) spend as long in a tile's prologue and store as in its
      // K loop.  258 = the 256 x 128 tile with a ring of three slabs (72 KB) and 229 registers per lane: two workgroups
      // share a CU and one's prologue and store overlap the other's MFMAs (measured on 1M rows: K = 576, N = 128
      // 157 -> 134 us, K = 1152, N = 256 479 -> 355 us; K = 2304 is better off with the 256 x 256 tile, 760 vs 807 us).
      // 128 x 128 tiles also fit twice.  257 = the 256 x 128 tile with a ring of five, by request only.
      tile = (N > 128 && K > 1536 && tiles(256, 256) >= 256) ? 256
             : (N >= 128 && tiles(256, 128) >= 512)          ? 258
             : (N > 64 && tiles(128, 128) >= 192)            ? 128
                                                             : 64;
   switch (tile) {
   case 256:
      if (pairs)
         return launch_mfma8_pair_src<MfmaI8, 256, 256, 64, 2, 2, 5, EPI, 0, ConvRows>(stream, a, Wp, M, N, K, K, ep);
      return launch_mfma8_dma_src<MfmaI8, 256, 256, 64, 2, 2, 4, EPI, 0, ConvRows>(stream, a, Wp, M, N, K, K, ep);
   case 257:
      if (pairs)
         return launch_mfma8_pair_src<MfmaI8, 256, 128, 64, 2, 2, 5, EPI, 0, ConvRows>(stream, a, Wp, M, N, K, K, ep);
      return launch_mfma8_dma_src<MfmaI8, 256, 128, 64, 2, 2, 4, EPI, 0, ConvRows>(stream, a, Wp, M, N, K, K, ep);
   case 258: return launch_mfma8_dma_src<MfmaI8, 256, 128, 64, 2, 2, 3, EPI, 0, ConvRows, 2>(stream, a, Wp, M, N, K, K, ep);
#ifdef SOFIE_HIP_TUNING
   case 259: return launch_mfma8_dma_src<MfmaI8, 256, 128, 64, 2, 2, 4, EPI, 0, ConvRows, 1>(stream, a, Wp, M, N, K, K, ep);
   case 260: return launch_mfma8_dma_src<MfmaI8, 128, 256, 64, 2, 2, 3, EPI, 0, ConvRows, 2>(stream, a, Wp, M, N, K, K, ep);
   case 129: return launch_mfma8_dma_src<MfmaI8, 128, 128, 64, 2, 2, 4, EPI, 0, ConvRows, 2>(stream, a, Wp, M, N, K, K, ep);
#endif
   case 128: return launch_mfma8_dma_src<MfmaI8, 128, 128, 64, 2, 2, 4, EPI, 0, ConvRows>(stream, a, Wp, M, N, K, K, ep);
   case 64: return launch_mfma8_dma_src<MfmaI8, 64, 64, 64, 2, 2, 4, EPI, 0, ConvRows>(stream, a, Wp, M, N, K, K, ep);
   default: return fail(SOFIE_HIP_ERR_INVALID, "conv: unknown tile %d", force_tile);
   }
}

} // namespace sofie_hip
