// Kernel choice for the int8 / FP8 GEMM and the int8 convolution: which tile, which pipelined kernel, or the general one.
#pragma once
#include "conv_i8_resident.hpp"

namespace sofie_hip {

// Chooses between the pipelined kernels (aligned operands, K a multiple of 64) and the general one.
// `variant` selects a tuning alternative of the pipelined kernel (0 = default); -1 forces the general kernel.
template <class MMA, class EPI>
static int launch_mfma8_best(const LaunchCfg &lc, const int8_t *A, const int8_t *Bt, int M, int N, int K, int lda, int ldb,
                             const EPI &ep)
{
   const int force_tile = lc.tile, variant = lc.variant;
   const bool aligned = (lda % 16 == 0) && (ldb % 16 == 0) && (((uintptr_t)A & 15) == 0) && (((uintptr_t)Bt & 15) == 0);
   if (variant < 0 || !aligned || K < 64 || K % 64 != 0)
      return launch_mfma8_auto<MMA, EPI>(lc, A, Bt, M, N, K, lda, ldb, ep);
   const int tile = pick_tile(M, N, force_tile);
   const bool k128 = (K % 128 == 0);
   if constexpr (MMA::KSTEP * 2 <= 64) {
      // Large products that divide into whole 256 x 256 tiles: the persistent kernel (512 asks for it by force)
      if ((force_tile == 512 || (!force_tile && variant == 0 && tile == 256)) && mfma8_persist_applies(A, Bt, M, N, K, lda, ldb, ep.elements_per_16_bytes()) &&
          ep.stores_plain_rows())
         return launch_mfma8_persist<MfmaI8x16, EPI>(lc, A, Bt, M, N, K, lda, ldb, ep);
      // Short reductions over many tiles: the 256 x 128 tile with a ring of three slabs fits twice on a CU, and one
      // workgroup's prologue and store overlap the other's K loop (8192 x 4096 x 512: 829 -> 1019 TOP/s, 8192 x 1024 x 1024:
      // 1003 -> 1091; no gain from K = 2048 on).  258 asks for it by force.
      const long long tiles_256x128 = (long long)((M + 255) / 256) * ((N + 127) / 128);
      if (force_tile == 258 || (!force_tile && variant == 0 && K <= 1024 && N >= 128 && tiles_256x128 >= 512))
         return launch_mfma8_dma_src<MMA, 256, 128, 64, 2, 2, 3, EPI, RowMajorRows, 2>(lc, RowMajorRows{A, lda}, Bt, M, N, K, ldb, ep);
   }
   if constexpr (MMA::KSTEP * 2 > 64) {
      // two K-steps per slab are the minimum: a 64-byte K-step needs 128-byte slabs
      if (!k128)
         return launch_mfma8_auto<MMA, EPI>(lc, A, Bt, M, N, K, lda, ldb, ep);
      if ((force_tile == 512 || (!force_tile && variant == 0 && tile == 256)) && mfma8_persist_applies(A, Bt, M, N, K, lda, ldb, ep.elements_per_16_bytes()) &&
          ep.stores_plain_rows())
         return launch_mfma8_persist<MMA, EPI>(lc, A, Bt, M, N, K, lda, ldb, ep);
      switch (tile) {
      case 256:
         if (variant == 1)
            return launch_mfma8_dma<MMA, 256, 128, 128, 2, 2, 3, EPI>(lc, A, Bt, M, N, K, lda, ldb, ep);
         return launch_mfma8_pair<MMA, 256, 256, 64, 2, 2, 5, EPI>(lc, A, Bt, M, N, K, lda, ldb, ep);
      case 128: return launch_mfma8_dma<MMA, 128, 128, 128, 2, 2, 3, EPI>(lc, A, Bt, M, N, K, lda, ldb, ep);
      case 64: return launch_mfma8_dma<MMA, 64, 64, 128, 2, 2, 4, EPI>(lc, A, Bt, M, N, K, lda, ldb, ep);
      default: return fail(SOFIE_HIP_ERR_INVALID, "gemm: unknown tile %d", tile);
      }
   } else {
      switch (tile) {
      case 256:
         if (variant == 1 || !k128)
            return launch_mfma8_dma<MMA, 256, 256, 64, 2, 2, 4, EPI>(lc, A, Bt, M, N, K, lda, ldb, ep);
         return launch_mfma8_pair<MMA, 256, 256, 64, 2, 2, 5, EPI>(lc, A, Bt, M, N, K, lda, ldb, ep);
      case 128:
         if (variant == 1 || !k128)
            return launch_mfma8_dma<MMA, 128, 128, 64, 2, 2, 4, EPI>(lc, A, Bt, M, N, K, lda, ldb, ep);
         return launch_mfma8_dma<MMA, 128, 128, 128, 2, 2, 3, EPI>(lc, A, Bt, M, N, K, lda, ldb, ep);
      case 64:
         if (variant == 1 || !k128)
            return launch_mfma8_dma<MMA, 64, 64, 64, 2, 2, 4, EPI>(lc, A, Bt, M, N, K, lda, ldb, ep);
         return launch_mfma8_dma<MMA, 64, 64, 128, 2, 2, 4, EPI>(lc, A, Bt, M, N, K, lda, ldb, ep);
      default: return fail(SOFIE_HIP_ERR_INVALID, "gemm: unknown tile %d", tile);
      }
   }
}

} // namespace sofie_hip

namespace sofie_hip {

// Convolution as one implicit GEMM: A is read through ConvRows (BK = 64 must divide the channels per group),
// Wp is the packed weight [N][K] with K = taps * Cg.
template <class EPI>
static int launch_mfma8_conv(const LaunchCfg &lc, const ConvRows &a, int Cg, const int8_t *Wp, int M, int N, int K, const EPI &ep)
{
   const int force_tile = lc.tile;
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
   // A small 3 x 3 layer (64 channels in, 128 out): weights resident in LDS, each tile's pixels fetched once with their halo.
   // 576 asks for it by force (and any other forced tile keeps it away).
   if ((force_tile == 576 || (!force_tile && lc.variant == 0 && tiles(256, 128) >= 256)) && conv_i8_resident_applies(a, Cg, Wp, M, N, K) &&
       ep.stores_plain_rows())
      return launch_conv_i8_resident<EPI>(lc, a, Wp, M, ep);
   // Whole 256 x 256 tiles, at least one per CU, and a store the register path handles (NHWC rows, or the plane sums of
   // planes that hold whole wave tiles): the persistent kernel.  512 asks for it by force.
   if ((force_tile == 512 || (!force_tile && lc.variant == 0 && tiles(256, 256) >= 256)) &&
       mfma8_persist_conv_applies(a, Wp, M, N, K, ep.elements_per_16_bytes(), !ep.stores_plain_rows()) &&
       (ep.stores_plain_rows() || ep.sums_rows_of_whole_wave_tiles(128)))
      return launch_mfma8_persist_src<MfmaI8x16, EPI, PersistConvRows>(lc, persist_conv_rows(a), Wp, M, N, K, K, ep);
   if (tile == 512 || tile == 576)
      tile = 256;
   switch (tile) {
   case 256:
      if (pairs)
         return launch_mfma8_pair_src<MfmaI8, 256, 256, 64, 2, 2, 5, EPI, ConvRows>(lc, a, Wp, M, N, K, K, ep);
      return launch_mfma8_dma_src<MfmaI8, 256, 256, 64, 2, 2, 4, EPI, ConvRows>(lc, a, Wp, M, N, K, K, ep);
   case 257:
      if (pairs)
         return launch_mfma8_pair_src<MfmaI8, 256, 128, 64, 2, 2, 5, EPI, ConvRows>(lc, a, Wp, M, N, K, K, ep);
      return launch_mfma8_dma_src<MfmaI8, 256, 128, 64, 2, 2, 4, EPI, ConvRows>(lc, a, Wp, M, N, K, K, ep);
   case 258: return launch_mfma8_dma_src<MfmaI8, 256, 128, 64, 2, 2, 3, EPI, ConvRows, 2>(lc, a, Wp, M, N, K, K, ep);
   case 128: return launch_mfma8_dma_src<MfmaI8, 128, 128, 64, 2, 2, 4, EPI, ConvRows>(lc, a, Wp, M, N, K, K, ep);
   case 64: return launch_mfma8_dma_src<MfmaI8, 64, 64, 64, 2, 2, 4, EPI, ConvRows>(lc, a, Wp, M, N, K, K, ep);
   default: return fail(SOFIE_HIP_ERR_INVALID, "conv: unknown tile %d", force_tile);
   }
}

} // namespace sofie_hip
