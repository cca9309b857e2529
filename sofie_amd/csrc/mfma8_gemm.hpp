// General tile loop of the int8 and the FP8 GEMM: any K, any alignment.  1-byte operands, both
// K-contiguous in HBM ("NT" form: A is [M,K] row-major, Bt is [N,K] row-major), 32x32 MFMA tiles,
// slabs staged global -> registers -> LDS with one slab of prefetch.  Shapes that allow it run the
// pipelined kernel of mfma8_gemm_dma.hpp instead; this one is the safety net (K tails, odd strides).
//
// A workgroup owns a BM x BN tile of Y and walks K in slabs of BK bytes kept in the swizzled LDS layout
// of lds_chunk_offset.  The MFMA is issued with the Bt rows as its first operand and the A rows as its
// second, so that a lane ends up holding 4 consecutive output columns n of one output row m.  Which K
// bytes a lane feeds to the MFMA only has to be the same for both operands, because the dot product does
// not depend on the order of its terms (exactly for int8, to rounding for FP8).
#pragma once
#include "mfma8_common.hpp"

namespace sofie_hip {

// Loads one 16-byte chunk (bytes k..k+15 of the row at `row_ptr`); bytes at k >= K read as 0.
template <bool ALIGNED>
__device__ __forceinline__ v4i load_chunk(const int8_t *row_ptr, int k, int K)
{
   const int8_t *p = row_ptr + k;
   if (ALIGNED) {
      if (k < K)
         return *(const v4i *)p;
      return v4i{0, 0, 0, 0};
   } else {
      union {
         v4i v;
         int8_t b[16];
      } u;
      u.v = v4i{0, 0, 0, 0};
#pragma unroll
      for (int i = 0; i < 16; ++i)
         if (k + i < K)
            u.b[i] = p[i];
      return u.v;
   }
}

template <int BM, int BN, int BK, int WAVES_M, int WAVES_N>
constexpr size_t mfma8_general_lds_bytes()
{
   constexpr size_t ring = 2 * (size_t)(BM + BN) * BK;
   constexpr size_t store = (size_t)WAVES_M * WAVES_N * tile_store_lds_bytes(BN / WAVES_N);
   return ring > store ? ring : store;
}

// OCC: waves per SIMD the register allocation leaves room for.
template <class MMA, int BM, int BN, int BK, int WAVES_M, int WAVES_N, bool ALIGNED, class EPI, class ASRC = RowMajorRows, int OCC = 1>
__global__ __launch_bounds__(WAVES_M *WAVES_N * 64, OCC) void mfma8_gemm_kernel(ASRC A, RowMajorRows Bt, int M, int N,
                                                                            int K, EPI ep, int tiles_m, int tiles_n, int sw)
{
   constexpr int NTHREADS = WAVES_M * WAVES_N * 64;
   constexpr int CPR = BK / 16;
   constexpr int TM = BM / WAVES_M, TN = BN / WAVES_N; // wave tile
   constexpr int MT = TM / 32, NT = TN / 32;           // 32x32 MFMA tiles per wave
   constexpr int A_LD = BM * CPR / NTHREADS, B_LD = BN * CPR / NTHREADS;
   static_assert(BM * CPR % NTHREADS == 0 && BN * CPR % NTHREADS == 0, "tile must divide over the threads");
   static_assert(TM % 32 == 0 && TN % 32 == 0, "wave tile must be a multiple of 32x32");
   static_assert(BK % MMA::KSTEP == 0, "BK must be a multiple of the MFMA K");
   typedef typename MMA::acc_t acc_t;
   typedef typename MMA::frag_t frag_t;

   extern __shared__ __attribute__((aligned(16))) int8_t smem[];
   int8_t *sA = smem;               // [2][BM*BK]
   int8_t *sB = smem + 2 * BM * BK; // [2][BN*BK]

   int tm, tn;
   tile_of_block(blockIdx.x, gridDim.x, tiles_m, tiles_n, sw, tm, tn);
   const int m0 = tm * BM, n0 = tn * BN;
   const int t = threadIdx.x;
   const int lane = t & 63, wave = t >> 6;
   const int wm = wave / WAVES_N, wn = wave % WAVES_N;

   acc_t acc[MT][NT];
#pragma unroll
   for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
         for (int v = 0; v < 16; ++v)
            acc[i][j][v] = 0;

   // global -> register staging: chunk id = t + i*NTHREADS -> (row, chunk)
   v4i ra[A_LD], rb[B_LD];
   const int8_t *a_row[A_LD], *b_row[B_LD];
   if constexpr (!ASRC::kGather) {
#pragma unroll
      for (int i = 0; i < A_LD; ++i) {
         int gr = m0 + (t + i * NTHREADS) / CPR;
         a_row[i] = A.row(gr < M ? gr : M - 1);
      }
   } else {
      // the whole reduction is one slab: every lane gathers the 64 bytes of its own row (pixel)
      static_assert(!ASRC::kGather || (BM == NTHREADS && BK == 64), "the gathered source fills one row per thread of one 64-byte slab");
      const auto ref = A.ref_of(m0 + t, M);
      unsigned w[16];
#pragma unroll
      for (int i = 0; i < 16; ++i)
         w[i] = 0;
      // every load is issued unconditionally (a tap outside the image reads the first byte of the tensor instead and is
      // masked afterwards), so that the loads of a row are in flight together instead of one memory round trip per tap
      constexpr int KP = ASRC::kKP;
      unsigned v[KP];
      unsigned ok_lo = 0, ok_hi = 0; // bit k: tap k lies inside the image
#pragma unroll
      for (int k = 0; k < KP; ++k) {
         const int ih = ref.ih0 + A.dy[k], iw = ref.iw0 + A.dx[k];
         const bool in = k < A.K && (unsigned)ih < (unsigned)A.H && (unsigned)iw < (unsigned)A.W; // k >= K: padding of the reduction
         if (k < 32)
            ok_lo |= in ? (1u << (k & 31)) : 0u;
         else
            ok_hi |= in ? (1u << (k & 31)) : 0u;
         const int8_t *p = in ? ref.origin + A.koff[k] : A.X;
         v[k] = (unsigned char)*p;
      }
#pragma unroll
      for (int k = 0; k < KP; ++k) {
         const unsigned bit = ((k < 32 ? ok_lo : ok_hi) >> (k & 31)) & 1u;
         w[k / 4] |= (bit ? v[k] : 0u) << (8 * (k % 4));
      }
#pragma unroll
      for (int c = 0; c < 4; ++c)
         *(v4i *)(sA + lds_chunk_offset<BK>(t, c)) = v4i{(int)w[4 * c], (int)w[4 * c + 1], (int)w[4 * c + 2], (int)w[4 * c + 3]};
   }
#pragma unroll
   for (int i = 0; i < B_LD; ++i) {
      int gr = n0 + (t + i * NTHREADS) / CPR;
      b_row[i] = Bt.row(gr < N ? gr : N - 1);
   }
   auto load_global = [&](int k0) {
      if constexpr (!ASRC::kGather) {
#pragma unroll
         for (int i = 0; i < A_LD; ++i)
            ra[i] = load_chunk<ALIGNED>(a_row[i], k0 + ((t + i * NTHREADS) % CPR) * 16, K);
      }
#pragma unroll
      for (int i = 0; i < B_LD; ++i)
         rb[i] = load_chunk<ALIGNED>(b_row[i], k0 + ((t + i * NTHREADS) % CPR) * 16, K);
   };
   auto store_lds = [&](int stage) {
      if constexpr (!ASRC::kGather) {
#pragma unroll
         for (int i = 0; i < A_LD; ++i) {
            int id = t + i * NTHREADS;
            *(v4i *)(sA + stage * BM * BK + lds_chunk_offset<BK>(id / CPR, id % CPR)) = ra[i];
         }
      }
#pragma unroll
      for (int i = 0; i < B_LD; ++i) {
         int id = t + i * NTHREADS;
         *(v4i *)(sB + stage * BN * BK + lds_chunk_offset<BK>(id / CPR, id % CPR)) = rb[i];
      }
   };

   const int KT = (K + BK - 1) / BK;
   load_global(0);
   store_lds(0);
   __syncthreads();

   const int lr = lane & 31, lk = lane >> 5;
   for (int kt = 0; kt < KT; ++kt) {
      const int cur = kt & 1;
      if (kt + 1 < KT)
         load_global((kt + 1) * BK);
      const int8_t *cA = sA + cur * BM * BK;
      const int8_t *cB = sB + cur * BN * BK;
#pragma unroll
      for (int ks = 0; ks < BK / MMA::KSTEP; ++ks) {
         frag_t fa[MT], fb[NT];
#pragma unroll
         for (int j = 0; j < NT; ++j)
#pragma unroll
            for (int c = 0; c < MMA::CHUNKS; ++c)
               fb[j].c[c] = *(const v4i *)(cB + lds_chunk_offset<BK>(wn * TN + j * 32 + lr, (ks * 2 + lk) * MMA::CHUNKS + c));
#pragma unroll
         for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int c = 0; c < MMA::CHUNKS; ++c)
               fa[i].c[c] = *(const v4i *)(cA + lds_chunk_offset<BK>(wm * TM + i * 32 + lr, (ks * 2 + lk) * MMA::CHUNKS + c));
#pragma unroll
         for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < NT; ++j)
               acc[i][j] = MMA::mma(fb[j], fa[i], acc[i][j]);
      }
      if (kt + 1 < KT)
         store_lds(cur ^ 1);
      __syncthreads();
   }

   // the slabs are dead (the loop ends with a barrier): the tile store reuses LDS, one region per wave
   char *wsm = (char *)smem + wave * tile_store_lds_bytes(TN);
   ep.dispatch([&](auto mode) {
      tile_store_via_lds<decltype(mode)::value, MT, NT>(ep, acc, m0 + wm * TM, n0 + wn * TN, M, N, lane, wsm);
   });
}

// One attribute call per kernel and device (it is far slower than a launch).
template <class KERN>
static int configure_lds_once(KERN kern, size_t smem, bool (&configured)[64])
{
   int dev = 0;
   SOFIE_HIP_CHECK(hipGetDevice(&dev));
   if (dev < 0 || dev >= 64 || !configured[dev]) {
      SOFIE_HIP_CHECK(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
      if (dev >= 0 && dev < 64)
         configured[dev] = true;
   }
   return SOFIE_HIP_OK;
}

template <class MMA, int BM, int BN, int BK, int WAVES_M, int WAVES_N, class EPI>
static int launch_mfma8(const LaunchCfg &lc, const int8_t *A, const int8_t *Bt, int M, int N, int K, int lda, int ldb,
                        const EPI &ep, bool aligned)
{
   const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
   const long long nwg = (long long)tiles_m * tiles_n;
   if (nwg > 0x7fffffffLL)
      return fail(SOFIE_HIP_ERR_INVALID, "gemm: too many tiles");
   constexpr size_t smem = mfma8_general_lds_bytes<BM, BN, BK, WAVES_M, WAVES_N>();
   constexpr int NTHREADS = WAVES_M * WAVES_N * 64;
   RowMajorRows a{A, lda}, b{Bt, ldb};
      int st;
   if (aligned) {
      auto kern = mfma8_gemm_kernel<MMA, BM, BN, BK, WAVES_M, WAVES_N, true, EPI>;
      static bool configured[64] = {};
      if ((st = configure_lds_once(kern, smem, configured)))
         return st;
      hipLaunchKernelGGL(kern, dim3((unsigned)nwg), dim3(NTHREADS), smem, lc.stream, a, b, M, N, K, ep, tiles_m, tiles_n, lc.swizzle);
   } else {
      auto kern = mfma8_gemm_kernel<MMA, BM, BN, BK, WAVES_M, WAVES_N, false, EPI>;
      static bool configured[64] = {};
      if ((st = configure_lds_once(kern, smem, configured)))
         return st;
      hipLaunchKernelGGL(kern, dim3((unsigned)nwg), dim3(NTHREADS), smem, lc.stream, a, b, M, N, K, ep, tiles_m, tiles_n, lc.swizzle);
   }
   return launch_status("mfma8_gemm_kernel");
}

// Tile choice: the largest one that still gives every one of the 256 CUs a workgroup.
inline int pick_tile(int M, int N, int force_tile)
{
   if (force_tile == 256 || force_tile == 128 || force_tile == 64)
      return force_tile;
   // any other request (the convolution's extra tile shapes) leaves the plain product to the heuristic
   auto tiles = [&](int bm, int bn) { return (long long)((M + bm - 1) / bm) * ((N + bn - 1) / bn); };
   // a tile wider than the matrix would spend its matrix-core time on columns that do not exist
   if (N > 128 && tiles(256, 256) >= 256)
      return 256;
   if (N > 64 && tiles(128, 128) >= 192)
      return 128;
   return 64;
}

// Convolution over few input channels as ONE launch: 256 x 64 tiles (one output pixel per thread in the gather), a single
// 64-byte slab.  Wp is the packed weight [N][Kp], Kp = the reduction length rounded up to 16, at most 64.
template <class EPI, int KP>
static int launch_mfma8_gather_kp(const LaunchCfg &lc, const GatherConvRows &a, const int8_t *Wp, int M, int N, const EPI &ep)
{
   constexpr int BM = 256, BN = 64, BK = 64;
   const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
   const long long nwg = (long long)tiles_m * tiles_n;
   if (nwg > 0x7fffffffLL)
      return fail(SOFIE_HIP_ERR_INVALID, "conv: too many tiles");
   constexpr size_t smem = mfma8_general_lds_bytes<BM, BN, BK, 4, 1>();
   // three waves per SIMD (at most 170 registers; the kernel needs 168): each workgroup is one chain of memory round trips
   // (gather, weights, store), so the time goes down with the number of workgroups a CU holds (first layer of the benchmark CNN:
   // 74 us with two, 59 us with three; four would spill)
   auto kern = mfma8_gemm_kernel<MfmaI8, BM, BN, BK, 4, 1, true, EPI, GatherConvRowsT<KP>, 3>;
   static bool configured[64] = {};
   if (int st = configure_lds_once(kern, smem, configured))
      return st;
   GatherConvRowsT<KP> src;
   static_cast<GatherConvRows &>(src) = a;
   hipLaunchKernelGGL(kern, dim3((unsigned)nwg), dim3(256), smem, lc.stream, src, RowMajorRows{Wp, KP}, M, N, KP, ep, tiles_m, tiles_n, 0);
   return launch_status("mfma8_gemm_kernel (gathered convolution)");
}

// Convolution over few input channels as ONE launch: 256 x 64 tiles (one output pixel per thread in the gather), a single
// 64-byte slab.  Wp is the packed weight [N][Kp], Kp = the reduction length rounded up to 16, at most 64.
template <class EPI>
static int launch_mfma8_gather(const LaunchCfg &lc, const GatherConvRows &a, const int8_t *Wp, int M, int N, int Kp, const EPI &ep)
{
   if (a.K > Kp)
      return fail(SOFIE_HIP_ERR_INVALID, "conv: the gathered form needs a reduction of at most 64 bytes");
   switch (Kp) {
   case 16: return launch_mfma8_gather_kp<EPI, 16>(lc, a, Wp, M, N, ep);
   case 32: return launch_mfma8_gather_kp<EPI, 32>(lc, a, Wp, M, N, ep);
   case 48: return launch_mfma8_gather_kp<EPI, 48>(lc, a, Wp, M, N, ep);
   case 64: return launch_mfma8_gather_kp<EPI, 64>(lc, a, Wp, M, N, ep);
   default: return fail(SOFIE_HIP_ERR_INVALID, "conv: the gathered form needs a reduction of at most 64 bytes");
   }
}

template <class MMA, class EPI>
static int launch_mfma8_auto(const LaunchCfg &lc, const int8_t *A, const int8_t *Bt, int M, int N, int K, int lda, int ldb,
                             const EPI &ep)
{
   const int force_tile = lc.tile;
   const bool aligned = (K % 16 == 0) && (lda % 16 == 0) && (ldb % 16 == 0) && (((uintptr_t)A & 15) == 0) &&
                        (((uintptr_t)Bt & 15) == 0);
   switch (pick_tile(M, N, force_tile)) {
   case 256: return launch_mfma8<MMA, 256, 256, 64, 2, 2, EPI>(lc, A, Bt, M, N, K, lda, ldb, ep, aligned);
   case 128: return launch_mfma8<MMA, 128, 128, 64, 2, 2, EPI>(lc, A, Bt, M, N, K, lda, ldb, ep, aligned);
   case 64: return launch_mfma8<MMA, 64, 64, 64, 2, 2, EPI>(lc, A, Bt, M, N, K, lda, ldb, ep, aligned);
   default: return fail(SOFIE_HIP_ERR_INVALID, "gemm: unknown tile %d", force_tile);
   }
}

} // namespace sofie_hip
