// Pipelined tile loop of the int8 / FP8 GEMM for full-speed shapes: K a multiple of BK, rows 16-byte
// aligned.  Same tile ownership, LDS layout, operand roles and epilogue as mfma8_gemm_tile, but
//   * the K slabs go from HBM/L2 straight into LDS (global_load_lds_dwordx4: a wave instruction fills
//     1024 consecutive LDS bytes, lane l writing bytes [16 l, 16 l + 16), and each lane picks the
//     global address whose chunk belongs at that position of the XOR-swizzled layout);
//   * LDS is a ring of STAGES slabs, loads run STAGES-1 slabs ahead of the MFMAs;
//   * one workgroup barrier per slab, placed inside the last K-step of the slab before it: passing it
//     means the next slab has landed for every wave and every wave is done reading the slab before the
//     current one, whose ring slot is refilled right after;
//   * operand fragments are double-buffered in registers and the ds_reads of K-step s+1 are slotted
//     between the MFMAs of step s, so LDS traffic of the four waves spreads over the MFMA time.
#pragma once
#include "mfma8_gemm.hpp"
#include <cstdlib>

namespace sofie_hip {

typedef __attribute__((address_space(3))) void lds_void_t;
typedef __attribute__((address_space(1))) const void global_void_t;

template <int N>
__device__ __forceinline__ void wait_vmcnt()
{
   // s_waitcnt immediate: vmcnt in bits [3:0] and [15:14], expcnt [6:4] and lgkmcnt [11:8] left at "no wait"
   static_assert(N >= 0 && N < 64, "vmcnt range");
   __builtin_amdgcn_s_waitcnt((N & 0xf) | ((N >> 4) << 14) | (0x7 << 4) | (0xf << 8));
}

template <class MMA, int BM, int BN, int BK, int WAVES_M, int WAVES_N, int STAGES, class EPI, int DBG = 0>
__global__ __launch_bounds__(WAVES_M *WAVES_N * 64) void mfma8_gemm_dma_kernel(RowMajorRows A, RowMajorRows Bt, int M, int N,
                                                                                int K, EPI ep, int tiles_m, int tiles_n, int sw)
{
   constexpr int NW = WAVES_M * WAVES_N;
   constexpr int CPR = BK / 16;           // 16-byte chunks per LDS row
   constexpr int RPI = 64 / CPR;          // rows filled by one wave instruction (1024 bytes)
   constexpr int A_LD = BM / RPI / NW, B_LD = BN / RPI / NW;
   constexpr int LPT = A_LD + B_LD;       // loads per lane and slab
   constexpr int TM = BM / WAVES_M, TN = BN / WAVES_N;
   constexpr int MT = TM / 32, NT = TN / 32;
   constexpr int KS = BK / MMA::KSTEP;
   constexpr int STAGE_BYTES = (BM + BN) * BK;
   static_assert(BM % (RPI * NW) == 0 && BN % (RPI * NW) == 0, "tile rows must divide over the waves");
   static_assert(STAGES >= 3 && (STAGES - 1) * LPT < 64, "ring needs >= 3 slots; vmcnt counts < 64 loads");
   typedef typename MMA::acc_t acc_t;
   typedef typename MMA::frag_t frag_t;

   extern __shared__ __attribute__((aligned(16))) int8_t smem[];

   int tm, tn;
   tile_of_block(blockIdx.x, gridDim.x, tiles_m, tiles_n, sw, tm, tn);
   const int m0 = tm * BM, n0 = tn * BN;
   const int t = threadIdx.x;
   const int lane = t & 63, wave = t >> 6;
   const int wm = wave / WAVES_N, wn = wave % WAVES_N;
   const int lr = lane & 31, lk = lane >> 5;

   // per-lane global source of every load instruction of a slab (k offset added per slab)
   const int8_t *ga[A_LD], *gb[B_LD];
#pragma unroll
   for (int i = 0; i < A_LD; ++i) {
      const int row = (i * NW + wave) * RPI + lane / CPR; // row of the tile this lane fills
      constexpr int RPB = (256 / BK) > 0 ? (256 / BK) : 1;
      const int c = (lane % CPR) ^ ((row / RPB) % CPR);   // logical chunk stored at this lane's LDS position
      const int gr = m0 + row;
      ga[i] = A.row(gr < M ? gr : M - 1) + c * 16;
   }
#pragma unroll
   for (int i = 0; i < B_LD; ++i) {
      const int row = (i * NW + wave) * RPI + lane / CPR;
      constexpr int RPB = (256 / BK) > 0 ? (256 / BK) : 1;
      const int c = (lane % CPR) ^ ((row / RPB) % CPR);
      const int gr = n0 + row;
      gb[i] = Bt.row(gr < N ? gr : N - 1) + c * 16;
   }
   auto issue_loads = [&](int kt, int stage) {
      if (DBG & 1)
         return;
      int8_t *sA = smem + stage * STAGE_BYTES;
      int8_t *sB = sA + BM * BK;
      const int koff = kt * BK;
#pragma unroll
      for (int i = 0; i < A_LD; ++i)
         __builtin_amdgcn_global_load_lds((global_void_t *)(ga[i] + koff), (lds_void_t *)(sA + (i * NW + wave) * 1024), 16, 0, 0);
#pragma unroll
      for (int i = 0; i < B_LD; ++i)
         __builtin_amdgcn_global_load_lds((global_void_t *)(gb[i] + koff), (lds_void_t *)(sB + (i * NW + wave) * 1024), 16, 0, 0);
   };

   acc_t acc[MT][NT];
#pragma unroll
   for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
         for (int v = 0; v < 16; ++v)
            acc[i][j][v] = 0;

   const int KT = K / BK;
#pragma unroll
   for (int s = 0; s < STAGES - 1; ++s)
      if (s < KT)
         issue_loads(s, s);

   auto read_frags = [&](const int8_t *cA, const int8_t *cB, int ks, frag_t(&fa)[MT], frag_t(&fb)[NT]) {
      if (DBG & 2)
         return;
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
   };

   // Software pipeline.  The fragments of K-step s+1 are read from LDS while the MFMAs of step s issue
   // (one ds_read slotted after every second MFMA), across slab boundaries too: the wait for the next
   // slab and the workgroup barrier sit inside the last K-step of the current slab, so the first
   // fragments of slab kt+1 are on their way before the MFMAs of slab kt have drained.
   //   barrier in the last step of slab kt  =>  every wave's loads of slab kt+1 have landed, and every
   //   wave has issued all its reads of slab kt-1 (and kt), so the ring slot of slab kt-1 can be refilled.
   frag_t fa[2][MT], fb[2][NT];
   wait_vmcnt<(STAGES - 2) * LPT>();
   if (KT < STAGES - 1)
      wait_vmcnt<0>();
   __builtin_amdgcn_s_barrier();
   read_frags(smem, smem + BM * BK, 0, fa[0], fb[0]);
   int stage = 0;
   int cur = 0;
   for (int kt = 0; kt < KT; ++kt) {
      const int8_t *cA = smem + stage * STAGE_BYTES;
      const int8_t *cB = cA + BM * BK;
      const int nstage = (stage + 1 == STAGES) ? 0 : stage + 1;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
         if (ks == KS - 1) {
            // slab kt+1 must have landed before its first fragments are read below; slab kt+STAGES-1 is then
            // requested into the slot slab kt-1 occupied
            const int ahead = KT - 2 - kt; // slabs issued after kt+1
            if (ahead >= STAGES - 3)
               wait_vmcnt<(STAGES - 3) * LPT>();
            else
               wait_vmcnt<0>();
            __builtin_amdgcn_s_barrier();
            if (kt + STAGES - 1 < KT)
               issue_loads(kt + STAGES - 1, (stage + STAGES - 1) % STAGES);
            // unconditional (after the last slab it reads a dead ring slot and the values are dropped):
            // a branch here would split the block and undo the read/MFMA interleave
            read_frags(smem + nstage * STAGE_BYTES, smem + nstage * STAGE_BYTES + BM * BK, 0, fa[cur ^ 1], fb[cur ^ 1]);
         } else {
            read_frags(cA, cB, ks + 1, fa[cur ^ 1], fb[cur ^ 1]);
         }
#pragma unroll
         for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < NT; ++j)
               if (!(DBG & 4))
                  acc[i][j] = MMA::mma(fb[cur][j], fa[cur][i], acc[i][j]);
               else
                  acc[i][j][0] += fb[cur][j].c[0][0] + fa[cur][i].c[0][0];
         // interleave: one LDS read after every second MFMA
#pragma unroll
         for (int g = 0; g < (MT + NT) * MMA::CHUNKS; ++g) {
            __builtin_amdgcn_sched_group_barrier(0x008, (MT * NT) / ((MT + NT) * MMA::CHUNKS) > 0 ? (MT * NT) / ((MT + NT) * MMA::CHUNKS) : 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
         }
         cur ^= 1;
      }
      stage = nstage;
   }

   // every wave is done with the ring (and nothing is in flight into it): the tile store reuses it
   wait_vmcnt<0>();
   __syncthreads();
   char *wsm = (char *)smem + wave * tile_store_lds_bytes(TN);
   ep.dispatch([&](auto mode) {
      tile_store_via_lds<decltype(mode)::value, MT, NT>(ep, acc, m0 + wm * TM, n0 + wn * TN, M, N, lane, wsm);
   });
}

template <class MMA, int BM, int BN, int BK, int WAVES_M, int WAVES_N, int STAGES, class EPI, int DBG = 0>
static int launch_mfma8_dma(hipStream_t stream, const int8_t *A, const int8_t *Bt, int M, int N, int K, int lda, int ldb,
                            const EPI &ep)
{
   const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
   const long long nwg = (long long)tiles_m * tiles_n;
   if (nwg > 0x7fffffffLL)
      return fail(SOFIE_HIP_ERR_INVALID, "gemm: too many tiles");
   if (K % BK != 0 || K < BK)
      return fail(SOFIE_HIP_ERR_INVALID, "gemm: the pipelined kernel needs K to be a multiple of %d", BK);
   constexpr size_t smem = (size_t)STAGES * (BM + BN) * BK;
   static_assert(smem <= 160 * 1024, "LDS ring larger than the CU's LDS");
   static_assert(smem >= (size_t)WAVES_M * WAVES_N * tile_store_lds_bytes(BN / WAVES_N), "ring too small for the tile store");
   constexpr int NTHREADS = WAVES_M * WAVES_N * 64;
   RowMajorRows a{A, lda}, b{Bt, ldb};
   auto kern = mfma8_gemm_dma_kernel<MMA, BM, BN, BK, WAVES_M, WAVES_N, STAGES, EPI, DBG>;
   static bool configured[64] = {};
   if (int st = configure_lds_once(kern, smem, configured))
      return st;
   hipLaunchKernelGGL(kern, dim3((unsigned)nwg), dim3(NTHREADS), smem, stream, a, b, M, N, K, ep, tiles_m, tiles_n, swizzle_mode());
   return launch_status("mfma8_gemm_dma_kernel");
}

} // namespace sofie_hip

namespace sofie_hip {

// Chooses between the pipelined kernel (aligned operands, K a multiple of 64) and the general one.
// `variant` selects a tuning alternative of the pipelined kernel (0 = default); -1 forces the general kernel.
template <class MMA, class EPI>
static int launch_mfma8_best(hipStream_t stream, const int8_t *A, const int8_t *Bt, int M, int N, int K, int lda, int ldb,
                             const EPI &ep, int force_tile, int variant)
{
   const bool aligned = (lda % 16 == 0) && (ldb % 16 == 0) && (((uintptr_t)A & 15) == 0) && (((uintptr_t)Bt & 15) == 0);
   if (variant < 0 || !aligned || K < 64 || K % 64 != 0)
      return launch_mfma8_auto<MMA, EPI>(stream, A, Bt, M, N, K, lda, ldb, ep, force_tile);
   const int tile = pick_tile(M, N, force_tile);
   switch (tile) {
   case 256:
      if (variant == 1)
         return launch_mfma8_dma<MMA, 256, 256, 64, 2, 2, 3, EPI>(stream, A, Bt, M, N, K, lda, ldb, ep);
      if (variant == 2)
         return launch_mfma8_dma<MMA, 256, 256, 64, 2, 2, 5, EPI>(stream, A, Bt, M, N, K, lda, ldb, ep);
#ifdef SOFIE_HIP_TUNING
      if (variant == 11)
         return launch_mfma8_dma<MMA, 256, 256, 64, 2, 2, 4, EPI, 1>(stream, A, Bt, M, N, K, lda, ldb, ep);
      if (variant == 12)
         return launch_mfma8_dma<MMA, 256, 256, 64, 2, 2, 4, EPI, 2>(stream, A, Bt, M, N, K, lda, ldb, ep);
      if (variant == 13)
         return launch_mfma8_dma<MMA, 256, 256, 64, 2, 2, 4, EPI, 3>(stream, A, Bt, M, N, K, lda, ldb, ep);
      if (variant == 14)
         return launch_mfma8_dma<MMA, 256, 256, 64, 2, 2, 4, EPI, 4>(stream, A, Bt, M, N, K, lda, ldb, ep);
      if (variant == 16)
         return launch_mfma8_dma<MMA, 256, 256, 64, 2, 2, 4, EPI, 6>(stream, A, Bt, M, N, K, lda, ldb, ep);
#endif
      return launch_mfma8_dma<MMA, 256, 256, 64, 2, 2, 4, EPI>(stream, A, Bt, M, N, K, lda, ldb, ep);
   case 128: return launch_mfma8_dma<MMA, 128, 128, 64, 2, 2, 4, EPI>(stream, A, Bt, M, N, K, lda, ldb, ep);
   case 64: return launch_mfma8_dma<MMA, 64, 64, 64, 2, 2, 4, EPI>(stream, A, Bt, M, N, K, lda, ldb, ep);
   default: return fail(SOFIE_HIP_ERR_INVALID, "gemm: unknown tile %d", tile);
   }
}

} // namespace sofie_hip
