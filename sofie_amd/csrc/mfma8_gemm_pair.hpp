// Pipelined tile loop for the largest tile (256 x 256, 64-byte K slabs), where the LDS ring cannot hold
// slabs of whole 128-byte cache lines: the slabs are loaded in PAIRS.  Slab 2p holds bytes [0,64) and slab
// 2p+1 bytes [64,128) of the same cache line of every row; the two load instructions that fetch the two
// halves of a line are issued back to back, so the vector L1 serves the second one and L2 is asked for
// each line once (loading the halves a slab apart asks L2 twice: the measured L2 -> LDS rate is 13 TB/s
// that way against 21 TB/s for whole lines).
//
// Ring of STAGES (odd) slab slots; slab s lives in slot s % STAGES.  Per pair p the loop runs slab 2p
// (no loads issued) and slab 2p+1, during which the loads of pair p + (STAGES-1)/2 are issued, spread over
// its K-steps, into the slots of slabs 2p-1 and 2p (both released by the barrier that ends slab 2p).
// Everything else (operand roles, LDS layout, fragment double buffer, epilogue) is as in
// mfma8_gemm_dma.hpp; the K-step index runs over the pair, so the fragment parity is a compile-time
// constant for any number of K-steps per slab.
#pragma once
#include "mfma8_gemm_dma.hpp"

namespace sofie_hip {


template <class MMA, int BM, int BN, int BK, int WAVES_M, int WAVES_N, int STAGES, class EPI, class ASRC = RowMajorRows>
__global__ __launch_bounds__(WAVES_M *WAVES_N * 64) void mfma8_gemm_pair_kernel(ASRC A, RowMajorRows Bt, int M, int N,
                                                                                 int K, EPI ep, int tiles_m, int tiles_n, int sw)
{
   constexpr int NW = WAVES_M * WAVES_N;
   constexpr int CPR = BK / 16;
   constexpr int RPI = 64 / CPR;
   constexpr int A_LD = BM / RPI / NW, B_LD = BN / RPI / NW;
   constexpr int LPT = A_LD + B_LD; // loads per lane and slab
   constexpr int TM = BM / WAVES_M, TN = BN / WAVES_N;
   constexpr int MT = TM / 32, NT = TN / 32;
   constexpr int KS = BK / MMA::KSTEP;
   constexpr int STAGE_BYTES = (BM + BN) * BK;
   constexpr int AHEAD = (STAGES - 1) / 2; // pairs between the one computing and the one being requested
   static_assert(STAGES % 2 == 1 && STAGES >= 5, "an odd number of slots, at least five");
   static_assert(BM % (RPI * NW) == 0 && BN % (RPI * NW) == 0, "tile rows must divide over the waves");
   static_assert((STAGES - 1) * LPT < 64, "vmcnt counts fewer than 64 loads");
   static_assert((2 * LPT) % KS == 0, "the loads of a pair must divide over the K-steps of a slab");
   typedef typename MMA::acc_t acc_t;
   typedef typename MMA::frag_t frag_t;

   extern __shared__ __attribute__((aligned(16))) int8_t smem[];

   int tm, tn;
   tile_of_block(blockIdx.x, gridDim.x, tiles_m, tiles_n, sw, tm, tn);
   const int m0 = tm * BM, n0 = tn * BN;
   const int t = threadIdx.x;
   const int lane = t & 63;
   const int wave = __builtin_amdgcn_readfirstlane(t >> 6); // uniform: keeps the LDS destinations of the loads in scalar registers
   const int wm = wave / WAVES_N, wn = wave % WAVES_N;
   const int lr = lane & 31, lk = lane >> 5;

   // Source of every load instruction of a slab: a uniform part (tile origin + k offset, scalar registers)
   // plus a 32-bit per-lane offset, so that the address needs (almost) no vector arithmetic inside the loop.
   typename ASRC::template lane_state<A_LD> as;
   typename RowMajorRows::template lane_state<B_LD> bs;
#pragma unroll
   for (int i = 0; i < A_LD; ++i) {
      const int row = (i * NW + wave) * RPI + lane / CPR; // row of the tile this lane fills
      constexpr int RPB = (256 / BK) > 0 ? (256 / BK) : 1;
      const int c = (lane % CPR) ^ ((row / RPB) % CPR);   // logical chunk stored at this lane's LDS position
      A.template init<A_LD>(as, i, m0, row, c * 16, M);
   }
#pragma unroll
   for (int i = 0; i < B_LD; ++i) {
      const int row = (i * NW + wave) * RPI + lane / CPR;
      constexpr int RPB = (256 / BK) > 0 ? (256 / BK) : 1;
      const int c = (lane % CPR) ^ ((row / RPB) % CPR);
      Bt.template init<B_LD>(bs, i, n0, row, c * 16, N);
   }

   // Loads [Q0, Q1) of the 2*LPT load instructions of pair `pair`: instruction q fetches row group q/2 of
   // slab 2*pair + q%2, so the two halves of a cache line are requested by consecutive instructions.
   auto issue_pair = [&](int pair, int slot0, int slot1, auto q0_c, auto q1_c) {
      constexpr int Q0 = decltype(q0_c)::value, Q1 = decltype(q1_c)::value;
      const int koff = pair * 2 * BK;
      static_for<Q1 - Q0>([&](auto qc) {
         constexpr int q = Q0 + decltype(qc)::value;
         constexpr int l = q / 2, half = q % 2;
         int8_t *sA = smem + (half ? slot1 : slot0) * STAGE_BYTES;
         int8_t *sB = sA + BM * BK;
         if constexpr (l < A_LD)
            __builtin_amdgcn_global_load_lds((global_void_t *)A.template load_ptr<A_LD>(as, l, koff + half * BK), (lds_void_t *)(sA + (l * NW + wave) * 1024), 16, 0, 0);
         else
            __builtin_amdgcn_global_load_lds((global_void_t *)Bt.template load_ptr<B_LD>(bs, l - A_LD, koff + half * BK),
                                             (lds_void_t *)(sB + ((l - A_LD) * NW + wave) * 1024), 16, 0, 0);
      });
   };

   acc_t acc[MT][NT];
#pragma unroll
   for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
         for (int v = 0; v < 16; ++v)
            acc[i][j][v] = 0;

   // prologue: pairs 0 .. AHEAD-1 (a pair index past the end re-reads the last pair: filler that keeps the
   // number of loads per iteration, and with it the vmcnt bookkeeping, constant)
   const int KP = K / (2 * BK);
#pragma unroll
   for (int p = 0; p < AHEAD; ++p)
      issue_pair(p < KP ? p : KP - 1, 2 * p, 2 * p + 1, std::integral_constant<int, 0>{}, std::integral_constant<int, 2 * LPT>{});

   auto read_frags = [&](const int8_t *cA, const int8_t *cB, int ks, frag_t(&fa)[MT], frag_t(&fb)[NT]) {
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

   frag_t fa[2][MT], fb[2][NT];
   wait_vmcnt<(AHEAD - 1) * 2 * LPT>(); // pair 0 has landed
   __builtin_amdgcn_s_barrier();
   read_frags(smem, smem + BM * BK, 0, fa[0], fb[0]);
   int stage = 0;              // slot of the slab being computed
   int lslot0 = STAGES - 1;    // slots the next requested pair goes to: those of slabs 2p-1 and 2p
   int lslot1 = 0;
   for (int kp = 0; kp < KP; ++kp) {
      const int lpair = (kp + AHEAD < KP) ? kp + AHEAD : KP - 1;
      static_for<2 * KS>([&](auto g_c) {
         constexpr int g = decltype(g_c)::value; // K-step within the pair
         constexpr int h = g / KS, ks = g % KS;
         const int cur = (h == 0) ? stage : (stage + 1 == STAGES ? 0 : stage + 1);
         const int8_t *cA = smem + cur * STAGE_BYTES;
         const int8_t *cB = cA + BM * BK;
         if (ks == KS - 1) {
            const int nxt = (cur + 1 == STAGES) ? 0 : cur + 1;
            if (h == 1) {
               // issued so far, newest first: parts 0..KS-2 of pair kp+AHEAD, then pairs kp+AHEAD-1 ... kp+1.
               // Pair kp+1 must have landed (its first slab is read next, its second one a slab later).
               wait_vmcnt<(AHEAD - 2) * 2 * LPT + (KS - 1) * (2 * LPT / KS)>();
            }
            __builtin_amdgcn_s_waitcnt(0xc07f); // lgkmcnt(0): this wave's LDS reads of the current slab are complete
            __builtin_amdgcn_s_barrier();
            read_frags(smem + nxt * STAGE_BYTES, smem + nxt * STAGE_BYTES + BM * BK, 0, fa[(g + 1) & 1], fb[(g + 1) & 1]);
         } else {
            read_frags(cA, cB, ks + 1, fa[(g + 1) & 1], fb[(g + 1) & 1]);
         }
         constexpr int NLOAD = (h == 1) ? 2 * LPT / KS : 0;
         if constexpr (h == 1)
            issue_pair(lpair, lslot0, lslot1, std::integral_constant<int, ks * NLOAD>{}, std::integral_constant<int, (ks + 1) * NLOAD>{});
#pragma unroll
         for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < NT; ++j)
               acc[i][j] = MMA::mma(fb[g & 1][j], fa[g & 1][i], acc[i][j]);
         // issue order within the step: MFMAs with the LDS reads and the loads slotted in between
         constexpr int NMFMA = MT * NT;
         constexpr int NREAD = (MT + NT) * MMA::CHUNKS;
         constexpr int GROUPS = NLOAD > 0 ? NLOAD : 4;
         constexpr int MPG = NMFMA / GROUPS > 0 ? NMFMA / GROUPS : 1;
         constexpr int RPG = (NREAD + GROUPS - 1) / GROUPS;
#pragma unroll
         for (int gg = 0; gg < GROUPS; ++gg) {
            constexpr int HALF = MPG / 2 > 0 ? MPG / 2 : 1;
            if (NLOAD > 0)
               __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, HALF, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, RPG - RPG / 2, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, MPG - HALF, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, RPG / 2, 0);
         }
      });
      stage = (stage + 2 >= STAGES) ? stage + 2 - STAGES : stage + 2;
      lslot0 = (lslot0 + 2 >= STAGES) ? lslot0 + 2 - STAGES : lslot0 + 2;
      lslot1 = (lslot1 + 2 >= STAGES) ? lslot1 + 2 - STAGES : lslot1 + 2;
   }

   wait_vmcnt<0>();
   __syncthreads();
   char *wsm = (char *)smem + wave * tile_store_lds_bytes(TN);
   ep.dispatch([&](auto mode) {
      tile_store_via_lds<decltype(mode)::value, MT, NT>(ep, acc, m0 + wm * TM, n0 + wn * TN, M, N, lane, wsm);
   });
}

template <class MMA, int BM, int BN, int BK, int WAVES_M, int WAVES_N, int STAGES, class EPI, class ASRC = RowMajorRows>
static int launch_mfma8_pair_src(const LaunchCfg &lc, const ASRC &a, const int8_t *Bt, int M, int N, int K, int ldb,
                             const EPI &ep)
{
   const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
   const long long nwg = (long long)tiles_m * tiles_n;
   if (nwg > 0x7fffffffLL)
      return fail(SOFIE_HIP_ERR_INVALID, "gemm: too many tiles");
   if (K % (2 * BK) != 0 || K < 2 * BK)
      return fail(SOFIE_HIP_ERR_INVALID, "gemm: the paired-slab kernel needs K to be a multiple of %d", 2 * BK);
   constexpr size_t ring = (size_t)STAGES * (BM + BN) * BK;
   constexpr size_t store = (size_t)WAVES_M * WAVES_N * tile_store_lds_bytes(BN / WAVES_N);
   constexpr size_t smem = ring > store ? ring : store;
   static_assert(smem <= 160 * 1024, "LDS ring larger than the CU's LDS");
   constexpr int NTHREADS = WAVES_M * WAVES_N * 64;
   RowMajorRows b{Bt, ldb};
   auto kern = mfma8_gemm_pair_kernel<MMA, BM, BN, BK, WAVES_M, WAVES_N, STAGES, EPI, ASRC>;
   static bool configured[64] = {};
   if (int st = configure_lds_once(kern, smem, configured))
      return st;
   hipLaunchKernelGGL(kern, dim3((unsigned)nwg), dim3(NTHREADS), smem, lc.stream, a, b, M, N, K, ep, tiles_m, tiles_n, lc.swizzle);
   return launch_status("mfma8_gemm_pair_kernel");
}


template <class MMA, int BM, int BN, int BK, int WAVES_M, int WAVES_N, int STAGES, class EPI>
static int launch_mfma8_pair(const LaunchCfg &lc, const int8_t *A, const int8_t *Bt, int M, int N, int K, int lda, int ldb, const EPI &ep)
{
   return launch_mfma8_pair_src<MMA, BM, BN, BK, WAVES_M, WAVES_N, STAGES, EPI, RowMajorRows>(lc, RowMajorRows{A, lda}, Bt, M, N, K, ldb, ep);
}

} // namespace sofie_hip
