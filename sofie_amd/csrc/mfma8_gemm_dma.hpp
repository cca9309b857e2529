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

// OCC: workgroups meant to share a CU (waves per SIMD); 2 halves the register budget to 256 per lane so that one
// workgroup's tile store overlaps the other's K loop.
template <class MMA, int BM, int BN, int BK, int WAVES_M, int WAVES_N, int STAGES, class EPI, class ASRC = RowMajorRows, int OCC = 1>
__global__ __launch_bounds__(WAVES_M *WAVES_N * 64, OCC) void mfma8_gemm_dma_kernel(ASRC A, RowMajorRows Bt, int M, int N,
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
   static_assert((STAGES - 1) * LPT < 64, "vmcnt counts fewer than 64 loads");
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

   // per-lane global source of every load instruction of a slab (k offset added per slab)
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
   // One K-step's share of a slab's load instructions (A's first, then Bt's): part `part` of KS equal parts.
   constexpr int KS_ = BK / MMA::KSTEP;
   static_assert(LPT % KS_ == 0, "slab loads must divide over the K-steps");
   auto issue_loads = [&](int kt, int stage, auto part_c) {
      constexpr int part = decltype(part_c)::value; // 0..KS-1, or -1 for the whole slab
      int8_t *sA = smem + stage * STAGE_BYTES;
      int8_t *sB = sA + BM * BK;
      const int koff = kt * BK;
      constexpr int L0 = part < 0 ? 0 : part * (LPT / KS_), L1 = part < 0 ? LPT : (part + 1) * (LPT / KS_);
      static_for<L1 - L0>([&](auto lc) {
         constexpr int l = L0 + decltype(lc)::value;
         if constexpr (l < A_LD)
            __builtin_amdgcn_global_load_lds((global_void_t *)A.template load_ptr<A_LD>(as, l, koff), (lds_void_t *)(sA + (l * NW + wave) * 1024), 16, 0, 0);
         else
            __builtin_amdgcn_global_load_lds((global_void_t *)Bt.template load_ptr<B_LD>(bs, l - A_LD, koff), (lds_void_t *)(sB + ((l - A_LD) * NW + wave) * 1024), 16, 0, 0);
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

   // prologue: slabs 0..STAGES-2 (a slab index past the end re-reads the last slab: harmless filler that
   // keeps the number of loads per iteration, and with it the vmcnt bookkeeping, constant)
   const int KT = K / BK;
#pragma unroll
   for (int s = 0; s < STAGES - 1; ++s)
      issue_loads(s < KT ? s : KT - 1, s, std::integral_constant<int, -1>{});

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

   // Software pipeline, one slab per iteration, everything interleaved at instruction granularity so
   // that neither the LDS nor the vector-memory queue ever sees a burst (a burst of loads blocks the
   // wave at issue and with it the MFMAs behind them):
   //   K-step s:  MFMAs of step s  |  ds_reads of the fragments of step s+1  |  1/KS of the loads of slab kt+STAGES-1
   // The loads of slab kt+STAGES-1 go to the ring slot of slab kt-1.  That slot was released by the barrier
   // of iteration kt-1, which sits in the LAST K-step of a slab, after the wave has waited for its own
   // LDS reads: passing it means every wave's loads of the NEXT slab have landed and every wave is done
   // reading the CURRENT slab's LDS data (its last fragments are in registers).
   static_assert(KS % 2 == 0, "the fragment double buffer is indexed by the parity of the K-step");
   static_assert(STAGES >= 3, "the ring needs three slots: one computing, one landing, one being refilled");
   frag_t fa[2][MT], fb[2][NT];
   wait_vmcnt<(STAGES - 2) * LPT>();
   __builtin_amdgcn_s_barrier();
   read_frags(smem, smem + BM * BK, 0, fa[0], fb[0]);
   int stage = 0;
   int lstage = STAGES - 1; // slot refilled during this iteration
   for (int kt = 0; kt < KT; ++kt) {
      const int8_t *cA = smem + stage * STAGE_BYTES;
      const int8_t *cB = cA + BM * BK;
      const int nstage = (stage + 1 == STAGES) ? 0 : stage + 1;
      const int lslab = (kt + STAGES - 1 < KT) ? kt + STAGES - 1 : KT - 1;
      static_for<KS>([&](auto ks_c) {
         constexpr int ks = decltype(ks_c)::value;
         if (ks == KS - 1) {
            // issued so far, newest first: parts 0..KS-2 of slab kt+STAGES-1, then slabs kt+STAGES-2 ... kt+1.
            // Slab kt+1 must have landed.
            wait_vmcnt<(STAGES - 3) * LPT + (KS - 1) * (LPT / KS)>();
            __builtin_amdgcn_s_waitcnt(0xc07f); // lgkmcnt(0): this wave's LDS reads of slab kt are complete
            __builtin_amdgcn_s_barrier();
            read_frags(smem + nstage * STAGE_BYTES, smem + nstage * STAGE_BYTES + BM * BK, 0, fa[0], fb[0]);
         } else {
            read_frags(cA, cB, ks + 1, fa[(ks + 1) & 1], fb[(ks + 1) & 1]);
         }
         issue_loads(lslab, lstage, ks_c);
#pragma unroll
         for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < NT; ++j)
               acc[i][j] = MMA::mma(fb[ks & 1][j], fa[ks & 1][i], acc[i][j]);
         // issue order within the step: MFMAs with the LDS reads and the loads slotted in between
         constexpr int NMFMA = MT * NT;
         constexpr int NREAD = (MT + NT) * MMA::CHUNKS;
         constexpr int NLOAD = LPT / KS;
         constexpr int GROUPS = NLOAD > 0 ? NLOAD : 1;
         constexpr int MPG = NMFMA / GROUPS > 0 ? NMFMA / GROUPS : 1; // MFMAs per group
         constexpr int RPG = (NREAD + GROUPS - 1) / GROUPS;            // LDS reads per group
#pragma unroll
         for (int g = 0; g < GROUPS; ++g) {
            constexpr int HALF = MPG / 2 > 0 ? MPG / 2 : 1;
            __builtin_amdgcn_sched_group_barrier(0x008, HALF, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, RPG - RPG / 2, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, MPG - HALF, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, RPG / 2, 0);
            __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
         }
      });
      stage = nstage;
      lstage = (lstage + 1 == STAGES) ? 0 : lstage + 1;
   }

   // every wave is done with the ring (and nothing is in flight into it): the tile store reuses it
   wait_vmcnt<0>();
   __syncthreads();
   char *wsm = (char *)smem + wave * tile_store_lds_bytes(TN);
   ep.dispatch_with_reciprocal([&](auto mode) {
      tile_store_via_lds<decltype(mode)::value, MT, NT>(ep, acc, m0 + wm * TM, n0 + wn * TN, M, N, lane, wsm);
   });
}

template <class MMA, int BM, int BN, int BK, int WAVES_M, int WAVES_N, int STAGES, class EPI, class ASRC = RowMajorRows, int OCC = 1>
static int launch_mfma8_dma_src(const LaunchCfg &lc, const ASRC &a, const int8_t *Bt, int M, int N, int K, int ldb,
                            const EPI &ep)
{
   const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
   const long long nwg = (long long)tiles_m * tiles_n;
   if (nwg > 0x7fffffffLL)
      return fail(SOFIE_HIP_ERR_INVALID, "gemm: too many tiles");
   if (K % BK != 0 || K < BK)
      return fail(SOFIE_HIP_ERR_INVALID, "gemm: the pipelined kernel needs K to be a multiple of %d", BK);
   constexpr size_t ring = (size_t)STAGES * (BM + BN) * BK;
   constexpr size_t store = (size_t)WAVES_M * WAVES_N * tile_store_lds_bytes(BN / WAVES_N);
   constexpr size_t smem = ring > store ? ring : store;
   static_assert(smem * OCC <= 160 * 1024, "LDS ring larger than the CU's LDS");
   constexpr int NTHREADS = WAVES_M * WAVES_N * 64;
   RowMajorRows b{Bt, ldb};
   auto kern = mfma8_gemm_dma_kernel<MMA, BM, BN, BK, WAVES_M, WAVES_N, STAGES, EPI, ASRC, OCC>;
   static bool configured[64] = {};
   if (int st = configure_lds_once(kern, smem, configured))
      return st;
   hipLaunchKernelGGL(kern, dim3((unsigned)nwg), dim3(NTHREADS), smem, lc.stream, a, b, M, N, K, ep, tiles_m, tiles_n, lc.swizzle);
   return launch_status("mfma8_gemm_dma_kernel");
}


template <class MMA, int BM, int BN, int BK, int WAVES_M, int WAVES_N, int STAGES, class EPI>
static int launch_mfma8_dma(const LaunchCfg &lc, const int8_t *A, const int8_t *Bt, int M, int N, int K, int lda, int ldb, const EPI &ep)
{
   return launch_mfma8_dma_src<MMA, BM, BN, BK, WAVES_M, WAVES_N, STAGES, EPI, RowMajorRows>(lc, RowMajorRows{A, lda}, Bt, M, N, K, ldb, ep);
}

} // namespace sofie_hip

