// Persistent tile loop of the int8 / FP8 GEMM for large shapes, walked in 256 x 256 tiles.
//
// One workgroup of EIGHT waves per CU (two per SIMD, 256 registers each) walks a list of output tiles; the K loop runs
// straight through the tile boundaries:
//   * the ring of five 64-byte K slabs (paired as in mfma8_gemm_pair.hpp: the two halves of a 128-byte line are
//     requested back to back) never drains: while the last slabs of a tile are multiplied, the first slabs of the
//     workgroup's next tile are already landing;
//   * a wave owns a 128 x 64 piece of the tile (128 accumulator registers), so two waves share a SIMD: while one waits
//     (barrier, LDS, the tile store), the matrix core runs the other's MFMAs;
//   * the tile store needs no LDS (the ring takes all 160 KB): the lanes exchange the converted elements through
//     v_permlane16_swap / v_permlane32_swap until every lane holds 16 consecutive output bytes, and store them.
//
// Step t of the loop multiplies slab t (its fragments are in registers) while the fragments of slab t + 1 are read from
// LDS into the other register buffer, and, on even t, the eight loads of the pair of slabs t + 4, t + 5 are issued.
// One workgroup barrier opens each step.  Before it a wave has waited for its own LDS reads of slab t (so after the
// barrier the ring slot of slab t may be overwritten: that is where slab t + 5 goes) and, on odd t, for its own loads
// of the pair that starts at slab t + 1 (so after the barrier that pair is complete for every wave).
#pragma once
#include "mfma8_gemm_pair.hpp"

namespace sofie_hip {

// Tile store straight from the accumulator registers.  With the Bt fragment as the first MFMA operand a lane holds, per
// register group g, 4 consecutive columns  n = j*R + g*4*LK + lk*4 + (0..3)  of row  m = i*R + lr   (R = rows of the MFMA
// block, lr = lane % R, lk = lane / R, LK = 64 / R).
//   4-byte elements: those are 16 bytes, stored as they are (the LK lanes of a row cover 16*LK consecutive bytes).
//   1-byte elements, R = 16, four column blocks per wave (NT = 4): the four lanes of a row hold a 4 x 4 matrix of dwords
//   (lane lk, block j) -> columns j*16 + lk*4; transposing it (two swap stages) leaves lane lk with the dwords of
//   columns lk*16 .. lk*16 + 15: one 16-byte store per lane and 16-row block.
// The per-column constants of the epilogue (bias, scale) arrive one column per lane (lane l holds those of column
// n_base + l; the wave tile is 64 columns wide) and are handed to the lanes that need them by ds_bpermute: two loads per
// tile instead of one round trip to memory per group of columns.
template <int MODE, class MMA, int MT, int NT, class EPI, class ACC>
__device__ __forceinline__ void tile_store_from_registers(const EPI &ep, ACC (&acc)[MT][NT], int m_base, int n_base, int lane,
                                                          const uint32_t (&col_words)[EPI::kColWords])
{
   constexpr int ESZ = EPI::template out_bytes<MODE>();
   constexpr int R = MMA::ROWS, LK = MMA::LK, G = MMA::ACC / 4;
   static_assert(NT * R == 64, "one column constant per lane");
   const int lr = lane % R, lk = lane / R;
   char *out = ep.out_base();
   // byte address (for ds_bpermute) of the lane that holds the constants of this lane's first column; made opaque so that the
   // sixteen addresses derived from it are recomputed where they are used (one addition each) instead of being kept, and
   // spilled, across the K loop
   int first_col_addr = lk * 16;
   asm volatile("" : "+v"(first_col_addr));
   auto column_constants = [&](int c0, typename EPI::template col_params<4> &prm) { // columns lk*4 + c0 .. + 3 of the wave tile
#pragma unroll
      for (int v = 0; v < 4; ++v) {
         uint32_t w[EPI::kColWords];
#pragma unroll
         for (int k = 0; k < EPI::kColWords; ++k)
            w[k] = (EPI::kBiasInAccumulator && k == EPI::kBiasWord) ? 0u : (uint32_t)__builtin_amdgcn_ds_bpermute(first_col_addr + (c0 + v) * 4, (int)col_words[k]);
         EPI::template set_column<4>(prm, v, w);
      }
   };
   // the conversion of 4 accumulators; an epilogue whose bias sits in the accumulators is told so
   auto convert4 = [&](auto mode_c, const typename EPI::template col_params<4> &prm, const auto &a, int g, uint32_t *w) {
      constexpr int M = decltype(mode_c)::value;
      if constexpr (EPI::kBiasInAccumulator)
         ep.template pack4<M, 4, true>(prm, 0, a[4 * g + 0], a[4 * g + 1], a[4 * g + 2], a[4 * g + 3], w);
      else
         ep.template pack4<M, 4>(prm, 0, a[4 * g + 0], a[4 * g + 1], a[4 * g + 2], a[4 * g + 3], w);
   };
   constexpr std::integral_constant<int, MODE> mode_c{};
   if constexpr (ESZ == 4) {
      static_for<NT>([&](auto cj) {
         constexpr int j = decltype(cj)::value;
         static_for<G>([&](auto cg) {
            constexpr int g = decltype(cg)::value;
            constexpr int cb = j * R + g * 4 * LK;
            const int c0 = cb + lk * 4;
            typename EPI::template col_params<4> prm;
            column_constants(cb, prm);
            static_for<MT>([&](auto ci) {
               constexpr int i = decltype(ci)::value;
               uint32_t w[4];
               convert4(mode_c, prm, acc[i][j], g, w);
               typedef unsigned int u4 __attribute__((ext_vector_type(4)));
               const u4 v = {w[0], w[1], w[2], w[3]};
               __builtin_nontemporal_store(v, (u4 *)(out + ep.out_index_of_plain_rows(m_base + i * R + lr, n_base + c0) * 4));
            });
         });
      });
   } else if constexpr (ESZ == 2) {
      // 2-byte elements, R = 32: a lane's 4 columns of group g are 8 bytes at column g*8 + lk*4 of the 32-column block.  First
      // the two lanes of a row swap so that lane lk holds the 8 columns (16 bytes) of group 2p + lk, for p = 0 and p = 1: the
      // four 16-byte chunks of the block's 64-byte row segment, two per lane.  Then the lanes of rows 0..15 and of rows 16..31
      // swap chunks, so that one register holds all four chunks of rows 0..15 and the other those of rows 16..31: a wave
      // instruction writes whole 64-byte segments (stored pairwise instead, every segment would be written as two halves).
      static_assert(R == 32 && G == 4, "2-byte outputs are exchanged between the two lanes of a row of the 32 x 32 block");
      const int q16 = lane >> 4;
      const int chunk = ((q16 & 1) << 1) | (q16 >> 1); // which chunk a lane ends up with: lanes 0-15: 0, 16-31: 2, 32-47: 1, 48-63: 3
      static_for<NT>([&](auto cj) {
         constexpr int j = decltype(cj)::value;
         typename EPI::template col_params<4> prm[4];
         static_for<4>([&](auto cg) { column_constants(j * R + decltype(cg)::value * 4 * LK, prm[decltype(cg)::value]); });
         static_for<MT>([&](auto ci) {
            constexpr int i = decltype(ci)::value;
            uint32_t lo[4], hi[4]; // the 16 bytes of group lk (lo) and of group 2 + lk (hi)
            static_for<2>([&](auto cp) {
               constexpr int ge = decltype(cp)::value * 2, go = ge + 1;
               uint32_t we[2], wo[2];
               convert4(mode_c, prm[ge], acc[i][j], ge, we);
               convert4(mode_c, prm[go], acc[i][j], go, wo);
               // swap(a, b): a keeps its lower 32 lanes and receives b's lower 32 lanes in its upper half; b the other way round
               auto s0 = __builtin_amdgcn_permlane32_swap(we[0], wo[0], false, false);
               auto s1 = __builtin_amdgcn_permlane32_swap(we[1], wo[1], false, false);
               uint32_t *dst = decltype(cp)::value ? hi : lo;
               dst[0] = s0[0], dst[1] = s1[0], dst[2] = s0[1], dst[3] = s1[1];
            });
            uint32_t top[4], bot[4];
#pragma unroll
            for (int d = 0; d < 4; ++d) {
               // swap(a, b) of 16-lane rows: a = {a.row0, b.row0, a.row2, b.row2}, b = {a.row1, b.row1, a.row3, b.row3}
               auto t = __builtin_amdgcn_permlane16_swap(lo[d], hi[d], false, false);
               top[d] = t[0];
               bot[d] = t[1];
            }
            const int n = n_base + j * R + chunk * 8;
            // (streamed like the 1-byte tiles below: FP8 4096^3 -3.8 %, 8192^3 -1 %)
            typedef unsigned int u4 __attribute__((ext_vector_type(4)));
            const u4 vt = {top[0], top[1], top[2], top[3]}, vb = {bot[0], bot[1], bot[2], bot[3]};
            __builtin_nontemporal_store(vt, (u4 *)(out + ep.out_index_of_plain_rows(m_base + i * R + (lane & 15), n) * 2));
            __builtin_nontemporal_store(vb, (u4 *)(out + ep.out_index_of_plain_rows(m_base + i * R + 16 + (lane & 15), n) * 2));
         });
      });
   } else {
      static_assert(ESZ == 1 && R == 16 && NT == 4 && G == 1, "1-byte outputs are exchanged as a 4 x 4 matrix of dwords between the four lanes of a row");
      // IB row blocks at a time (the column constants are permuted again for each group of blocks: few registers live at once;
      // four at a time against two: -1.8 % on the int8 CNN, eight: no further gain)
      constexpr int IB = 4;
      static_assert(MT % IB == 0, "row blocks per wave");
      static_for<MT / IB>([&](auto cb) {
         constexpr int i0 = decltype(cb)::value * IB;
         uint32_t w[IB][NT];
         static_for<NT>([&](auto cj) {
            constexpr int j = decltype(cj)::value;
            typename EPI::template col_params<4> prm;
            column_constants(j * R, prm);
            static_for<IB>([&](auto ci) {
               constexpr int i = decltype(ci)::value;
               ep.template pack4_short<MODE, 4, EPI::kBiasInAccumulator>(prm, 0, acc[i0 + i][j][0], acc[i0 + i][j][1], acc[i0 + i][j][2], acc[i0 + i][j][3], &w[i][j]);
            });
         });
         static_for<IB>([&](auto ci) {
            constexpr int i = decltype(ci)::value;
            // (lane lk, register j) <-> (lane j, register lk): first the high bits (rows 2,3 of 16 lanes <-> registers 2,3), then the low ones
            auto s02 = __builtin_amdgcn_permlane32_swap(w[i][0], w[i][2], false, false);
            auto s13 = __builtin_amdgcn_permlane32_swap(w[i][1], w[i][3], false, false);
            auto t01 = __builtin_amdgcn_permlane16_swap(s02[0], s13[0], false, false);
            auto t23 = __builtin_amdgcn_permlane16_swap(s02[1], s13[1], false, false);
            {
               // streamed past the caches' retention (the tile is not read again by this launch; the weights and the
               // neighbouring pixels, which are, keep their lines): -0.8 % on the int8 CNN
               typedef unsigned int u4 __attribute__((ext_vector_type(4)));
               const u4 v = {t01[0], t01[1], t23[0], t23[1]};
               __builtin_nontemporal_store(v, (u4 *)(out + ep.out_index_of_plain_rows(m_base + (i0 + i) * R + lr, n_base + lk * 16)));
            }
         });
      });
   }
}

// The plane sums of a convolution that feeds a global average pool, from the accumulator registers: the int8 results of the
// wave tile's rows (all in one plane) are added up per column instead of stored.  A lane adds its row blocks in registers
// (the converted words as they are, two per addition; their common offset leaves once per sum), the R = 16 lanes that share
// columns, one row of the data-parallel-primitive network, combine in four additions that read a neighbour's register
// (pairs, quads, the mirrored half row, the mirrored row), and one lane per group of 4 columns adds the sums to memory.
template <int MODE, class MMA, int MT, int NT, class EPI, class ACC>
__device__ __forceinline__ void tile_sum_from_registers(const EPI &ep, ACC (&acc)[MT][NT], int m_base, int n_base, int lane,
                                                        const uint32_t (&col_words)[EPI::kColWords])
{
   constexpr int R = MMA::ROWS, LK = MMA::LK, G = MMA::ACC / 4;
   static_assert(NT * R == 64, "one column constant per lane");
   static_assert(R == 16 && MT % 2 == 0, "the lanes of a 16-lane row share columns; row blocks are added in pairs");
   const int lr = lane % R, lk = lane / R;
   int first_col_addr = lk * 16;
   asm volatile("" : "+v"(first_col_addr));
   static_for<NT>([&](auto cj) {
      constexpr int j = decltype(cj)::value;
      static_for<G>([&](auto cg) {
         constexpr int g = decltype(cg)::value;
         constexpr int cb = j * R + g * 4 * LK;
         typename EPI::template col_params<4> prm;
#pragma unroll
         for (int v = 0; v < 4; ++v) {
            uint32_t w[EPI::kColWords];
#pragma unroll
            for (int k = 0; k < EPI::kColWords; ++k)
               w[k] = (EPI::kBiasInAccumulator && k == EPI::kBiasWord) ? 0u : (uint32_t)__builtin_amdgcn_ds_bpermute(first_col_addr + (cb + v) * 4, (int)col_words[k]);
            EPI::template set_column<4>(prm, v, w);
         }
         uint32_t sum[4] = {0, 0, 0, 0};
         static_for<MT / 2>([&](auto ci) {
            constexpr int i = 2 * decltype(ci)::value;
            uint32_t q0[4], q1[4];
            ep.template quantize4_biased<MODE, 4, EPI::kBiasInAccumulator>(prm, 0, acc[i][j][4 * g + 0], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3], q0);
            ep.template quantize4_biased<MODE, 4, EPI::kBiasInAccumulator>(prm, 0, acc[i + 1][j][4 * g + 0], acc[i + 1][j][4 * g + 1], acc[i + 1][j][4 * g + 2],
                                                                           acc[i + 1][j][4 * g + 3], q1);
#pragma unroll
            for (int v = 0; v < 4; ++v)
               sum[v] = sum[v] + q0[v] + q1[v];
         });
         int total[4];
#pragma unroll
         for (int v = 0; v < 4; ++v) {
            int t = (int)(sum[v] - (uint32_t)MT * EPI::kI8BitsBias);
            t += __builtin_amdgcn_update_dpp(0, t, 0xB1, 0xf, 0xf, false);  // quad_perm [1,0,3,2]: lane ^ 1
            t += __builtin_amdgcn_update_dpp(0, t, 0x4E, 0xf, 0xf, false);  // quad_perm [2,3,0,1]: lane ^ 2
            t += __builtin_amdgcn_update_dpp(0, t, 0x141, 0xf, 0xf, false); // row_half_mirror: the other quad of the half row
            t += __builtin_amdgcn_update_dpp(0, t, 0x140, 0xf, 0xf, false); // row_mirror: the other half row
            total[v] = t;
         }
         if (lr == 0)
            ep.add_row_sums(m_base, n_base + cb + lk * 4, ep.N, total);
      });
   });
}

template <int MODE, class MMA, int MT, int NT, class EPI, class ACC>
__device__ __forceinline__ void tile_store_or_sum_from_registers(const EPI &ep, ACC (&acc)[MT][NT], int m_base, int n_base, int lane,
                                                                 const uint32_t (&col_words)[EPI::kColWords])
{
   if constexpr (epi_can_sum_rows<EPI>::value && EPI::template out_bytes<MODE>() == 1) {
      if (ep.sums_rows()) {
         tile_sum_from_registers<MODE, MMA, MT, NT>(ep, acc, m_base, n_base, lane, col_words);
         return;
      }
   }
   tile_store_from_registers<MODE, MMA, MT, NT>(ep, acc, m_base, n_base, lane, col_words);
}

// The A operand of the persistent kernel.  A lane issues two load instructions per slab of A (tile rows row[0], row[1], the
// 16 bytes at slab offset cbyte[i]).  The source keeps what it needs per TILE in a tile_state (the kernel holds two: the
// tile being loaded and the one after it) and turns (state, instruction, reduction offset of the slab) into an address.
struct PersistPlainRows {
   static constexpr bool kConv = false;
   const int8_t *A;
   int lda;
   struct lane_state {
      uint32_t off[2];
   };
   struct tile_state {
      const int8_t *origin; // uniform
   };
   __device__ __forceinline__ void init_lane(lane_state &ls, int i, int row, int cbyte) const
   {
      ls.off[i] = (uint32_t)row * (uint32_t)lda + (uint32_t)cbyte;
   }
   __device__ __forceinline__ void tile(tile_state &ts, const lane_state &, int m0) const { ts.origin = A + (size_t)m0 * (size_t)lda; }
   static __device__ __forceinline__ void take(tile_state &dst, const tile_state &src, bool yes) { dst.origin = yes ? src.origin : dst.origin; }
   __device__ __forceinline__ const int8_t *src(const lane_state &ls, const tile_state &ts, int i, int kbyte) const
   {
      return (ts.origin + kbyte) + ls.off[i]; // uniform base (scalar registers) + 32-bit lane offset
   }
};

// Rows of a convolution read straight from the NHWC activations (the addressing of ConvRows): GEMM row m is the output
// pixel (n, oh, ow), a 64-byte slab is 64 consecutive channels of one input pixel of one filter tap, and a tap that falls
// outside the image reads the zero page.  Per tile a lane keeps the offsets of its two pixels and one bit per (pixel, tap).
struct PersistConvRows {
   static constexpr bool kConv = true;
   ConvRows g;
   // log2(OW) when a tile is whole output rows of one image (OW a power of two that divides 256, planes of whole tiles), else
   // -1.  A tile's image and first output row are then the same for all lanes (scalar arithmetic, once), and a lane's pixel is
   // a fixed number of rows and columns from there: no division per lane and tile.
   int ow_shift;
   struct lane_state {
      int row[2], swz[2]; // swz: the chunk of the 64-byte slab row this lane supplies
   };
   struct tile_state {
      int32_t off[2];
      uint32_t mask; // bit 16*i + t: tap t of pixel i lies inside the image (at most 16 taps)
   };
   __device__ __forceinline__ void init_lane(lane_state &ls, int i, int row, int cbyte) const
   {
      ls.row[i] = row;
      ls.swz[i] = cbyte;
   }
   __device__ __forceinline__ void tile(tile_state &ts, const lane_state &ls, int m0) const
   {
      if (ow_shift >= 0) {
         const int ohw = g.OH * g.OW;
         const int m0u = __builtin_amdgcn_readfirstlane(m0);
         const int n = g.ohw_mul ? (int)__umul64hi((unsigned long long)(unsigned)m0u, g.ohw_mul) : m0u;
         const int oh0 = (m0u - n * ohw) >> ow_shift;
         uint32_t mask = 0;
#pragma unroll
         for (int i = 0; i < 2; ++i) {
            const int oh = oh0 + (ls.row[i] >> ow_shift), ow = ls.row[i] & (g.OW - 1);
            const int ih0 = oh * g.stride_h - g.pad_h0, iw0 = ow * g.stride_w - g.pad_w0;
            ts.off[i] = ((n * g.H + ih0) * g.W + iw0) * g.C + ls.swz[i];
            uint32_t cols = 0, mk = 0;
            for (int kwi = 0, iw = iw0; kwi < g.kw; ++kwi, iw += g.dil_w)
               cols |= ((unsigned)iw < (unsigned)g.W ? 1u : 0u) << kwi;
            for (int t0 = 0, ih = ih0; t0 < g.ntaps; t0 += g.kw, ih += g.dil_h)
               mk |= ((unsigned)ih < (unsigned)g.H ? cols : 0u) << t0;
            mask |= mk << (16 * i);
         }
         ts.mask = mask;
         return;
      }
      ConvRows::lane_state<2> st;
      g.template init<2>(st, 0, m0, ls.row[0], ls.swz[0], 0x7fffffff);
      g.template init<2>(st, 1, m0, ls.row[1], ls.swz[1], 0x7fffffff);
      ts.off[0] = st.off[0];
      ts.off[1] = st.off[1];
      ts.mask = st.mask[0] | (st.mask[1] << 16);
   }
   static __device__ __forceinline__ void take(tile_state &dst, const tile_state &src, bool yes)
   {
      dst.off[0] = yes ? src.off[0] : dst.off[0];
      dst.off[1] = yes ? src.off[1] : dst.off[1];
      dst.mask = yes ? src.mask : dst.mask;
   }
   __device__ __forceinline__ const int8_t *src(const lane_state &, const tile_state &ts, int i, int kbyte) const
   {
      const int tap = kbyte >> g.cg_shift; // uniform
      const int cb = kbyte & ((1 << g.cg_shift) - 1);
      const int khi = (tap * g.kw_recip) >> 16, kwi = tap - khi * g.kw;
      const int toff = (khi * g.dil_h * g.W + kwi * g.dil_w) * g.C + cb;
      const int8_t *p = g.X + (ptrdiff_t)(ts.off[i] + toff);
      return ((ts.mask >> (16 * i + tap)) & 1u) ? p : (const int8_t *)conv_zero_page;
   }
};

template <class MMA, class EPI, class ASRC>
__global__ __launch_bounds__(512) void mfma8_gemm_persist_kernel(ASRC A, const int8_t *__restrict__ Bt, int ldb, int M, int N, int K, EPI ep,
                                                                  int tiles_m, int tiles_n, int sw)
{
   constexpr int BM = 256, BN = 256, BK = 64, STAGES = 5, NW = 8, WAVES_N = 4;
   constexpr int R = MMA::ROWS;
   constexpr int TM = 128, TN = 64, MT = TM / R, NT = TN / R;
   constexpr int LD = BM / 16 / NW;            // wave instructions per operand and slab (an instruction fills 16 rows of 64 bytes)
   constexpr int STAGE_BYTES = (BM + BN) * BK; // 32 KB
   static_assert(MMA::KSTEP == BK, "one MFMA step per slab");
   static_assert(BM == BN && LD == 2, "the load schedule below is written for 2 + 2 wave instructions per slab");
   typedef typename MMA::acc_t acc_t;
   typedef typename MMA::frag_t frag_t;

   extern __shared__ __attribute__((aligned(16))) int8_t smem[];

   const int t = threadIdx.x;
   const int lane = t & 63;
   const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
   const int wm = wave / WAVES_N, wn = wave % WAVES_N;
   const int lr = lane % R, lk = lane / R;
   const int nwg = gridDim.x, bid = blockIdx.x;
   const int ntiles = tiles_m * tiles_n;
   const int my_tiles = (ntiles - bid + nwg - 1) / nwg;
   const int KP = K / (2 * BK);

   // loader: wave instruction i of an operand fills rows (i*NW + wave)*16 .. +15 of a slab; a lane supplies the chunk that
   // belongs at its position of the swizzled layout (chunk c of row r sits at position c ^ MMA::lds_swizzle(r); the swizzle has
   // period 16 in r, so a fragment's rows r = 16*k + lr swizzle like lr)
   typename ASRC::lane_state a_lane;
   uint32_t b_off[LD];
   auto init_a_lane = [&](typename ASRC::lane_state &ls, int ln) {
#pragma unroll
      for (int i = 0; i < LD; ++i) {
         const int row = (i * NW + wave) * 16 + ln / 4;
         A.init_lane(ls, i, row, ((ln % 4) ^ MMA::lds_swizzle(row)) * 16);
      }
   };
   init_a_lane(a_lane, lane);
#pragma unroll
   for (int i = 0; i < LD; ++i) {
      const int row = (i * NW + wave) * 16 + lane / 4;
      const int c = (lane % 4) ^ MMA::lds_swizzle(row);
      b_off[i] = (uint32_t)row * (uint32_t)ldb + (uint32_t)c * 16u;
   }
   // The loads run two pairs ahead of the MFMAs and cross into the next tile of the list before the current one is stored.
   // l_a, l_b: the tile being loaded; n_a, n_b: the one after it, worked out once per tile (in the tile store, which needs
   // the tile order anyway) so that the step itself has no branch.  Past the end of the list the loads start over on the
   // last tile: filler that keeps the count of loads in flight constant; nobody reads it.
   auto tile_origin = [&](int it, int &m0, int &n0) {
      int tm, tn;
      tile_of_block((it < my_tiles ? it : my_tiles - 1) * nwg + bid, ntiles, tiles_m, tiles_n, sw, tm, tn);
      // Sizes that are not multiples of the tile: the last tile of a row or column of tiles is moved back until it ends at
      // the edge.  It then overlaps its neighbour, and both compute (and store) the rows or columns they share: the same
      // values twice, instead of loads and stores that would have to be predicated lane by lane.
      m0 = min(tm * BM, M - BM);
      n0 = min(tn * BN, N - BN);
   };
   auto load_origin = [&](int m0, int n0, typename ASRC::tile_state &ta, const int8_t *&pb) {
      if constexpr (ASRC::kConv) {
         // what the source keeps per lane is only needed here, once per tile: worked out again from the lane number (made
         // opaque, so that it is not kept in registers across the K loop instead)
         int ln = lane;
         asm volatile("" : "+v"(ln));
         typename ASRC::lane_state ls;
         init_a_lane(ls, ln);
         A.tile(ta, ls, m0);
      } else {
         A.tile(ta, a_lane, m0);
      }
      pb = Bt + (size_t)n0 * (size_t)ldb;
   };
   int l_kp = 0; // pair (of the tile being loaded) the next loads fetch
   typename ASRC::tile_state l_a, n_a;
   const int8_t *l_b, *n_b;
   // origins of the tile in work and of the one after it (the tile order costs a few integer divisions: once per tile)
   int m_cur, n_cur, m_nxt, n_nxt;
   tile_origin(0, m_cur, n_cur);
   tile_origin(1, m_nxt, n_nxt);
   load_origin(m_cur, n_cur, l_a, l_b);
   load_origin(m_nxt, n_nxt, n_a, n_b);
   // load q (0..7) of the pair: operand q/4, wave instruction (q/2)%2, half q%2 of the 128-byte line
   auto issue_load = [&](int slot0, int slot1, auto q_c) {
      constexpr int q = decltype(q_c)::value;
      constexpr int opnd = q / 4, i = (q / 2) % 2, half = q % 2;
      int8_t *dst = smem + (half ? slot1 : slot0) * STAGE_BYTES + opnd * (BM * BK) + (i * NW + wave) * 1024;
      // (The instruction's own offset field cannot supply the second half of the line: it is added to the LDS address as well.)
      const int kbyte = l_kp * (2 * BK) + half * BK;
      const int8_t *src;
      if constexpr (opnd == 0)
         src = A.src(a_lane, l_a, i, kbyte);
      else
         src = (l_b + kbyte) + b_off[i]; // uniform base (scalar registers) + 32-bit lane offset
      __builtin_amdgcn_global_load_lds((global_void_t *)src, (lds_void_t *)dst, 16, 0, 0);
   };
   auto advance_loader = [&]() {
      const bool wrap = (l_kp + 1 == KP);
      l_kp = wrap ? 0 : l_kp + 1;
      ASRC::take(l_a, n_a, wrap);
      l_b = wrap ? n_b : l_b;
   };

   const int a_frag = (wm * TM + lr) * BK, b_frag = BM * BK + (wn * TN + lr) * BK;
   auto read_frags = [&](int slot, frag_t(&fa)[MT], frag_t(&fb)[NT]) {
      const int8_t *base = smem + slot * STAGE_BYTES;
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
         for (int c = 0; c < MMA::CHUNKS; ++c)
            fb[j].c[c] = *(const v4i *)(base + b_frag + j * R * BK + (((lk * MMA::CHUNKS + c) ^ MMA::lds_swizzle(lr)) << 4));
#pragma unroll
      for (int i = 0; i < MT; ++i)
#pragma unroll
         for (int c = 0; c < MMA::CHUNKS; ++c)
            fa[i].c[c] = *(const v4i *)(base + a_frag + i * R * BK + (((lk * MMA::CHUNKS + c) ^ MMA::lds_swizzle(lr)) << 4));
   };

   // The epilogue's constants of column n0 + wn*TN + lane: col_words for the tile in work, col_next for the one after it
   // (fetched a whole tile ahead: an integer epilogue starts the next tile's accumulators at its bias, straight after the
   // store of this one, and must not wait for memory there).
   uint32_t col_words[EPI::kColWords], col_next[EPI::kColWords];
   ep.load_column_for_registers(n_cur + wn * TN + lane, col_words);
   ep.load_column_for_registers(n_nxt + wn * TN + lane, col_next);
   acc_t acc[MT][NT];
   // accumulators of a new tile: zero, or (EPI::kBiasInAccumulator: exact integer sums, whatever the order) the bias of the
   // lane's columns, which then costs the store nothing
   auto start_acc = [&](const uint32_t (&cw)[EPI::kColWords]) {
      if constexpr (EPI::kBiasInAccumulator) {
         static_assert(MMA::ACC == 4 && NT * R == 64, "one bias per lane and column: a lane's columns are j*R + lk*4 + v");
         int first_col_addr = lk * 16;
         asm volatile("" : "+v"(first_col_addr));
         static_for<NT>([&](auto cj) {
            constexpr int j = decltype(cj)::value;
            acc_t b;
#pragma unroll
            for (int v = 0; v < 4; ++v)
               b[v] = __builtin_amdgcn_ds_bpermute(first_col_addr + (j * R + v) * 4, (int)cw[EPI::kBiasWord]);
#pragma unroll
            for (int i = 0; i < MT; ++i)
               acc[i][j] = b;
         });
      } else {
#pragma unroll
         for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < NT; ++j)
#pragma unroll
               for (int v = 0; v < MMA::ACC; ++v)
                  acc[i][j][v] = 0;
      }
   };
   if constexpr (EPI::kBiasInAccumulator)
      wait_vmcnt<0>(); // the first tile's constants
   start_acc(col_words);

   // prologue: pairs 0 and 1 into slots 0..3
   static_for<8>([&](auto q) { issue_load(0, 1, q); });
   advance_loader();
   static_for<8>([&](auto q) { issue_load(2, 3, q); });
   advance_loader();
   frag_t fa[2][MT], fb[2][NT];
   wait_vmcnt<8>();
   __builtin_amdgcn_s_barrier();
   read_frags(0, fa[0], fb[0]);

   int rslot = 1; // slot of the slab whose fragments are read during the current step
   int lslot = 4; // slot of the first slab of the pair requested during the current (even) step
   constexpr int NMFMA = MT * NT, NREAD = (MT + NT) * MMA::CHUNKS;
   static_assert(NMFMA % 8 == 0 && NREAD <= 16 && NREAD >= 8, "issue pattern below: 8 groups per step");
   // The MFMAs of a step walk the wave tile's blocks in a serpentine, so that one operand changes from one instruction to the
   // next and the other stays (measured in register-only loops on random operands: 4.16 POP/s against 4.07 for a plain
   // double loop and 3.93 when both change every time).  Which index runs outside is the instruction's matter
   // (MMA::kColumnsOutside): measured in this kernel, -1.0 % for int8 with the columns outside, -0.5 % for FP8 with the rows.
   auto mfmas = [&](auto odd_c) {
      constexpr int odd = decltype(odd_c)::value;
      if constexpr (MMA::kColumnsOutside) {
         static_for<NT>([&](auto cj) {
            constexpr int j = decltype(cj)::value;
            static_for<MT>([&](auto ci) {
               constexpr int i = (j & 1) ? MT - 1 - decltype(ci)::value : decltype(ci)::value;
               acc[i][j] = MMA::mma(fb[odd][j], fa[odd][i], acc[i][j]);
            });
         });
      } else {
         static_for<MT>([&](auto ci) {
            constexpr int i = decltype(ci)::value;
            static_for<NT>([&](auto cj) {
               constexpr int j = (i & 1) ? NT - 1 - decltype(cj)::value : decltype(cj)::value;
               acc[i][j] = MMA::mma(fb[odd][j], fa[odd][i], acc[i][j]);
            });
         });
      }
   };
   // One step: multiplies the slab whose fragments are in fa[ODD], fb[ODD] while the next slab's fragments are read into
   // the other buffer and four loads of the pair two pairs ahead are issued (even step: its A rows, odd step: its Bt rows).
   auto step = [&](auto odd_c, int slot0, int slot1) {
      constexpr int odd = decltype(odd_c)::value;
      // (the scheduling fences keep the compiler from mixing the instructions of two steps)
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (odd)
         wait_vmcnt<4>(); // all but the four loads just issued: the pair that starts with the next slab has landed
      __builtin_amdgcn_s_waitcnt(0xc07f); // lgkmcnt(0)
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
      read_frags(rslot, fa[1 - odd], fb[1 - odd]);
      static_for<4>([&](auto q) { issue_load(slot0, slot1, std::integral_constant<int, 4 * odd + decltype(q)::value>{}); });
      if constexpr (odd)
         advance_loader();
      mfmas(odd_c);
      // issue order: the compiler keeps the LDS reads ahead of the loads into LDS (it cannot tell that they touch different
      // slots), so the reads go between the MFMAs of the first half of the step and the loads between those of the second
      static_for<4>([&](auto gc) {
         __builtin_amdgcn_sched_group_barrier(0x008, NMFMA / 8, 0);
         __builtin_amdgcn_sched_group_barrier(0x100, (NREAD + 3) / 4, 0);
      });
      static_for<4>([&](auto gc) {
         __builtin_amdgcn_sched_group_barrier(0x008, NMFMA / 8, 0);
         __builtin_amdgcn_sched_group_barrier(0x010, 1, 0);
      });
      __builtin_amdgcn_sched_barrier(0);
      rslot = (rslot + 1 == STAGES) ? 0 : rslot + 1;
   };
   for (int it = 0; it < my_tiles; ++it) {
      for (int kp = 0; kp < KP; ++kp) {
         const int lslot1 = (lslot + 1 == STAGES) ? 0 : lslot + 1;
         step(std::integral_constant<int, 0>{}, lslot, lslot1);
         step(std::integral_constant<int, 1>{}, lslot, lslot1);
         lslot = (lslot + 2 >= STAGES) ? lslot + 2 - STAGES : lslot + 2;
      }
      ep.dispatch_for_registers([&](auto mode) {
         tile_store_or_sum_from_registers<decltype(mode)::value, MMA, MT, NT>(ep, acc, m_cur + wm * TM, n_cur + wn * TN, lane, col_words);
      });
      start_acc(col_next);
      // The loads have moved on to tile it + 1 (K spans at least three pairs): the tile after that is it + 2.  Its lane
      // state is worked out here, behind the stores, whose acknowledgements are still on their way.
      int m2, n2;
      tile_origin(it + 2, m2, n2);
      load_origin(m2, n2, n_a, n_b);
      // the column constants of the tile after the next: fetched now, used from the end of the next tile's K loop on
#pragma unroll
      for (int k = 0; k < EPI::kColWords; ++k)
         col_words[k] = col_next[k];
      ep.load_column_for_registers(n2 + wn * TN + lane, col_next);
      m_cur = m_nxt, n_cur = n_nxt;
      m_nxt = m2, n_nxt = n2;
   }
   wait_vmcnt<0>();
}

// Whether the persistent kernel takes this product: at least one whole 256 x 256 tile in each direction (a last tile that
// does not fit is moved back to end at the edge, see tile_origin in the kernel), K a multiple of 128, 16-byte aligned rows.
// `n_align` = elements per 16 bytes of output: the moved tile must start on a 16-byte boundary of the output rows.
inline bool mfma8_persist_applies(const int8_t *A, const int8_t *Bt, int M, int N, int K, int lda, int ldb, int n_align)
{
   return M >= 256 && N >= 256 && N % n_align == 0 && K >= 384 && K % 128 == 0 && lda % 16 == 0 && ldb % 16 == 0 &&
          (((uintptr_t)A | (uintptr_t)Bt) & 15) == 0 && (long long)((M + 255) / 256) * ((N + 255) / 256) <= 0x7fffffLL &&
          (size_t)256 * (size_t)(lda > ldb ? lda : ldb) < 0xffffffffULL;
}
// The same for a convolution read through ConvRows (whose own conditions the caller has checked: channels per group a power
// of two >= 64, 32-bit offsets): one bit per tap and pixel must fit the lane's mask.  `whole_tiles`: the store adds results up
// (plane sums), so no output may be computed twice.
inline bool mfma8_persist_conv_applies(const ConvRows &a, const int8_t *Wp, int M, int N, int K, int n_align, bool whole_tiles)
{
   return M >= 256 && N >= 256 && N % n_align == 0 && (!whole_tiles || (M % 256 == 0 && N % 256 == 0)) && K >= 384 && K % 128 == 0 && a.ntaps <= 16 &&
          (((uintptr_t)a.X | (uintptr_t)Wp) & 15) == 0 && (long long)((M + 255) / 256) * ((N + 255) / 256) <= 0x7fffffLL &&
          (size_t)256 * (size_t)K < 0xffffffffULL;
}

inline int cu_count_of_current_device(int &ncu)
{
   static int cus[64] = {};
   int dev = 0;
   SOFIE_HIP_CHECK(hipGetDevice(&dev));
   ncu = (dev >= 0 && dev < 64) ? cus[dev] : 0;
   if (ncu == 0) {
      SOFIE_HIP_CHECK(hipDeviceGetAttribute(&ncu, hipDeviceAttributeMultiprocessorCount, dev));
      if (dev >= 0 && dev < 64)
         cus[dev] = ncu;
   }
   return SOFIE_HIP_OK;
}

template <class MMA, class EPI, class ASRC>
static int launch_mfma8_persist_src(const LaunchCfg &lc, const ASRC &a, const int8_t *Bt, int M, int N, int K, int ldb, const EPI &ep)
{
   const int tiles_m = (M + 255) / 256, tiles_n = (N + 255) / 256;
   const int ntiles = tiles_m * tiles_n;
   constexpr size_t smem = (size_t)5 * 512 * 64;
   static_assert(smem <= 160 * 1024, "LDS ring larger than the CU's LDS");
   auto kern = mfma8_gemm_persist_kernel<MMA, EPI, ASRC>;
   static bool configured[64] = {};
   if (int st = configure_lds_once(kern, smem, configured))
      return st;
   int ncu = 0;
   if (int st = cu_count_of_current_device(ncu))
      return st;
   const int grid = ntiles < ncu ? ntiles : ncu;
   hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(512), smem, lc.stream, a, Bt, ldb, M, N, K, ep, tiles_m, tiles_n, lc.swizzle);
   return launch_status("mfma8_gemm_persist_kernel");
}

inline PersistConvRows persist_conv_rows(const ConvRows &a)
{
   PersistConvRows p;
   p.g = a;
   p.ow_shift = -1;
   if (a.OW >= 1 && a.OW <= 256 && (a.OW & (a.OW - 1)) == 0 && (a.OH * a.OW) % 256 == 0)
      for (int sh = 0; sh <= 8; ++sh)
         if ((1 << sh) == a.OW)
            p.ow_shift = sh;
   return p;
}

template <class MMA, class EPI>
static int launch_mfma8_persist(const LaunchCfg &lc, const int8_t *A, const int8_t *Bt, int M, int N, int K, int lda, int ldb, const EPI &ep)
{
   return launch_mfma8_persist_src<MMA, EPI, PersistPlainRows>(lc, PersistPlainRows{A, lda}, Bt, M, N, K, ldb, ep);
}

} // namespace sofie_hip
