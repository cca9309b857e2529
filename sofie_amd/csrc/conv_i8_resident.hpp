// int8 convolution of a SMALL layer (64 input channels per group, 128 output channels, 3 x 3, stride 1): the weights stay in
// LDS for the whole launch and every tile's input pixels are fetched once, with their halo, instead of once per filter tap.
//
// As an implicit GEMM such a layer has a reduction of only 9 slabs, and the slab-by-slab kernels spend as long at a tile's
// edges (prologue, one barrier per slab, the conversion of the accumulators, which no MFMA overlaps) as in its K loop.  Here
//   * the packed weights [128][576] are loaded once per workgroup into LDS (rows padded to 608 bytes);
//   * a tile is 256 consecutive output pixels of one image = 256 / OW whole output rows; its input patch, (256 / OW + 2) rows
//     of OW + 2 pixels of 64 channels (zeros outside the image), is loaded with global_load_lds into one of two buffers while
//     the tile before it is multiplied: the only loads of the loop, 9 times fewer bytes than tap-by-tap gathering;
//   * the A fragment of tap (ky, kx) is read from the patch at a tap offset, the B fragment from the resident weights: no
//     barrier inside a tile.  The eight waves meet once per tile;
//   * pixels and weight rows are 64 + 32 (576 + 32) bytes apart in LDS: records 96 bytes (mod 256) apart are read by
//     ds_read_b128 at the full rate from any starting record (measured: 237 B/clk; 80, 112, 144 or 592 bytes apart: 123), so no
//     swizzle is needed and every fragment address is a lane constant plus a uniform offset;
//   * a wave's 64 x 64 tile is worked in two halves of 64 x 32, each over all nine taps: 32 accumulators per half, so TWO
//     halves fit the registers, and the half finished last is converted and stored between the MFMAs of the half in work,
//     one output element (four vector instructions) per pair of MFMAs.  The MFMAs run through the halves and through the
//     tile boundaries: during the last tap of a half the first fragments of the next one are read.
// Workgroup = 8 waves (4 x 2), v_mfma_i32_16x16x64_i8, store from registers.
//
// What bounds it (batch 256 of 64 x 64 images, 67 us against 33 us of MFMA at the clock it runs at): the matrix cores, the LDS
// reads of the fragments and the vector instructions of the conversion each need about half of the launch and do not overlap
// freely.  Measured: the loop without store and conversion 57 us; with one MFMA in eight 48 us; neither 31 us (864 KB of
// fragment reads per tile and CU, 208 B/clk: near the LDS's rate); a wave of vector instructions beside a wave of MFMAs on one
// SIMD runs at 61 % of its own rate and does not slow the MFMAs.  The HBM traffic (134 MB written, 100 MB read) is not the
// bound: the same time with every tile stored to one place.  Wave tiles of 64 x 64 as ONE piece (one set of accumulators, the
// store of one wave of each SIMD delayed behind the next barrier so that it runs under the other's MFMAs) read a third fewer
// fragments and take 69 - 70 us; sixteen waves of 32 x 64 take 72 us.
#pragma once
#include "mfma8_gemm_persist.hpp"

namespace sofie_hip {

struct ResidentConv {
   const int8_t *X; // NHWC, first channel of the group
   int H, W, C;     // C = channel stride of a pixel (all groups)
   int OH, OW, pad_h0, pad_w0;
   int ow_shift;    // log2(OW)
   int tiles_per_image;
};

template <int KH, int KW, class EPI>
__global__ __launch_bounds__(512) void conv_i8_resident_kernel(ResidentConv g, const int8_t *__restrict__ Wp, EPI ep, int ntiles)
{
   typedef MfmaI8x16 MMA;
   constexpr int R = 16, TM = 64, TN = 64, MT = TM / R, NT = TN / R, NW = 8, BN = 128;
   constexpr int NTAPS = KH * KW, K = NTAPS * 64;
   constexpr int WROW = K + 32, WCHUNKS = WROW / 16;       // a weight row in LDS, in bytes and in 16-byte chunks
   constexpr int WBYTES = ((BN * WROW + 1023) / 1024 + 1) * 1024; // the loads write whole kilobytes: room for the last one
   constexpr int PIX = 96, PCH = PIX / 16;                // a patch pixel in LDS: 64 channels + 32 bytes
   constexpr int PLD = 5;                                 // load instructions per wave and patch
   constexpr int PBYTES = PLD * NW * 1024;                // 40 KB per patch buffer
   typedef MMA::acc_t acc_t;
   typedef MMA::frag_t frag_t;
   extern __shared__ __attribute__((aligned(16))) int8_t smem[];
   int8_t *const wl = smem, *const patch = smem + WBYTES;

   const int t = threadIdx.x;
   const int lane = t & 63;
   const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
   const int wm = wave >> 1, wn = wave & 1;
   const int lr = lane % R, lk = lane / R;
   const int nwg = gridDim.x, bid = blockIdx.x;
   const int my_tiles = (ntiles - bid + nwg - 1) / nwg;
   const int rows_per_tile = 256 >> g.ow_shift;
   const int PW = g.OW + KW - 1, PP = (rows_per_tile + KH - 1) * PW; // patch width and pixels

   // ---- the weights, once: LDS chunk q holds chunk q % WCHUNKS of row q / WCHUNKS (the last two chunks of a row are padding)
   for (int j = 0; (j * NW + wave) * 64 < BN * WCHUNKS; ++j) {
      const int q = (j * NW + wave) * 64 + lane;
      const int row = q / WCHUNKS, c = q - row * WCHUNKS;
      const int8_t *src = (row < BN && c < K / 16) ? Wp + (size_t)row * K + c * 16 : (const int8_t *)conv_zero_page;
      __builtin_amdgcn_global_load_lds((global_void_t *)src, (lds_void_t *)(wl + (j * NW + wave) * 1024), 16, 0, 0);
   }

   // ---- the patch loader: LDS chunk q of a buffer holds chunk q % 6 of patch pixel q / 6 (chunks 4 and 5 are padding)
   int p_off[PLD];      // byte offset of the lane's chunk from the patch's first pixel (row -pad_h0 of the tile, column -pad_w0)
   int p_row[PLD];      // its patch row, or a large number when the chunk is padding or its column lies outside the image
#pragma unroll
   for (int j = 0; j < PLD; ++j) {
      const int q = (j * NW + wave) * 64 + lane;
      const int p = q / PCH, c = q - p * PCH;
      const int pr = p / PW, pc = p - pr * PW;
      const int iw = pc - g.pad_w0;
      const bool ok = p < PP && c < 4 && (unsigned)iw < (unsigned)g.W;
      p_off[j] = (pr * g.W + iw) * g.C + c * 16;
      p_row[j] = ok ? pr : (1 << 20);
   }
   auto tile_of = [&](int it, int &m0, int &img, int &oh0) {
      const int T = (it < my_tiles ? it : my_tiles - 1) * nwg + bid;
      m0 = T * 256;
      img = T / g.tiles_per_image;
      oh0 = (T - img * g.tiles_per_image) * rows_per_tile;
   };
   auto load_patch = [&](int buf, int img, int oh0) {
      const int ih0 = oh0 - g.pad_h0;
      const int8_t *origin = g.X + ((ptrdiff_t)img * g.H + ih0) * (ptrdiff_t)g.W * g.C; // may lie before X: only added to offsets of valid rows
#pragma unroll
      for (int j = 0; j < PLD; ++j) {
         const bool ok = (unsigned)(ih0 + p_row[j]) < (unsigned)g.H;
         const int8_t *src = ok ? origin + p_off[j] : (const int8_t *)conv_zero_page;
         __builtin_amdgcn_global_load_lds((global_void_t *)src, (lds_void_t *)(patch + buf * PBYTES + (j * NW + wave) * 1024), 16, 0, 0);
      }
   };

   // ---- fragment addresses.  B: a lane constant plus compile-time offsets.  A: one register per (row of taps, row block) holding
   // the LDS byte offset of the lane's chunk at tap (ky, 0) in the patch buffer of the tile in work, so that a fragment read is
   // that register plus a compile-time kx * PIX; the registers move to the other buffer once per tile (one addition each).
   const int b_lane = (wn * TN + lr) * WROW + lk * 16;
   int a_row[KH][MT];
#pragma unroll
   for (int i = 0; i < MT; ++i) {
      const int p = wm * TM + i * R;
      const int blk = ((p >> g.ow_shift) * PW + (p & (g.OW - 1))) * PIX; // first pixel of the wave's i-th block of 16 output pixels, tap (0, 0)
#pragma unroll
      for (int ky = 0; ky < KH; ++ky)
         a_row[ky][i] = WBYTES + blk + ky * PW * PIX + lr * PIX + lk * 16;
   }

   int m_cur, img, oh0;
   tile_of(0, m_cur, img, oh0);
   load_patch(0, img, oh0);
   uint32_t col_words[EPI::kColWords];
   ep.load_column_for_registers(wn * TN + lane, col_words); // one column tile: the constants are the same for every tile
   static_assert(EPI::kBiasInAccumulator && MMA::ACC == 4, "integer epilogue: the accumulators start at the bias");
   char *const out = ep.out_base();
   // The store mode is fixed for the launch: the whole tile loop exists once per mode, so that a tap's MFMAs and the part of the
   // store that goes with them are one straight piece of code.
   ep.dispatch_for_registers([&](auto mode_c) {
      constexpr int MODE = decltype(mode_c)::value;
      constexpr int ESZ = EPI::template out_bytes<MODE>();
      constexpr int HN = NT / 2; // column blocks of a half
      // scale and bias of the lane's columns (4 per column block), once for the launch
      typename EPI::template col_params<4> prm[NT];
      acc_t acc0[NT];
      {
         int first_col_addr = lk * 16;
#pragma unroll
         for (int j = 0; j < NT; ++j)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
               uint32_t w[EPI::kColWords];
#pragma unroll
               for (int k = 0; k < EPI::kColWords; ++k)
                  w[k] = (uint32_t)__builtin_amdgcn_ds_bpermute(first_col_addr + (j * R + v) * 4, (int)col_words[k]);
               acc0[j][v] = (int)w[EPI::kBiasWord];
               w[EPI::kBiasWord] = 0;
               EPI::template set_column<4>(prm[j], v, w);
            }
      }
      // A wave's 64 x 64 tile is worked in two HALVES of 64 x 32 (column blocks 2 h, 2 h + 1), each over all nine taps, into
      // acc[h]: 32 accumulators per half, so that two halves fit the registers and the one finished last is converted and
      // stored, slice by slice, between the MFMAs of the one in work.  (The A fragments are read once per half: half as many
      // LDS reads again.)
      acc_t acc[2][MT][HN];
      uint32_t packed[MT][NT]; // 1-byte modes: the converted dwords of a tile until its second half completes the rows
      // Slice sl (0 .. 8 MT - 1) of the store of half h: one output element of a 1-byte store (convert, scale, clamp,
      // round-and-place: four vector instructions); the second half's last slice of a row block exchanges the dwords between the
      // four lanes of a row (see tile_store_from_registers) and stores 16 bytes per lane.  4-byte outputs convert and store a
      // column block (16 bytes per lane) in every fourth slice.
      auto store_slice = [&](auto h_c, auto slice_c, int m_tile) {
         constexpr int h = decltype(h_c)::value, sl = decltype(slice_c)::value;
         constexpr int i = sl / (4 * HN), jj = (sl / 4) % HN, j = HN * h + jj, v = sl % 4;
         typedef unsigned int u4 __attribute__((ext_vector_type(4)));
         if constexpr (ESZ == 4) {
            if constexpr (v == 3) {
               const int m = m_tile + wm * TM + i * R + lr;
               uint32_t w[4];
               ep.template pack4<MODE, 4, true>(prm[j], 0, acc[h][i][jj][0], acc[h][i][jj][1], acc[h][i][jj][2], acc[h][i][jj][3], w);
               const u4 x = {w[0], w[1], w[2], w[3]};
               __builtin_nontemporal_store(x, (u4 *)(out + ep.out_index_of_plain_rows(m, wn * TN + j * R + lk * 4) * 4));
            }
         } else {
            const float c = ep.template clamp1_short<MODE, true>(acc[h][i][jj][v], 0, prm[j].s[v]);
            EPI::template place_i8_byte<v>(packed[i][j], c);
            if constexpr (h == 1 && jj == HN - 1 && v == 3) {
               const int m = m_tile + wm * TM + i * R + lr;
               auto s02 = __builtin_amdgcn_permlane32_swap(packed[i][0], packed[i][2], false, false);
               auto s13 = __builtin_amdgcn_permlane32_swap(packed[i][1], packed[i][3], false, false);
               auto t01 = __builtin_amdgcn_permlane16_swap(s02[0], s13[0], false, false);
               auto t23 = __builtin_amdgcn_permlane16_swap(s02[1], s13[1], false, false);
               const u4 x = {t01[0], t01[1], t23[0], t23[1]};
               __builtin_nontemporal_store(x, (u4 *)(out + ep.out_index_of_plain_rows(m, wn * TN + lk * 16)));
            }
         }
      };
      constexpr int STORES = ESZ == 4 ? MT * NT : MT; // memory stores of one tile per wave
      constexpr int SLICES = 4 * MT * HN;             // of one half
      constexpr int GROUPS = MT * HN / 2;             // of a tap: two MFMAs each
      constexpr int PER_GROUP = (SLICES + (NTAPS - 1) * GROUPS - 1) / ((NTAPS - 1) * GROUPS); // slices per group, the last tap left free
      // The MFMAs run through the halves and the tile boundaries.  During the last tap of a half the first fragments of the
      // next one are read (of the next tile's patch after the second half).  The workgroup meets once per tile, in front of
      // that last tap of the second half: by then a wave holds the last fragments of this tile's patch in registers and has
      // its own loads of the next patch back, so past the barrier the next patch is complete for everybody and this tile's
      // buffer is free for the patch after the next.
      frag_t fa[2][MT], fb[2][HN]; // fragments of the tap in work and of the one after it; nine taps: the roles swap per half
      auto half_body = [&](auto h_c, auto prev_c, int it) {
         constexpr int h = decltype(h_c)::value;
         constexpr bool prev = decltype(prev_c)::value; // a half before this one is waiting to be stored
         // the half before: the other half of this tile, or the second half of the tile before
         const int m_prev = ((h ? it : it - 1) * nwg + bid) * 256;
         static_for<NTAPS>([&](auto tc) {
            constexpr int tap = decltype(tc)::value;
            constexpr int cur = (tap + h) % 2;
            constexpr bool last = tap + 1 == NTAPS;
            constexpr int ntap = last ? 0 : tap + 1;     // the tap whose fragments are read meanwhile (of the next half after the last one)
            constexpr int nh = last ? 1 - h : h;         // and its half
            constexpr int ky = ntap / KW, kx = ntap % KW;
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (last && h == 1) {
               if (it + 1 < my_tiles) { // (uniform)
                  // a wave's loads of the next patch are older than the stores it has issued since, which may stay in flight
                  wait_vmcnt<STORES>();
                  __builtin_amdgcn_s_waitcnt(0xc07f); // lgkmcnt(0): this tap's fragments
                  __builtin_amdgcn_s_barrier();
                  if (it + 2 < my_tiles) {
                     int m2, img2, oh2;
                     tile_of(it + 2, m2, img2, oh2);
                     load_patch(it & 1, img2, oh2);
                  }
               }
               // from here on the fragments come from the next tile's patch: the other buffer
               const int to_other = (it & 1) ? -PBYTES : PBYTES;
#pragma unroll
               for (int ky2 = 0; ky2 < KH; ++ky2)
#pragma unroll
                  for (int i2 = 0; i2 < MT; ++i2)
                     a_row[ky2][i2] += to_other;
               __builtin_amdgcn_sched_barrier(0);
            }
            // A tap in groups, each fenced so that it is issued as written: two MFMAs and slices of the store of the half
            // before, then two LDS reads of the next tap's fragments (all of them in the first groups, so that the wait in
            // front of the next tap's first MFMA finds them done).  (Left to the scheduler, the store's instructions end up
            // in runs of thirty to fifty between runs of MFMAs.)
            static_for<GROUPS>([&](auto gc) {
               constexpr int grp = decltype(gc)::value;
               static_for<2>([&](auto qc) {
                  constexpr int n = grp * 2 + decltype(qc)::value;
                  constexpr int jj = n / MT, i = (jj & 1) ? MT - 1 - n % MT : n % MT;
                  if constexpr (tap == 0)
                     acc[h][i][jj] = MMA::mma(fb[cur][jj], fa[cur][i], acc0[HN * h + jj]);
                  else
                     acc[h][i][jj] = MMA::mma(fb[cur][jj], fa[cur][i], acc[h][i][jj]);
               });
               if constexpr (prev && !last) {
                  static_for<PER_GROUP>([&](auto sc) {
                     constexpr int sl = (tap * GROUPS + grp) * PER_GROUP + decltype(sc)::value;
                     if constexpr (sl < SLICES)
                        store_slice(std::integral_constant<int, 1 - h>{}, std::integral_constant<int, sl>{}, m_prev);
                  });
               }
               __builtin_amdgcn_sched_barrier(0);
               if constexpr (2 * grp < MT + HN) {
                  static_for<2>([&](auto rc) {
                     constexpr int f = 2 * grp + decltype(rc)::value;
                     if constexpr (f < HN)
                        fb[1 - cur][f].c[0] = *(const v4i *)(wl + b_lane + (HN * nh + f) * R * WROW + ntap * 64);
                     else if constexpr (f < HN + MT)
                        fa[1 - cur][f - HN].c[0] = *(const v4i *)(smem + (a_row[ky][f - HN] + kx * PIX));
                  });
                  __builtin_amdgcn_sched_barrier(0);
               }
            });
         });
      };
      constexpr std::integral_constant<int, 0> h0{};
      constexpr std::integral_constant<int, 1> h1{};
      // the patches of the first two tiles, the first tap of the first half
      {
         int m1, img1, oh1;
         tile_of(1, m1, img1, oh1);
         if (1 < my_tiles)
            load_patch(1, img1, oh1);
         wait_vmcnt<0>();
         __builtin_amdgcn_s_barrier();
#pragma unroll
         for (int f = 0; f < HN; ++f)
            fb[0][f].c[0] = *(const v4i *)(wl + b_lane + f * R * WROW);
#pragma unroll
         for (int i = 0; i < MT; ++i)
            fa[0][i].c[0] = *(const v4i *)(smem + a_row[0][i]);
      }
      half_body(h0, std::false_type{}, 0);
      half_body(h1, std::true_type{}, 0);
      for (int it = 1; it < my_tiles; ++it) {
         half_body(h0, std::true_type{}, it);
         half_body(h1, std::true_type{}, it);
      }
      // the last half: nothing left to multiply
      const int m_last = ((my_tiles - 1) * nwg + bid) * 256;
      static_for<SLICES>([&](auto sc) { store_slice(h1, sc, m_last); });
   });
   wait_vmcnt<0>();
}

// Shapes the kernel takes: one group's 64 input channels, 128 output channels, KH x KW = 3 x 3, stride and dilation 1, output
// rows of a power-of-two width that divides 256 (so that a tile is whole rows of one image), planes of whole tiles, a patch
// that fits its buffer, and a store the register path handles.
inline bool conv_i8_resident_applies(const ConvRows &a, int Cg, const int8_t *Wp, int M, int N, int K)
{
   if (Cg != 64 || N != 128 || a.ntaps != 9 || a.kw != 3 || K != 576)
      return false;
   if (a.stride_h != 1 || a.stride_w != 1 || a.dil_h != 1 || a.dil_w != 1)
      return false;
   if (a.OW < 16 || a.OW > 256 || (a.OW & (a.OW - 1)) != 0 || (a.OH * a.OW) % 256 != 0 || M % 256 != 0)
      return false;
   const int rows = 256 / a.OW;
   if ((rows + 2) * (a.OW + 2) * 6 > 5 * 8 * 64) // patch chunks against the lanes of its load instructions
      return false;
   return (((uintptr_t)a.X | (uintptr_t)Wp) & 15) == 0 && a.C % 16 == 0;
}

template <class EPI>
static int launch_conv_i8_resident(const LaunchCfg &lc, const ConvRows &a, const int8_t *Wp, int M, const EPI &ep)
{
   ResidentConv g;
   g.X = a.X; g.H = a.H; g.W = a.W; g.C = a.C; g.OH = a.OH; g.OW = a.OW; g.pad_h0 = a.pad_h0; g.pad_w0 = a.pad_w0;
   g.ow_shift = 0;
   while ((1 << g.ow_shift) < a.OW)
      ++g.ow_shift;
   g.tiles_per_image = a.OH * a.OW / 256;
   const int ntiles = M / 256;
   constexpr int K = 9 * 64, WROW = K + 32;
   constexpr size_t wbytes = ((128 * WROW + 1023) / 1024 + 1) * 1024, smem = wbytes + 2 * 5 * 8 * 1024;
   static_assert(smem <= 160 * 1024, "weights and two patch buffers in the CU's LDS");
   auto kern = conv_i8_resident_kernel<3, 3, EPI>;
   static bool configured[64] = {};
   if (int st = configure_lds_once(kern, smem, configured))
      return st;
   int ncu = 0;
   if (int st = cu_count_of_current_device(ncu))
      return st;
   const int grid = ntiles < ncu ? ntiles : ncu;
   hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(512), smem, lc.stream, g, Wp, ep, ntiles);
   return launch_status("conv_i8_resident_kernel");
}

} // namespace sofie_hip
