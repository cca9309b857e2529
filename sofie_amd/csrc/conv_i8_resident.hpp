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
//     barrier inside a tile.  The eight waves meet once per tile, and one of the two waves of every SIMD stores its tile after
//     the next tile's barrier: one wave's conversion and store run under the other's MFMAs;
//   * pixels and weight rows are 64 + 32 (576 + 32) bytes apart in LDS: records 96 bytes (mod 256) apart are read by
//     ds_read_b128 at the full rate from any starting record (measured: 237 B/clk; 80, 112, 144 or 592 bytes apart: 123), so no
//     swizzle is needed and every fragment address is a lane constant plus a uniform offset.
// Workgroup = 8 waves (4 x 2), wave tile 64 x 64 (v_mfma_i32_16x16x64_i8, 64 accumulators), store from registers.
//
// What bounds it (batch 256 of 64 x 64 images, 70 us): not the matrix cores (33 us of MFMA at the clock it runs at) and not
// the LDS reads (the same time with the fragments of taps 2..8 not read at all), but the memory side: 134 MB of output and
// 67 MB of input (100 MB with the halo rows) per launch.  With one MFMA in sixteen the launch still takes 52 us.
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

   // ---- fragment addresses: a lane constant plus uniform offsets
   const int a_lane = lr * PIX + lk * 16;
   const int b_lane = (wn * TN + lr) * WROW + lk * 16;
   int a_blk[MT]; // patch byte offset of the first pixel of the wave's i-th block of 16 output pixels, tap (0, 0)
#pragma unroll
   for (int i = 0; i < MT; ++i) {
      const int p = wm * TM + i * R;
      a_blk[i] = ((p >> g.ow_shift) * PW + (p & (g.OW - 1))) * PIX;
   }
   auto read_tap = [&](const int8_t *pbuf, int tap_off_a, int tap, frag_t(&fa)[MT], frag_t(&fb)[NT]) {
#pragma unroll
      for (int j = 0; j < NT; ++j)
         fb[j].c[0] = *(const v4i *)(wl + b_lane + j * R * WROW + tap * 64);
#pragma unroll
      for (int i = 0; i < MT; ++i)
         fa[i].c[0] = *(const v4i *)(pbuf + a_lane + a_blk[i] + tap_off_a);
   };

   int m_cur, img, oh0;
   tile_of(0, m_cur, img, oh0);
   load_patch(0, img, oh0);
   uint32_t col_words[EPI::kColWords];
   ep.load_column_for_registers(wn * TN + lane, col_words); // one column tile: the constants are the same for every tile
   constexpr bool kBias = EPI::kBiasInAccumulator;
   acc_t acc[MT][NT];
   // Half of the waves, one of the two on every SIMD (waves w and w + 4 share one), store a tile only after the NEXT tile's
   // barrier: their conversion and store then run while the other wave of the SIMD multiplies, and the other way round
   // later in the tile.  Every wave passes the same number of barriers (one per tile and one more).
   const bool late_store = wave >= NW / 2;
   auto store_tile = [&](int m_tile) {
      ep.dispatch_for_registers([&](auto mode) {
         tile_store_or_sum_from_registers<decltype(mode)::value, MMA, MT, NT>(ep, acc, m_tile + wm * TM, wn * TN, lane, col_words);
      });
   };
   int m_prev = m_cur;
   for (int it = 0; it <= my_tiles; ++it) {
      // the patch of this tile has landed for every wave, and every wave is done multiplying the tile before (whose buffer the
      // next patch goes to).  A wave's loads of the patch are older than the stores it has issued since, which may stay in
      // flight: loads return in order, so "at most as many operations outstanding as one tile's stores" means the loads are done.
      if (it == 0 || !ep.stores_one_byte_rows())
         wait_vmcnt<0>();
      else
         wait_vmcnt<MT>();
      __builtin_amdgcn_s_barrier();
      int m_nxt, img_n, oh_n;
      tile_of(it + 1, m_nxt, img_n, oh_n);
      if (it < my_tiles)
         load_patch((it + 1) & 1, img_n, oh_n);
      if (late_store && it > 0)
         store_tile(m_prev);
      if (it == my_tiles)
         break;
      // accumulators: the bias of the lane's columns (or zero)
      {
         int first_col_addr = lk * 16;
         asm volatile("" : "+v"(first_col_addr));
         static_for<NT>([&](auto cj) {
            constexpr int j = decltype(cj)::value;
            acc_t b = {0, 0, 0, 0};
            if constexpr (kBias) {
#pragma unroll
               for (int v = 0; v < 4; ++v)
                  b[v] = __builtin_amdgcn_ds_bpermute(first_col_addr + (j * R + v) * 4, (int)col_words[EPI::kBiasWord]);
            }
#pragma unroll
            for (int i = 0; i < MT; ++i)
               acc[i][j] = b;
         });
      }
      const int8_t *pbuf = patch + (it & 1) * PBYTES;
      // fragments of three taps in registers: tap t is multiplied while those of tap t + 2 are on their way (the reads of one
      // tap ahead would have the 16 MFMAs of a tap to arrive in: too short with eight waves reading)
      frag_t fa[3][MT], fb[3][NT];
      __builtin_amdgcn_sched_barrier(0);
      read_tap(pbuf, 0, 0, fa[0], fb[0]);
      read_tap(pbuf, (1 / KW * PW + 1 % KW) * PIX, 1, fa[1], fb[1]);
      static_for<NTAPS>([&](auto tc) {
         constexpr int tap = decltype(tc)::value;
         constexpr int cur = tap % 3;
         // (the scheduling fences keep the reads where they are written: left alone, the compiler sinks each one to just in
         // front of its first use and waits for it there, every four MFMAs)
         __builtin_amdgcn_sched_barrier(0);
         if constexpr (tap + 2 < NTAPS) {
            constexpr int ky = (tap + 2) / KW, kx = (tap + 2) % KW;
            read_tap(pbuf, (ky * PW + kx) * PIX, tap + 2, fa[(tap + 2) % 3], fb[(tap + 2) % 3]);
         }
         static_for<NT>([&](auto cj) {
            constexpr int j = decltype(cj)::value;
            static_for<MT>([&](auto ci) {
               constexpr int i = (j & 1) ? MT - 1 - decltype(ci)::value : decltype(ci)::value;
               acc[i][j] = MMA::mma(fb[cur][j], fa[cur][i], acc[i][j]);
            });
         });
         if constexpr (tap + 2 < NTAPS) {
            static_for<MT + NT>([&](auto gc) {
               __builtin_amdgcn_sched_group_barrier(0x008, (MT * NT) / (MT + NT), 0);
               __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            });
         }
         __builtin_amdgcn_sched_barrier(0);
      });
      if (!late_store)
         store_tile(m_cur);
      m_prev = m_cur;
      m_cur = m_nxt;
   }
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
