// int8 convolution over FEW input channels (the first layer of an image network: 3 channels, 3 x 3), NCHW input, 64 output
// channels, output rows stored NHWC.
//
// The reduction is short (channels x kh x kw <= 64 bytes: one MFMA step), so the work is reading each output pixel's window
// and storing 64 bytes per pixel; no LDS tile, no barrier in the loop, every wave on its own:
//   * the reduction index is re-ordered to (channel, ky) pairs of FOUR kx positions each (kw <= 4; the weights of kx >= kw
//     are zero): k' = (channel * kh + ky) * 4 + kx, at most 16 pairs.  For stride 1 and dilation 1 in x the four bytes of a
//     pair are the input row's bytes iw0 .. iw0 + 3, consecutive in memory: one window per pair instead of one byte per tap;
//   * a window is cut out of an aligned 8-byte load that never leaves the row: the load starts at (iw0 & ~3) clamped to
//     [0, W - 8], and a 64-bit shift by the distance to iw0 moves the window down (or up, left of the image) and shifts in
//     the zeros of the padding on either side.  A row outside the image gives a zero window (its load reads a valid address);
//   * lane (lr, lk) of the MFMA holds the pairs 4 lk .. 4 lk + 3 of pixel lr: four windows are its whole A fragment;
//   * the weights, re-ordered once per workgroup through LDS, stay in registers (four fragments), and the bias is the addend
//     of the only MFMA of each accumulator;
//   * a wave works on 64 consecutive output pixels at a time (4 x 4 MFMAs of 16 x 16 x 64) and stores them from registers.
#pragma once
#include "mfma8_gemm_persist.hpp"

namespace sofie_hip {

template <class EPI>
__global__ __launch_bounds__(256) void conv_i8_few_channels_kernel(FewChannelConv g, const int8_t *__restrict__ Wp, int Kp, EPI ep, int ngroups)
{
   typedef MfmaI8x16 MMA;
   constexpr int R = 16, MT = 4, NT = 4;
   typedef MMA::acc_t acc_t;
   typedef MMA::frag_t frag_t;
   typedef uint64_t u64_dword_aligned __attribute__((aligned(4))); // the loads start on dword boundaries
   __shared__ v4i wfrag[64 * 4]; // [column][quarter of the reduction]: 16 bytes each
   const int t = threadIdx.x;
   const int lane = t & 63;
   const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
   const int lr = lane % R, lk = lane / R;
   const int npairs = g.Cg * g.kh;

   // ---- weights: column t / 4, bytes k' = 16 (t % 4) .. + 15, gathered from the packed order k = (ky * kw + kx) * Cg + channel
   {
      const int col = t >> 2, q = t & 3;
      uint32_t w[4] = {0, 0, 0, 0};
      for (int b = 0; b < 16; ++b) {
         const int pair = q * 4 + (b >> 2), kx = b & 3;
         const int c = g.pair_c[pair], ky = g.pair_ky[pair];
         int8_t v = 0;
         if (pair < npairs && kx < g.kw)
            v = Wp[(size_t)col * Kp + (ky * g.kw + kx) * g.Cg + c];
         w[b >> 2] |= (uint32_t)(uint8_t)v << (8 * (b & 3));
      }
      const v4i wv = {(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
      wfrag[col * 4 + q] = wv;
   }
   __syncthreads();
   frag_t fb[NT];
#pragma unroll
   for (int j = 0; j < NT; ++j)
      fb[j].c[0] = wfrag[(j * R + lr) * 4 + lk];

   // ---- the lane's four pairs: plane and row offset, and the row distance (a pair past the end never lies inside the image)
   int pair_off[4], pair_dy[4];
#pragma unroll
   for (int q = 0; q < 4; ++q) {
      const int pair = lk * 4 + q;
      const int c = g.pair_c[pair], ky = g.pair_ky[pair];
      pair_off[q] = (c * g.H + ky * g.dil_h) * g.W;
      pair_dy[q] = pair < npairs ? ky * g.dil_h : (1 << 24);
   }

   // ---- epilogue constants of the lane's column, and the accumulators' start values (bias or zero), per column block
   uint32_t col_words[EPI::kColWords];
   ep.load_column_for_registers(lane, col_words);
   acc_t acc0[NT];
   {
      int first_col_addr = lk * 16;
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
         for (int v = 0; v < 4; ++v)
            acc0[j][v] = EPI::kBiasInAccumulator ? __builtin_amdgcn_ds_bpermute(first_col_addr + (j * R + v) * 4, (int)col_words[EPI::kBiasWord]) : 0;
   }

   // The windows of a group are requested one group ahead: while they are on their way, the group before is multiplied,
   // converted and stored.
   const int ohw = g.OH * g.OW;
   uint64_t chunk[MT][4];
   bool ok[MT][4];
   int rsh[MT], lsh[MT];
   auto request = [&](int grp) {
      // first pixel of the group (uniform): image, row, column
      const int p0 = grp * 64;
      const int n0 = p0 / ohw, r0 = p0 - n0 * ohw;
      const int oh0 = r0 / g.OW, ow0 = r0 - oh0 * g.OW;
      const int8_t *img0 = g.X + (long long)n0 * g.img_stride; // uniform: the loads take it as their scalar base
      // pixel p0 + lr, and the lane's other pixels 16, 32, 48 further on: at most one row further each time (OW >= 16),
      // which may be the first row of the next image
      int ow = ow0 + lr, oh = oh0, dn = 0;
      auto wrap = [&]() {
         if (ow >= g.OW) {
            ow -= g.OW;
            oh += 1;
            if (oh >= g.OH)
               oh = 0, dn += 1;
         }
      };
      wrap();
#pragma unroll
      for (int i = 0; i < MT; ++i) {
         const int ih0 = oh * g.stride_h - g.pad_h0, iw0 = ow - g.pad_w0;
         int cs = iw0 & ~3;
         cs = cs < 0 ? 0 : cs;
         cs = cs > g.W - 8 ? g.W - 8 : cs;
         const int s = iw0 - cs; // -3 .. 7
         rsh[i] = s > 0 ? 8 * s : 0;
         lsh[i] = s < 0 ? -8 * s : 0;
         const uint32_t row_off = (uint32_t)(dn * (int)g.img_stride + ih0 * g.W + cs);
#pragma unroll
         for (int q = 0; q < 4; ++q) {
            ok[i][q] = (unsigned)(ih0 + pair_dy[q]) < (unsigned)g.H;
            const uint32_t off = ok[i][q] ? row_off + (uint32_t)pair_off[q] : 0u;
            chunk[i][q] = *(const u64_dword_aligned *)(img0 + off);
         }
         ow += R;
         wrap();
      }
   };
   const int stride = gridDim.x * 4;
   int grp = blockIdx.x * 4 + wave;
   if (grp < ngroups)
      request(grp);
   for (; grp < ngroups; grp += stride) {
      frag_t fa[MT];
#pragma unroll
      for (int i = 0; i < MT; ++i)
#pragma unroll
         for (int q = 0; q < 4; ++q) {
            const uint32_t win = (uint32_t)((chunk[i][q] >> rsh[i]) << lsh[i]);
            fa[i].c[0][q] = ok[i][q] ? (int)win : 0;
         }
      if (grp + stride < ngroups)
         request(grp + stride);
      acc_t acc[MT][NT];
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
         for (int i = 0; i < MT; ++i)
            acc[i][j] = MMA::mma(fb[j], fa[i], acc0[j]);
      ep.dispatch_for_registers([&](auto mode) {
         tile_store_from_registers<decltype(mode)::value, MMA, MT, NT>(ep, acc, grp * 64, 0, lane, col_words);
      });
   }
}

// Shapes the kernel takes (the caller has checked the output: 64 channels, whole groups of 64 pixels, rows stored as they are).
inline bool conv_i8_few_channels_applies(const FewChannelConv &g, const int8_t *Wp)
{
   return g.kw <= 4 && g.Cg * g.kh <= 16 && g.pad_w0 <= 3 && g.W % 4 == 0 && g.W >= 8 && g.OW >= 16 && g.img_stride < (1LL << 28) &&
          (((uintptr_t)g.X | (uintptr_t)g.img_stride) & 3) == 0 && Wp != nullptr;
}

template <class EPI>
static int launch_conv_i8_few_channels(const LaunchCfg &lc, FewChannelConv g, const int8_t *Wp, int M, int Kp, const EPI &ep)
{
   const int ngroups = M / 64;
   int ncu = 0;
   if (int st = cu_count_of_current_device(ncu))
      return st;
   for (int pair = 0; pair < 16; ++pair) {
      g.pair_c[pair] = (unsigned char)(pair / g.kh);
      g.pair_ky[pair] = (unsigned char)(pair % g.kh);
   }
   // four waves per workgroup, two workgroups per CU (what the registers allow): all of them resident at once, the weights
   // re-ordered once per workgroup
   int grid = (ngroups + 3) / 4;
   if (grid > 2 * ncu)
      grid = 2 * ncu;
   hipLaunchKernelGGL(conv_i8_few_channels_kernel<EPI>, dim3((unsigned)grid), dim3(256), 0, lc.stream, g, Wp, Kp, ep, ngroups);
   return launch_status("conv_i8_few_channels_kernel");
}

} // namespace sofie_hip
