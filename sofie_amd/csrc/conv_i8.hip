// int8 convolution as a GEMM over the whole batch: rows = output pixels (image, oh, ow), columns =
// output channels, K = (kh, kw, ci) with ci fastest.  The weights are re-laid out once into
// [Cout][Kp] (Kp = K rounded up to 16, zero filled); the column matrix of a group of images is built
// in the workspace and multiplied on the matrix cores with the requantisation fused into the store.
// Activations may be NCHW (the ONNX layout) or NHWC (channels fastest: what a chain of convolutions
// keeps between layers, since it makes both the gather and the store contiguous).
#include "i8_epilogue.hpp"

namespace sofie_hip {

struct ConvGeom {
   int C, H, W, kh, kw, OH, OW, pad_h0, pad_w0, stride_h, stride_w, dil_h, dil_w;
   int Cg, K, Kp; // channels per group, kh*kw*Cg, K rounded up to 16
};

// [Cout][Cg][kh][kw] -> [Cout][Kp] with k' = (ky*kw + kx)*Cg + ci
__global__ __launch_bounds__(256) void pack_conv_weight_kernel(int8_t *__restrict__ dst, const int8_t *__restrict__ src, int Cout,
                                                                ConvGeom g)
{
   const size_t total = (size_t)Cout * g.Kp;
   const size_t stride = (size_t)gridDim.x * blockDim.x;
   for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < total; i += stride) {
      int co = (int)(i / g.Kp), k = (int)(i % g.Kp);
      int8_t v = 0;
      if (k < g.K) {
         int ci = k % g.Cg, t = k / g.Cg;
         int kx = t % g.kw, ky = t / g.kw;
         v = src[(((size_t)co * g.Cg + ci) * g.kh + ky) * g.kw + kx];
      }
      dst[i] = v;
   }
}

// One thread builds one 16-byte chunk of one row of the column matrix.
template <bool NHWC_FAST>
__global__ __launch_bounds__(256) void im2col_i8_kernel(int8_t *__restrict__ col, const int8_t *__restrict__ X, ConvGeom g,
                                                         int c_first, int x_nhwc, long long m_first, long long rows)
{
   const int cpr = g.Kp / 16;
   const size_t total = (size_t)rows * cpr;
   const size_t stride = (size_t)gridDim.x * blockDim.x;
   for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < total; i += stride) {
      const long long m = m_first + (long long)(i / cpr);
      const int chunk = (int)(i % cpr);
      const int ow = (int)(m % g.OW);
      const long long t = m / g.OW;
      const int oh = (int)(t % g.OH);
      const long long img = t / g.OH;
      v4i out = v4i{0, 0, 0, 0};
      if (NHWC_FAST) {
         // Cg % 16 == 0: the chunk is 16 consecutive channels of one tap
         const int k = chunk * 16;
         const int ci = k % g.Cg, tap = k / g.Cg;
         const int kx = tap % g.kw, ky = tap / g.kw;
         const int ih = oh * g.stride_h - g.pad_h0 + ky * g.dil_h;
         const int iw = ow * g.stride_w - g.pad_w0 + kx * g.dil_w;
         if (k < g.K && (unsigned)ih < (unsigned)g.H && (unsigned)iw < (unsigned)g.W)
            out = *(const v4i *)(X + (((size_t)img * g.H + ih) * g.W + iw) * g.C + c_first + ci);
      } else {
         union {
            v4i v;
            int8_t b[16];
         } u;
         u.v = out;
#pragma unroll
         for (int j = 0; j < 16; ++j) {
            const int k = chunk * 16 + j;
            if (k < g.K) {
               const int ci = k % g.Cg, tap = k / g.Cg;
               const int kx = tap % g.kw, ky = tap / g.kw;
               const int ih = oh * g.stride_h - g.pad_h0 + ky * g.dil_h;
               const int iw = ow * g.stride_w - g.pad_w0 + kx * g.dil_w;
               if ((unsigned)ih < (unsigned)g.H && (unsigned)iw < (unsigned)g.W) {
                  const size_t idx = x_nhwc ? (((size_t)img * g.H + ih) * g.W + iw) * g.C + c_first + ci
                                            : (((size_t)img * g.C + c_first + ci) * g.H + ih) * g.W + iw;
                  u.b[j] = X[idx];
               }
            }
         }
         out = u.v;
      }
      *(v4i *)(col + ((size_t)(m - m_first) * g.Kp) + chunk * 16) = out;
   }
}

static inline size_t round256(size_t v) { return (v + 255) & ~(size_t)255; }

static int check_conv(const sofie_conv_desc *d, ConvGeom &g, const char *who)
{
   SOFIE_HIP_REQUIRE(d->N >= 0 && d->C > 0 && d->H > 0 && d->W > 0 && d->Cout > 0 && d->kh > 0 && d->kw > 0, "%s: bad shape", who);
   SOFIE_HIP_REQUIRE(d->group > 0 && d->C % d->group == 0 && d->Cout % d->group == 0, "%s: group %d does not divide the channels", who, d->group);
   SOFIE_HIP_REQUIRE(d->stride_h > 0 && d->stride_w > 0 && d->dil_h > 0 && d->dil_w > 0, "%s: bad stride or dilation", who);
   SOFIE_HIP_REQUIRE(d->pad_h0 >= 0 && d->pad_w0 >= 0 && d->pad_h1 >= 0 && d->pad_w1 >= 0, "%s: negative padding", who);
   const int eff_kh = d->dil_h * (d->kh - 1) + 1, eff_kw = d->dil_w * (d->kw - 1) + 1;
   SOFIE_HIP_REQUIRE(d->H + d->pad_h0 + d->pad_h1 >= eff_kh && d->W + d->pad_w0 + d->pad_w1 >= eff_kw,
                     "%s: kernel larger than the padded image", who);
   const int OH = (d->H + d->pad_h0 + d->pad_h1 - eff_kh) / d->stride_h + 1;
   const int OW = (d->W + d->pad_w0 + d->pad_w1 - eff_kw) / d->stride_w + 1;
   SOFIE_HIP_REQUIRE(OH == d->OH && OW == d->OW, "%s: output shape %dx%d does not match the descriptor's %dx%d", who, OH, OW, d->OH, d->OW);
   g.C = d->C; g.H = d->H; g.W = d->W; g.kh = d->kh; g.kw = d->kw; g.OH = OH; g.OW = OW;
   g.pad_h0 = d->pad_h0; g.pad_w0 = d->pad_w0; g.stride_h = d->stride_h; g.stride_w = d->stride_w;
   g.dil_h = d->dil_h; g.dil_w = d->dil_w;
   g.Cg = d->C / d->group;
   const long long K = (long long)g.Cg * d->kh * d->kw;
   SOFIE_HIP_REQUIRE(K < (1 << 24), "%s: reduction too long", who);
   g.K = (int)K;
   g.Kp = (g.K + 15) & ~15;
   return SOFIE_HIP_OK;
}

} // namespace sofie_hip

using namespace sofie_hip;

extern "C" {

size_t sofie_hip_conv_weight_i8_packed_bytes(const sofie_conv_desc *d)
{
   if (!d || d->group <= 0)
      return 0;
   size_t K = (size_t)(d->C / d->group) * d->kh * d->kw;
   return round256((size_t)d->Cout * ((K + 15) & ~(size_t)15));
}

int sofie_hip_pack_conv_weight_i8(sofie_hip_ctx *ctx, const sofie_conv_desc *d, int8_t *dst, const int8_t *src)
{
   SOFIE_HIP_REQUIRE(ctx && d && dst && src, "sofie_hip_pack_conv_weight_i8: NULL argument");
   ConvGeom g;
   int st = check_conv(d, g, "sofie_hip_pack_conv_weight_i8");
   if (st)
      return st;
   size_t total = (size_t)d->Cout * g.Kp;
   size_t blocks = (total + 255) / 256;
   if (blocks > 4096)
      blocks = 4096;
   hipLaunchKernelGGL(pack_conv_weight_kernel, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, dst, src, d->Cout, g);
   return launch_status("pack_conv_weight_kernel");
}

// Shapes the implicit-GEMM kernels take (pointer alignment is checked at the call): NHWC input, channels per
// group a power of two >= 64 (a 64-byte K slab then lies inside one input pixel), at most 32 filter taps,
// 32-bit byte offsets.
static bool conv_i8_implicit_shape(const sofie_conv_desc *d, int x_layout)
{
   if (d->group <= 0 || d->C % d->group != 0)
      return false;
   const int Cg = d->C / d->group, ntaps = d->kh * d->kw;
   const long long xbytes = (long long)d->N * d->H * d->W * d->C;
   const long long reach = xbytes + (long long)(d->pad_h0 + d->kh * d->dil_h + 1) * d->W * d->C + (long long)(d->pad_w0 + d->kw * d->dil_w + 1) * d->C;
   const long long rows = (long long)d->N * d->OH * d->OW;
   const int kw_recip = (65536 + d->kw - 1) / d->kw;
   for (int t = 0; t < ntaps && t < 32; ++t)
      if (((t * kw_recip) >> 16) != t / d->kw)
         return false;
   return x_layout == SOFIE_LAYOUT_NHWC && (Cg & (Cg - 1)) == 0 && Cg >= 64 && ntaps <= 32 &&
          d->C % 16 == 0 && reach < (1LL << 31) && rows < (1LL << 31);
}

// The whole reduction (taps x channels per group) fits one 64-byte slab: the rows are gathered inside the GEMM kernel.
static bool conv_i8_gather_shape(const sofie_conv_desc *d)
{
   if (d->group <= 0 || d->C % d->group != 0)
      return false;
   const long long K = (long long)(d->C / d->group) * d->kh * d->kw;
   return K <= 64 && (long long)(d->kh - 1) * d->dil_h <= 127 && (long long)(d->kw - 1) * d->dil_w <= 127 &&
          (long long)d->C * d->H * d->W < (1LL << 31) && (long long)d->N * d->OH * d->OW < (1LL << 31);
}

size_t sofie_hip_conv_i8_workspace(const sofie_conv_desc *d, const sofie_conv_i8_args *a)
{
   if (!d || !a || d->group <= 0)
      return 0;
   size_t K = (size_t)(d->C / d->group) * d->kh * d->kw;
   size_t Kp = (K + 15) & ~(size_t)15;
   // the column matrix of one image, unless the kernel reads the activations directly
   size_t need = (conv_i8_implicit_shape(d, a->x_layout) || conv_i8_gather_shape(d)) ? 0 : round256((size_t)d->OH * d->OW * Kp);
   if (!a->w_is_packed)
      need += sofie_hip_conv_weight_i8_packed_bytes(d);
   return need;
}

size_t sofie_hip_conv_i8_column_matrix_bytes(const sofie_conv_desc *d)
{
   if (!d || d->group <= 0)
      return 0;
   const size_t K = (size_t)(d->C / d->group) * d->kh * d->kw;
   return round256((size_t)d->OH * d->OW * ((K + 15) & ~(size_t)15));
}

int sofie_hip_conv_i8(sofie_hip_ctx *ctx, const sofie_conv_desc *d, const sofie_conv_i8_args *a)
{
   SOFIE_HIP_REQUIRE(ctx && d && a, "sofie_hip_conv_i8: NULL argument");
   ConvGeom g;
   int st = check_conv(d, g, "sofie_hip_conv_i8");
   if (st)
      return st;
   SOFIE_HIP_REQUIRE(a->out == SOFIE_I8OUT_I32 || a->out == SOFIE_I8OUT_F32 || a->out == SOFIE_I8OUT_I8 || a->out == SOFIE_I8OUT_I8_PLANE_SUMS,
                     "sofie_hip_conv_i8: unknown output kind %d", a->out);
   // Plane sums ride in the tile store of the matrix-core kernels: a wave's tile (at most 128 rows of a 256-row tile) must lie in one
   // image and hold valid rows only.
   const bool plane_sums = a->out == SOFIE_I8OUT_I8_PLANE_SUMS;
   const int out_kind = plane_sums ? SOFIE_I8OUT_I8 : a->out;
   SOFIE_HIP_REQUIRE(!plane_sums || ((g.OH * g.OW) % 256 == 0 && (conv_i8_implicit_shape(d, a->x_layout) || conv_i8_gather_shape(d))),
                     "sofie_hip_conv_i8: plane sums need output planes of a multiple of 256 pixels (got %d) and a shape the kernel reads "
                     "without a column matrix", g.OH * g.OW);
   SOFIE_HIP_REQUIRE((a->x_layout == SOFIE_LAYOUT_NCHW || a->x_layout == SOFIE_LAYOUT_NHWC) &&
                        (a->y_layout == SOFIE_LAYOUT_NCHW || a->y_layout == SOFIE_LAYOUT_NHWC),
                     "sofie_hip_conv_i8: unknown layout");
   SOFIE_HIP_REQUIRE(a->out == SOFIE_I8OUT_I32 || a->scale != nullptr, "sofie_hip_conv_i8: per-channel scale is NULL");
   if (d->N == 0)
      return SOFIE_HIP_OK;
   SOFIE_HIP_REQUIRE(a->X && a->W && a->Y, "sofie_hip_conv_i8: NULL tensor pointer");
   const size_t need = sofie_hip_conv_i8_workspace(d, a);
   SOFIE_HIP_REQUIRE(need == 0 || (a->workspace != nullptr && a->workspace_bytes >= need),
                     "sofie_hip_conv_i8: a workspace of at least %zu bytes is needed", need);
   SOFIE_HIP_REQUIRE(((uintptr_t)a->workspace & 255) == 0, "sofie_hip_conv_i8: workspace must be 256-byte aligned");

   char *ws = (char *)a->workspace;
   size_t ws_left = a->workspace_bytes;
   const int8_t *Wp = a->W;
   if (!a->w_is_packed) {
      st = sofie_hip_pack_conv_weight_i8(ctx, d, (int8_t *)ws, a->W);
      if (st)
         return st;
      Wp = (const int8_t *)ws;
      size_t wb = sofie_hip_conv_weight_i8_packed_bytes(d);
      ws += wb;
      ws_left -= wb;
   }
   const int OHW = g.OH * g.OW;
   const int Cout_g = d->Cout / d->group;
   const size_t esz = out_kind == SOFIE_I8OUT_I8 ? 1 : 4;
   // the context's conv_explicit option sends every shape through the column matrix, provided the caller's workspace holds
   // one (a Session sized by sofie_hip_conv_i8_workspace keeps working, on the kernels that need none)
   const bool column_matrix_by_option = ctx->opt.conv_explicit && !plane_sums && ws != nullptr && ws_left >= (size_t)OHW * g.Kp;

   // Implicit GEMM: the kernel reads the NHWC activations directly, one launch per group over the whole batch.
   // Needs K slabs that lie inside one input pixel (channels per group a power of two >= 64) and 32-bit offsets.
   {
      const int ntaps = d->kh * d->kw;
      const int kw_recip = (65536 + d->kw - 1) / d->kw;
      const long long rows = (long long)d->N * OHW;
      const bool implicit = !column_matrix_by_option && conv_i8_implicit_shape(d, a->x_layout) && (((uintptr_t)a->X & 15) == 0) && (((uintptr_t)Wp & 15) == 0) &&
                            g.Kp == g.K;
      if (implicit) {
         int cg_shift = 0;
         while ((1 << cg_shift) < g.Cg)
            ++cg_shift;
         for (int grp = 0; grp < d->group; ++grp) {
            ConvRows src;
            src.X = a->X + (size_t)grp * g.Cg;
            src.H = d->H; src.W = d->W; src.C = d->C; src.OH = g.OH; src.OW = g.OW;
            src.stride_h = d->stride_h; src.stride_w = d->stride_w; src.pad_h0 = d->pad_h0; src.pad_w0 = d->pad_w0;
            src.dil_h = d->dil_h; src.dil_w = d->dil_w; src.kw = d->kw; src.ntaps = ntaps;
            src.cg_shift = cg_shift; src.kw_recip = kw_recip;
            // ceil(2^64 / d) for d >= 2; 0 stands for d == 1 (2^64 does not fit)
            auto recip64 = [](unsigned d) -> unsigned long long { return d <= 1 ? 0ull : (~0ull / d) + 1; };
            src.ohw_mul = recip64((unsigned)OHW);
            src.ow_mul = recip64((unsigned)g.OW);
            I8Epilogue ep;
            ep.bias = a->bias;
            ep.scale = a->scale;
            ep.scale_scalar = 1.0f;
            ep.q_scale = 1.0f;
            ep.relu_acc = (out_kind == SOFIE_I8OUT_I32) ? a->relu : 0;
            ep.relu_out = (out_kind == SOFIE_I8OUT_I32) ? 0 : a->relu;
            ep.out = out_kind;
            ep.ldy = d->Cout;
            ep.N = Cout_g;
            ep.n_offset = grp * Cout_g;
            ep.nchw_ohw = (a->y_layout == SOFIE_LAYOUT_NHWC || plane_sums) ? 0 : OHW;
            ep.rows_per_plane = plane_sums ? OHW : 0;
            ep.Y = a->Y;
            st = conv_i8_implicit(launch_cfg_i8(ctx), src, g.Cg, Wp + (size_t)grp * Cout_g * g.Kp, (int)rows, Cout_g, g.K, ep);
            if (st)
               return st;
         }
         return SOFIE_HIP_OK;
      }
   }
   // Few input channels (the first layer of an image network): K = taps x channels <= 64 is one slab, gathered in the kernel.
   if (!column_matrix_by_option && conv_i8_gather_shape(d) && (((uintptr_t)Wp & 15) == 0)) {
      const long long rows = (long long)d->N * OHW;
      const bool nhwc = a->x_layout == SOFIE_LAYOUT_NHWC;
      for (int grp = 0; grp < d->group; ++grp) {
         GatherConvRows src;
         src.X = a->X + (nhwc ? (size_t)grp * g.Cg : (size_t)grp * g.Cg * d->H * d->W);
         src.H = d->H; src.W = d->W; src.OH = g.OH; src.OW = g.OW;
         src.stride_h = d->stride_h; src.stride_w = d->stride_w; src.pad_h0 = d->pad_h0; src.pad_w0 = d->pad_w0;
         src.pix_mul = nhwc ? d->C : 1;
         src.img_stride = (long long)d->C * d->H * d->W;
         src.K = g.K;
         for (int k = 0; k < 64; ++k) {
            src.koff[k] = 0;
            src.dy[k] = src.dx[k] = 0;
            if (k < g.K) {
               const int ci = k % g.Cg, tap = k / g.Cg; // the order of the packed weights: tap-major, channel-minor
               const int dy = (tap / d->kw) * d->dil_h, dx = (tap % d->kw) * d->dil_w;
               src.dy[k] = (signed char)dy;
               src.dx[k] = (signed char)dx;
               src.koff[k] = nhwc ? (dy * d->W + dx) * d->C + ci : ci * d->H * d->W + dy * d->W + dx;
            }
         }
         I8Epilogue ep;
         ep.bias = a->bias;
         ep.scale = a->scale;
         ep.scale_scalar = 1.0f;
         ep.q_scale = 1.0f;
         ep.relu_acc = (out_kind == SOFIE_I8OUT_I32) ? a->relu : 0;
         ep.relu_out = (out_kind == SOFIE_I8OUT_I32) ? 0 : a->relu;
         ep.out = out_kind;
         ep.ldy = d->Cout;
         ep.N = Cout_g;
         ep.n_offset = grp * Cout_g;
         ep.nchw_ohw = (a->y_layout == SOFIE_LAYOUT_NHWC || plane_sums) ? 0 : OHW;
         ep.rows_per_plane = plane_sums ? OHW : 0;
         ep.Y = a->Y;
         if (!nhwc && d->stride_w == 1 && d->dil_w == 1) {
            FewChannelConv fc;
            fc.X = src.X;
            fc.H = d->H; fc.W = d->W; fc.OH = g.OH; fc.OW = g.OW;
            fc.stride_h = d->stride_h; fc.pad_h0 = d->pad_h0; fc.pad_w0 = d->pad_w0; fc.dil_h = d->dil_h;
            fc.kh = d->kh; fc.kw = d->kw; fc.Cg = g.Cg;
            fc.img_stride = src.img_stride;
            bool taken = false;
            st = conv_i8_few_channels(launch_cfg_i8(ctx), fc, Wp + (size_t)grp * Cout_g * g.Kp, (int)rows, Cout_g, g.Kp, ep, &taken);
            if (st)
               return st;
            if (taken)
               continue;
         }
         st = conv_i8_gather(launch_cfg_i8(ctx), src, Wp + (size_t)grp * Cout_g * g.Kp, (int)rows, Cout_g, g.Kp, ep);
         if (st)
            return st;
      }
      return SOFIE_HIP_OK;
   }
   SOFIE_HIP_REQUIRE(!plane_sums, "sofie_hip_conv_i8: plane sums need 16-byte aligned activations and weights");
   const size_t per_image = (size_t)OHW * g.Kp;
   SOFIE_HIP_REQUIRE(ws != nullptr && ws_left >= per_image,
                     "sofie_hip_conv_i8: the activations are not 16-byte aligned; a workspace of %zu bytes is needed for the column matrix",
                     per_image);
   long long imgs_per_chunk = (long long)(ws_left / per_image);
   // keep one column matrix within reach of the 256 MB last-level cache
   const long long cap = (long long)((192u << 20) / per_image);
   if (imgs_per_chunk > cap)
      imgs_per_chunk = cap > 0 ? cap : 1;
   if (imgs_per_chunk > d->N)
      imgs_per_chunk = d->N;
   SOFIE_HIP_REQUIRE(imgs_per_chunk >= 1, "sofie_hip_conv_i8: workspace too small for one image");
   SOFIE_HIP_REQUIRE(imgs_per_chunk * OHW < (1LL << 31), "sofie_hip_conv_i8: too many rows per chunk");
   const bool fast = a->x_layout == SOFIE_LAYOUT_NHWC && (g.Cg % 16 == 0) && (d->C % 16 == 0) && (((uintptr_t)a->X & 15) == 0);

   for (long long img0 = 0; img0 < d->N; img0 += imgs_per_chunk) {
      const long long imgs = (d->N - img0) < imgs_per_chunk ? (d->N - img0) : imgs_per_chunk;
      const long long rows = imgs * OHW;
      for (int grp = 0; grp < d->group; ++grp) {
         size_t work = (size_t)rows * (g.Kp / 16);
         size_t blocks = (work + 255) / 256;
         if (blocks > 16384)
            blocks = 16384;
         if (fast)
            hipLaunchKernelGGL(im2col_i8_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, (int8_t *)ws, a->X, g,
                               grp * g.Cg, 1, img0 * OHW, rows);
         else
            hipLaunchKernelGGL(im2col_i8_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, (int8_t *)ws, a->X, g,
                               grp * g.Cg, a->x_layout == SOFIE_LAYOUT_NHWC, img0 * OHW, rows);
         st = launch_status("im2col_i8_kernel");
         if (st)
            return st;
         I8Epilogue ep;
         ep.bias = a->bias;
         ep.scale = a->scale;
         ep.scale_scalar = 1.0f;
         ep.q_scale = 1.0f;
         ep.relu_acc = (out_kind == SOFIE_I8OUT_I32) ? a->relu : 0;
         ep.relu_out = (out_kind == SOFIE_I8OUT_I32) ? 0 : a->relu;
         ep.out = out_kind;
         ep.ldy = d->Cout;
         ep.stage_ok = 0;
         ep.vec_param = 0;
         ep.N = Cout_g;
         ep.n_offset = grp * Cout_g;
         if (a->y_layout == SOFIE_LAYOUT_NHWC) {
            ep.nchw_ohw = 0;
            ep.Y = (char *)a->Y + (size_t)img0 * OHW * d->Cout * esz;
         } else {
            ep.nchw_ohw = OHW;
            ep.Y = (char *)a->Y + (size_t)img0 * d->Cout * OHW * esz;
         }
         st = gemm_i8_nt(launch_cfg_i8(ctx), (const int8_t *)ws, Wp + (size_t)grp * Cout_g * g.Kp, (int)rows, Cout_g, g.Kp, g.Kp, g.Kp, ep);
         if (st)
            return st;
      }
   }
   return SOFIE_HIP_OK;
}

} // extern "C"
