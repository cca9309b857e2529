// Pieces shared by the int8 / FP8 matrix-core GEMM kernels: MFMA wrappers, the workgroup -> tile map,
// the swizzled LDS slab layout and the tile store through LDS.
#pragma once
#include "common.hpp"
#include <type_traits>
#include <utility>

namespace sofie_hip {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

// Compile-time loop: f(std::integral_constant<int,0>{}), ..., f(std::integral_constant<int,N-1>{}).
// Accumulator registers can only be named with compile-time indices; a run-time index would push the
// whole accumulator array out of the register file.
template <class F, int... Is>
__device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, Is...>)
{
   (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F &&f)
{
   static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// int8: v_mfma_i32_32x32x32_i8, 16 bytes of K per lane and step.
struct MfmaI8 {
   typedef v16i acc_t;
   typedef int elem_t;
   static constexpr int KSTEP = 32; // K bytes per MFMA
   static constexpr int CHUNKS = 1; // 16-byte chunks per lane and operand
   static constexpr int ROWS = 32;  // rows (and columns) of the output block; lane = lk * ROWS + row
   static constexpr int LK = 2;     // lanes that share a row
   static constexpr int ACC = 16;   // accumulator registers per lane
   struct frag_t {
      v4i c[1];
   };
   static __device__ __forceinline__ acc_t mma(const frag_t &a, const frag_t &b, acc_t c)
   {
      return __builtin_amdgcn_mfma_i32_32x32x32_i8(a.c[0], b.c[0], c, 0, 0, 0);
   }
};

// int8 with 16 x 16 output blocks: v_mfma_i32_16x16x64_i8, 16 bytes of K per lane and step, four lanes per row.  Per multiply-add
// it moves half as many accumulator registers as the 32 x 32 form; under the board's power limit (operands that toggle)
// it sustains about a sixth more, provided two waves share the SIMD (one wave alone cannot issue it back to back).
struct MfmaI8x16 {
   typedef v4i acc_t;
   typedef int elem_t;
   static constexpr int KSTEP = 64;
   static constexpr int CHUNKS = 1;
   static constexpr int ROWS = 16;
   static constexpr int LK = 4;
   static constexpr int ACC = 4;
   // XOR applied to the chunk index of row r in a slab of 64-byte rows so that this instruction's fragment read (lane = lk*16 + row,
   // chunk lk) is free of bank conflicts: measured 240 B/clk per CU against 126 B/clk with the (r/4)%4 of the 32-row fragments
   static __device__ __forceinline__ int lds_swizzle(int r) { return (r >> 1) & 3; }
   static constexpr bool kColumnsOutside = true; // order of a step's MFMAs in the persistent kernel
   struct frag_t {
      v4i c[1];
   };
   static __device__ __forceinline__ acc_t mma(const frag_t &a, const frag_t &b, acc_t c)
   {
      return __builtin_amdgcn_mfma_i32_16x16x64_i8(a.c[0], b.c[0], c, 0, 0, 0);
   }
};

// FP8 e4m3fn: v_mfma_f32_32x32x64_f8f6f4 (format code 0 = e4m3 for both operands, no block scaling),
// 32 bytes of K per lane and step.
struct MfmaF8 {
   typedef v16f acc_t;
   typedef float elem_t;
   static constexpr int KSTEP = 64;
   static constexpr int CHUNKS = 2;
   static constexpr int ROWS = 32;
   static constexpr int LK = 2;
   static constexpr int ACC = 16;
   // chunk XOR of row r in 64-byte LDS rows: conflict-free for this fragment (lane = lk*32 + row, chunks 2*lk and 2*lk + 1)
   static __device__ __forceinline__ int lds_swizzle(int r) { return (r >> 2) & 3; }
   static constexpr bool kColumnsOutside = false;
   struct frag_t {
      v4i c[2];
   };
   static __device__ __forceinline__ acc_t mma(const frag_t &a, const frag_t &b, acc_t c)
   {
      v8i va = {a.c[0][0], a.c[0][1], a.c[0][2], a.c[0][3], a.c[1][0], a.c[1][1], a.c[1][2], a.c[1][3]};
      v8i vb = {b.c[0][0], b.c[0][1], b.c[0][2], b.c[0][3], b.c[1][0], b.c[1][1], b.c[1][2], b.c[1][3]};
      return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(va, vb, c, 0, 0, 0, 0, 0, 0);
   }
};

// Maps the hardware workgroup id to an output tile.  Workgroups are dealt round-robin to the 8 XCDs,
// each with its own L2: ids that land on one XCD are made consecutive, and consecutive ids walk the
// tile grid in bands of `mode & 0xff` tile rows (0: plain row-major order), so the tiles resident on one
// XCD at a time share A and Bt slabs through that XCD's L2.  mode & 0x100 skips the XCD regrouping.
__device__ __forceinline__ void tile_of_block(int bid, int nwg, int tiles_m, int tiles_n, int mode, int &tm, int &tn)
{
   constexpr int NXCD = 8;
   int id = bid;
   if (!(mode & 0x100)) {
      const int per = nwg / NXCD, rem = nwg % NXCD;
      const int xcd = bid % NXCD, local = bid / NXCD;
      id = (xcd < rem ? xcd * (per + 1) : rem * (per + 1) + (xcd - rem) * per) + local;
   }
   const int gm = mode & 0xff;
   if (gm == 0) {
      tm = id / tiles_n;
      tn = id % tiles_n;
      return;
   }
   const int width = gm * tiles_n;
   const int group = id / width;
   const int first_m = group * gm;
   const int gsz = (tiles_m - first_m) < gm ? (tiles_m - first_m) : gm;
   tm = first_m + (id % width) % gsz;
   tn = (id % width) / gsz;
}

// Byte offset of 16-byte chunk c of row r in an LDS slab of BK-byte rows.  Chunk c is stored at chunk
// position c ^ ((r / rows_per_256B) % chunks_per_row): the 16 lanes served together by one ds_read_b128
// (16 consecutive rows, same logical chunk) then fall into 16 different 16-byte bank groups.
template <int BK>
__device__ __forceinline__ int lds_chunk_offset(int r, int c)
{
   constexpr int CPR = BK / 16;
   constexpr int RPB = (256 / BK) > 0 ? (256 / BK) : 1;
   return r * BK + (((c ^ ((r / RPB) % CPR))) << 4);
}

// Plain row-major operand: row r starts at base + r*ld.
// The pipelined kernels address an operand through three hooks, so that the A operand can also be a
// convolution input that is never laid out as a matrix (ConvRows below):
//   lane_state<LD>            what a lane keeps per load instruction of a slab
//   init(st, i, m0, row, cbyte, M)   load i of this lane fills tile row `row` with the 16 bytes at slab offset cbyte
//   load_ptr(st, i, koff)     global address of those bytes for the slab that starts at reduction offset koff
struct RowMajorRows {
   static constexpr bool kGather = false;
   const int8_t *base;
   int ld;
   __device__ __forceinline__ const int8_t *row(int r) const { return base + (size_t)r * (size_t)ld; }

   template <int LD>
   struct lane_state {
      const int8_t *tile; // uniform: first row of the tile
      uint32_t off[LD];
   };
   template <int LD>
   __device__ __forceinline__ void init(lane_state<LD> &st, int i, int m0, int row, int cbyte, int M) const
   {
      st.tile = this->row(m0);
      const int rc = (m0 + row < M) ? row : M - 1 - m0; // rows past the edge re-read the last row
      st.off[i] = (uint32_t)rc * (uint32_t)ld + (uint32_t)cbyte;
   }
   template <int LD>
   __device__ __forceinline__ const int8_t *load_ptr(const lane_state<LD> &st, int i, int koff) const
   {
      return (st.tile + koff) + st.off[i];
   }
};

// Rows of a convolution over few input channels (an RGB image: K = 3 * 3 * 3 = 27): GEMM row = output pixel, K = (tap, channel),
// K <= 64, so one 64-byte slab holds the whole reduction.  A lane gathers the bytes of ITS pixel one k at a time; for a
// given k the 64 lanes of a wave read 64 neighbouring pixels, i.e. (almost) consecutive bytes of one input plane.  The
// per-k offsets are tables in the kernel arguments, indexed by compile-time constants after unrolling.
struct GatherConvRows {
   static constexpr bool kGather = true;
   const int8_t *X;
   int H, W, OH, OW, stride_h, stride_w, pad_h0, pad_w0;
   int pix_mul;          // elements between horizontally adjacent pixels: 1 (NCHW) or C (NHWC)
   long long img_stride; // elements per image
   int K;
   int koff[64];         // offset of (channel, ky, kx) from the pixel at (ih0, iw0)
   signed char dy[64], dx[64];
   struct row_ref {
      const int8_t *origin; // address of channel 0 at (ih0, iw0); only dereferenced where the tap lies inside the image
      int ih0, iw0;
   };
   __device__ __forceinline__ row_ref ref_of(int m, int M) const
   {
      const int r = m < M ? m : M - 1; // rows past the edge re-read the last row (their outputs are not stored)
      const int ohw = OH * OW;
      const int img = r / ohw, rem = r - img * ohw;
      const int oh = rem / OW, ow = rem - oh * OW;
      row_ref f;
      f.ih0 = oh * stride_h - pad_h0;
      f.iw0 = ow * stride_w - pad_w0;
      f.origin = X + (long long)img * img_stride + ((long long)f.ih0 * W + f.iw0) * pix_mul;
      return f;
   }
};
// The same with the padded reduction length (16, 32, 48 or 64) as a compile-time constant: the gather loop has no
// run-time bounds.  Entries from K up to KP are padding and read as zero.
template <int KP>
struct GatherConvRowsT : GatherConvRows {
   static constexpr int kKP = KP;
};

// The geometry of a convolution over few input channels whose NCHW input is read window by window (conv_i8_few_channels.hpp).
struct FewChannelConv {
   const int8_t *X;      // NCHW, first channel of the group
   int H, W, OH, OW;
   int stride_h, pad_h0, pad_w0, dil_h;
   int kh, kw, Cg;
   long long img_stride; // bytes per image: all channels
   unsigned char pair_c[16], pair_ky[16]; // channel and row of taps of (channel, ky) pair p = channel * kh + ky (filled in by the launcher)
};

// 256 zero bytes: what a load of a padded (out-of-image) position reads.
static __device__ __attribute__((aligned(256))) int8_t conv_zero_page[256] = {};

// A operand of a convolution computed as one GEMM over the whole batch, read straight from the NHWC
// activation tensor: GEMM row m is the output pixel (n, oh, ow), the reduction index is
// k = (tap kh_i*kw + kw_i) * Cg + channel, so a K slab of BK <= Cg bytes is BK consecutive channels of ONE input pixel.
// Positions outside the image read zeros.  Needs Cg (channels per group) to be a power of two >= BK.
struct ConvRows {
   const int8_t *X;       // NHWC, first channel of the group
   int H, W, C;           // C = channel stride of a pixel (all groups)
   int OH, OW;
   int stride_h, stride_w, pad_h0, pad_w0, dil_h, dil_w;
   int kw, ntaps;
   int cg_shift;          // log2(Cg)
   int kw_recip;          // ceil(65536 / kw): tap / kw == (tap * kw_recip) >> 16 for every tap < ntaps (checked on the host)
   // m / (OH*OW) and r / OW by multiplication: floor(m / d) == (m * ceil(2^64 / d)) >> 64 for every 32-bit m
   // (the error of the rounded-up reciprocal, < m / 2^64 * d... < 2^-32, cannot reach the next integer)
   unsigned long long ohw_mul, ow_mul;

   template <int LD>
   struct lane_state {
      int32_t off[LD];   // byte offset of (n, oh*stride - pad, ow*stride - pad, cbyte) from X; may be negative
      uint32_t mask[LD]; // bit t: tap t of this output pixel lies inside the image
   };
   template <int LD>
   __device__ __forceinline__ void init(lane_state<LD> &st, int i, int m0, int row, int cbyte, int M) const
   {
      const int m = m0 + row;
      uint32_t mask = 0;
      int32_t off = 0;
      if (m < M) {
         const int ohw = OH * OW;
         const int n = ohw_mul ? (int)__umul64hi((unsigned long long)(unsigned)m, ohw_mul) : m; // 0 marks a divisor of 1
         const int r = m - n * ohw;
         const int oh = ow_mul ? (int)__umul64hi((unsigned long long)(unsigned)r, ow_mul) : r;
         const int ow = r - oh * OW;
         const int ih0 = oh * stride_h - pad_h0, iw0 = ow * stride_w - pad_w0;
         off = ((n * H + ih0) * W + iw0) * C + cbyte;
         // tap t = khi * kw + kwi lies inside when its row and its column do: one pass over the columns, one over the rows
         uint32_t cols = 0;
         for (int kwi = 0, iw = iw0; kwi < kw; ++kwi, iw += dil_w)
            cols |= ((unsigned)iw < (unsigned)W ? 1u : 0u) << kwi;
         for (int t0 = 0, ih = ih0; t0 < ntaps; t0 += kw, ih += dil_h)
            mask |= ((unsigned)ih < (unsigned)H ? cols : 0u) << t0;
      }
      st.off[i] = off;
      st.mask[i] = mask;
   }
   template <int LD>
   __device__ __forceinline__ const int8_t *load_ptr(const lane_state<LD> &st, int i, int koff) const
   {
      const int tap = koff >> cg_shift;            // uniform
      const int cbyte = koff & ((1 << cg_shift) - 1);
      const int khi = (tap * kw_recip) >> 16, kwi = tap - khi * kw;
      const int toff = (khi * dil_h * W + kwi * dil_w) * C + cbyte;
      const int8_t *p = X + (ptrdiff_t)(st.off[i] + toff);
      return ((st.mask[i] >> tap) & 1u) ? p : (const int8_t *)conv_zero_page;
   }
};

// Can epilogue EPI add the rows of a tile up instead of storing them?  (EPI::kCanSumRows, if the epilogue has it.)
template <class EPI, class = void>
struct epi_can_sum_rows : std::false_type {};
template <class EPI>
struct epi_can_sum_rows<EPI, std::enable_if_t<EPI::kCanSumRows>> : std::true_type {};

// LDS bytes one wave needs for the tile store below (TN = columns of the wave tile).
constexpr int tile_store_lds_bytes(int TN) { return 32 * (TN * 4 + 16); }

// Tile store through LDS.  After the MFMAs a lane holds, per register group, 4 consecutive columns of
// ONE row, and the 32 lanes of a half-wave hold 32 different rows; stored directly, a wave instruction
// would touch 64 rows with 4..16 bytes each.  Instead, for each 32-row block of its tile, a wave
//   1. converts its accumulators in registers (straight-line code, one pack4 per register group: bias,
//      scale, rounding, activation, narrowing), which leaves 4 output elements = 4, 8 or 16 bytes,
//   2. parks those bytes in its own LDS region, laid out as the output rows (row stride TN*ESZ+16 bytes),
//   3. re-reads the region 16 bytes per lane, a row being covered by consecutive lanes, and stores: a wave
//      instruction then writes whole 128-byte lines.
// Converting before the transposition keeps the LDS traffic at the size of the OUTPUT (a quarter of the
// accumulators for 1-byte outputs) and leaves nothing but a copy in the run-time loop of step 3.
//
// EPI provides
//   template <class F> void dispatch(F f) const     f(std::integral_constant<int, MODE>{}) for the output mode
//   template <int MODE> static constexpr int out_bytes()          bytes of one output element (1, 2, 4)
//   struct col_params<C>; template <int C> void load_params(int n, col_params<C> &p) const
//                                per-column constants (bias, scale) of columns n..n+C-1, clamped to N-1
//   template <int MODE, int C> void pack4(const col_params<C> &p, int q, T a0, T a1, T a2, T a3, uint32_t *w) const
//                                converts columns 4q..4q+3 of the C columns into 4*out_bytes bytes
//   bool rows_vectorizable() const                row-major output whose rows allow 16-byte stores
//   char *out_base() const;  size_t out_index(int m, int n) const     element index of (m,n)
template <int MODE, int MT, int NT, class EPI, class ACC>
__device__ __forceinline__ void tile_store_convert_first(const EPI &ep, ACC (&acc)[MT][NT], int m_base, int n_base, int M, int N,
                                                        int lane, char *wsm)
{
   constexpr int ESZ = EPI::template out_bytes<MODE>();
   constexpr int TN = NT * 32;
   constexpr int ROWB = TN * ESZ + 16; // 16-byte aligned rows, consecutive rows shifted over the banks
   constexpr int QW = ESZ;             // dwords produced per group of 4 columns
   const int lr = lane & 31, lk = lane >> 5;
   char *out = ep.out_base();
   const bool vec = ep.rows_vectorizable();

   // Row sums (an epilogue that can, asked at run time, 1-byte elements): instead of storing the converted elements, the wave
   // adds them up column by column over all MT * 32 rows of its tile (the caller guarantees that those rows are valid and
   // belong to one plane) and hands the epilogue 4 column sums per lane.  A lane takes dword `sum_dw` of every RG-th row of
   // the parked block.
   constexpr int DPR = TN / 4;                         // dwords per parked row
   constexpr int RG = (64 / DPR) > 0 ? (64 / DPR) : 1; // rows read per pass
   constexpr bool CAN_SUM = epi_can_sum_rows<EPI>::value && ESZ == 1 && DPR <= 64 && 64 % DPR == 0 && 32 % RG == 0;
   bool sums = false;
   if constexpr (CAN_SUM)
      sums = ep.sums_rows();
   const int sum_dw = lane % DPR, sum_rg = lane / DPR;
   int colsum[4] = {0, 0, 0, 0};

   // the lane's columns are the same in every 32-row block: their constants are fetched once
   typename EPI::template col_params<4> prm[NT][4];
   static_for<NT>([&](auto cj) {
      constexpr int j = decltype(cj)::value;
      static_for<4>([&](auto cg) {
         constexpr int g = decltype(cg)::value;
         const int n = n_base + j * 32 + g * 8 + lk * 4;
         ep.template load_params<4>(n < N ? n : N - 1, prm[j][g]);
      });
   });

   static_for<MT>([&](auto ci) {
      constexpr int i = decltype(ci)::value;
      static_for<NT>([&](auto cj) {
         constexpr int j = decltype(cj)::value;
         static_for<4>([&](auto cg) {
            constexpr int g = decltype(cg)::value;
            uint32_t w[QW];
            ep.template pack4<MODE, 4>(prm[j][g], 0, acc[i][j][4 * g + 0], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2],
                                       acc[i][j][4 * g + 3], w);
            char *dst = wsm + lr * ROWB + (j * 32 + g * 8 + lk * 4) * ESZ;
            if constexpr (QW == 1)
               *(uint32_t *)dst = w[0];
            else if constexpr (QW == 2)
               *(uint2 *)dst = make_uint2(w[0], w[1]);
            else
               *(uint4 *)dst = make_uint4(w[0], w[1], w[2], w[3]);
         });
      });
      __builtin_amdgcn_wave_barrier();
      const int m_first = m_base + i * 32;
      if (CAN_SUM && sums) {
#pragma unroll 4
         for (int row = sum_rg; row < 32; row += RG) {
            const int v = *(const int *)(wsm + row * ROWB + sum_dw * 4);
            colsum[0] += (v << 24) >> 24;
            colsum[1] += (v << 16) >> 24;
            colsum[2] += (v << 8) >> 24;
            colsum[3] += v >> 24;
         }
      } else if (vec) {
         constexpr int CPL = 16 / ESZ;          // columns per lane
         constexpr int LPR = TN / CPL;          // lanes per row
         constexpr int RPP = 64 / LPR;          // rows per pass
         static_assert(TN % CPL == 0 && LPR <= 64 && 32 % RPP == 0, "wave tile width not supported by the tile store");
         const int c0 = (lane % LPR) * CPL;
         const int n = n_base + c0;
#pragma unroll 2
         for (int row0 = 0; row0 < 32; row0 += RPP) {
            const int row = row0 + lane / LPR;
            const int m = m_first + row;
            const uint4 v = *(const uint4 *)(wsm + row * ROWB + c0 * ESZ);
            if (m < M && n < N) {
               char *y = out + ep.out_index(m, n) * ESZ;
               if (n + CPL <= N) {
                  *(uint4 *)y = v;
               } else {
                  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
                  for (int b = 0; b < (N - n) * ESZ; ++b)
                     y[b] = (char)(w[b >> 2] >> ((b & 3) * 8));
               }
            }
         }
      } else {
         // any layout: a lane takes 4 columns of a row and stores them one element at a time
         constexpr int LPR = TN / 4;
         constexpr int RPP = (64 / LPR) > 0 ? (64 / LPR) : 1;
         static_assert(LPR <= 64, "wave tile too wide");
         const int c0 = (lane % LPR) * 4;
         const int n = n_base + c0;
#pragma unroll 1
         for (int row0 = 0; row0 < 32; row0 += RPP) {
            const int row = row0 + lane / LPR;
            const int m = m_first + row;
            if (m < M && n < N) {
               const char *src = wsm + row * ROWB + c0 * ESZ;
               for (int e = 0; e < 4 && n + e < N; ++e) {
                  char *y = out + ep.out_index(m, n + e) * ESZ;
                  if constexpr (ESZ == 1)
                     y[0] = src[e];
                  else if constexpr (ESZ == 2)
                     *(uint16_t *)y = *(const uint16_t *)(src + 2 * e);
                  else
                     *(uint32_t *)y = *(const uint32_t *)(src + 4 * e);
               }
            }
         }
      }
      __builtin_amdgcn_wave_barrier();
   });
   if constexpr (CAN_SUM) {
      if (sums) {
         // lanes that share a dword column hold the sums of different rows: fold them onto the lanes of row group 0
#pragma unroll
         for (int d = DPR; d < 64; d *= 2)
#pragma unroll
            for (int e = 0; e < 4; ++e)
               colsum[e] += __shfl_xor(colsum[e], d, 64);
         if (sum_rg == 0)
            ep.add_row_sums(m_base, n_base + sum_dw * 4, N, colsum);
      }
   }
}

// The other order, for stores whose conversion is long (an erf per element): the raw 32-bit accumulators are parked and
// the conversion runs in the run-time loop of the re-read, so its code exists once instead of once per accumulator
// register.  (Unrolled over the 256 accumulators of a 256 x 256 tile, a GELU store is 80 KB of straight-line code that
// is executed once per tile: every instruction is an instruction-cache miss.)
template <int MODE, int MT, int NT, class EPI, class ACC>
__device__ __forceinline__ void tile_store_convert_after(const EPI &ep, ACC (&acc)[MT][NT], int m_base, int n_base, int M, int N,
                                                   int lane, char *wsm)
{
   typedef typename std::remove_reference<decltype(acc[0][0][0])>::type elem_t;
   constexpr int ESZ = EPI::template out_bytes<MODE>();
   constexpr int TN = NT * 32;
   constexpr int ROWB = TN * 4 + 16;
   const int lr = lane & 31, lk = lane >> 5;
   char *out = ep.out_base();
   const bool vec = ep.rows_vectorizable();
   static_for<MT>([&](auto ci) {
      constexpr int i = decltype(ci)::value;
      static_for<NT>([&](auto cj) {
         constexpr int j = decltype(cj)::value;
         static_for<4>([&](auto cg) {
            constexpr int g = decltype(cg)::value;
            typedef elem_t v4e __attribute__((ext_vector_type(4)));
            *(v4e *)(wsm + lr * ROWB + (j * 32 + g * 8 + lk * 4) * 4) =
               v4e{acc[i][j][4 * g + 0], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
         });
      });
      __builtin_amdgcn_wave_barrier();
      const int m_first = m_base + i * 32;
      if (vec) {
         constexpr int CPL = 16 / ESZ;     // columns per lane
         constexpr int LPR = TN / CPL;     // lanes per row
         constexpr int RPP = 64 / LPR;     // rows per pass
         static_assert(TN % CPL == 0 && LPR <= 64 && 32 % RPP == 0, "wave tile width not supported by the tile store");
         const int c0 = (lane % LPR) * CPL;
         const int n = n_base + c0;
         typename EPI::template col_params<CPL> prm;
         ep.template load_params<CPL>(n < N ? n : N - 1, prm);
#pragma unroll 1
         for (int row0 = 0; row0 < 32; row0 += RPP) {
            const int row = row0 + lane / LPR;
            const int m = m_first + row;
            if (m < M && n < N) {
               uint32_t w[4];
#pragma unroll
               for (int q = 0; q < CPL / 4; ++q) {
                  typedef elem_t v4e __attribute__((ext_vector_type(4)));
                  const v4e a = *(const v4e *)(wsm + row * ROWB + (c0 + 4 * q) * 4);
                  ep.template pack4<MODE, CPL>(prm, q, a[0], a[1], a[2], a[3], w + q * ESZ);
               }
               char *y = out + ep.out_index(m, n) * ESZ;
               if (n + CPL <= N) {
                  *(uint4 *)y = make_uint4(w[0], w[1], w[2], w[3]);
               } else {
                  const char *src = (const char *)w;
                  for (int b = 0; b < (N - n) * ESZ; ++b)
                     y[b] = src[b];
               }
            }
         }
      } else {
         // any layout: a lane converts 4 columns and stores them one element at a time
         constexpr int LPR = TN / 4;
         constexpr int RPP = (64 / LPR) > 0 ? (64 / LPR) : 1;
         static_assert(LPR <= 64, "wave tile too wide");
         const int c0 = (lane % LPR) * 4;
         const int n = n_base + c0;
         typename EPI::template col_params<4> prm;
         ep.template load_params<4>(n < N ? n : N - 1, prm);
#pragma unroll 1
         for (int row0 = 0; row0 < 32; row0 += RPP) {
            const int row = row0 + lane / LPR;
            const int m = m_first + row;
            if (m < M && n < N) {
               typedef elem_t v4e __attribute__((ext_vector_type(4)));
               const v4e a = *(const v4e *)(wsm + row * ROWB + c0 * 4);
               uint32_t w[4];
               ep.template pack4<MODE, 4>(prm, 0, a[0], a[1], a[2], a[3], w);
               const char *src = (const char *)w;
               for (int e = 0; e < 4 && n + e < N; ++e) {
                  char *y = out + ep.out_index(m, n + e) * ESZ;
                  for (int b = 0; b < ESZ; ++b)
                     y[b] = src[e * ESZ + b];
               }
            }
         }
      }
      __builtin_amdgcn_wave_barrier();
   });
}


// EPI::kConvertInRegisters picks the order: true for the short integer conversions, false for long ones.
template <int MODE, int MT, int NT, class EPI, class ACC>
__device__ __forceinline__ void tile_store_via_lds(const EPI &ep, ACC (&acc)[MT][NT], int m_base, int n_base, int M, int N,
                                                   int lane, char *wsm)
{
   if constexpr (EPI::kConvertInRegisters)
      tile_store_convert_first<MODE, MT, NT>(ep, acc, m_base, n_base, M, N, lane, wsm);
   else
      tile_store_convert_after<MODE, MT, NT>(ep, acc, m_base, n_base, M, N, lane, wsm);
}

int transpose_i8(hipStream_t stream, int8_t *dst, const int8_t *src, int rows, int cols, int ld_src, int ld_dst);

} // namespace sofie_hip
