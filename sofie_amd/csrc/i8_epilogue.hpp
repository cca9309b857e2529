// Store stage of the int8 GEMM and of the int8 convolution: bias, requantisation or dequantisation,
// optional relu, and the output addressing (row-major [M,N], or NCHW when the GEMM rows are the
// output pixels of a convolution).  Plugs into tile_store_via_lds (mfma8_common.hpp).
#pragma once
#include "exact_quotient.hpp"
#include "mfma8_dispatch.hpp"

namespace sofie_hip {

struct I8Epilogue {
   static constexpr bool kConvertInRegisters = true; // a handful of integer / fp32 instructions per element
   const int32_t *bias;
   const float *scale;
   float scale_scalar;
   float q_scale;
   int relu_acc, relu_out, out;
   void *Y;
   int ldy;
   int stage_ok;  // row-major Y whose rows allow 16-byte stores
   int vec_param; // bias/scale may be read as 16-byte vectors
   int N;         // number of valid columns
   int nchw_ohw;  // 0: Y[m*ldy + n]; else m = (img, pix) and Y[(img*ldy + n)*nchw_ohw + pix], ldy = Cout
   int n_offset;  // added to n for bias/scale/Y addressing (grouped convolution)
   int rows_per_plane = 0; // non-zero (with out = SOFIE_I8OUT_I8): the int8 values of the rows of a plane are added up instead of stored;
                       // Y is int32 [M / rows_per_plane][ldy]
   float q_rcp = 0.0f;     // RN(1 / q_scale) when q_by_rcp is set
   int q_by_rcp = 0;       // SOFIE_I8OUT_I8_DQQ: the quotient is formed with quotient_by_reciprocal (same bits as the division)

   template <class F>
   __device__ __forceinline__ void dispatch(F f) const
   {
      switch (out) {
      case SOFIE_I8OUT_I32: f(std::integral_constant<int, SOFIE_I8OUT_I32>{}); break;
      case SOFIE_I8OUT_F32: f(std::integral_constant<int, SOFIE_I8OUT_F32>{}); break;
      case SOFIE_I8OUT_I8: f(std::integral_constant<int, SOFIE_I8OUT_I8>{}); break;
      default: f(std::integral_constant<int, SOFIE_I8OUT_I8_DQQ>{}); break;
      }
   }
   // The same with a fifth store for SOFIE_I8OUT_I8_DQQ whose quotient may come from the reciprocal.  Only the kernels with
   // registers to spare for one more instance of the store take it (the 256 x 256 tiles have none).
   template <class F>
   __device__ __forceinline__ void dispatch_with_reciprocal(F f) const
   {
      if (out == SOFIE_I8OUT_I8_DQQ && q_by_rcp)
         f(std::integral_constant<int, kOutDqqByRcp>{});
      else
         dispatch(f);
   }
   // The store from registers (the 256 x 256 tile of the persistent kernel, where every instruction per element counts) has
   // SOFIE_I8OUT_I8 twice: with the relu on the accumulator and, kOutI8NoFloor, without that instruction.
   template <class F>
   __device__ __forceinline__ void dispatch_for_registers(F f) const
   {
      if (out == SOFIE_I8OUT_I8 && !relu_acc)
         f(std::integral_constant<int, kOutI8NoFloor>{});
      else
         dispatch(f);
   }
   // store modes of the kernels only: SOFIE_I8OUT_I8_DQQ with the quotient taken through the reciprocal, SOFIE_I8OUT_I8
   // without a relu on the accumulator
   static constexpr int kOutDqqByRcp = 5, kOutI8NoFloor = 6;
   template <int OUT>
   static constexpr bool requantizes()
   {
      return OUT == SOFIE_I8OUT_I8 || OUT == kOutI8NoFloor;
   }
   template <int OUT>
   static constexpr bool divides()
   {
      return OUT == SOFIE_I8OUT_I8_DQQ || OUT == kOutDqqByRcp;
   }
   // (float(acc) * s) / q_scale, correctly rounded
   template <int OUT>
   __device__ __forceinline__ float quotient(float v) const
   {
      if (OUT == kOutDqqByRcp)
         return quotient_by_reciprocal(v, q_scale, q_rcp);
      return __fdiv_rn(v, q_scale);
   }
   template <int OUT>
   static constexpr int out_bytes()
   {
      return (OUT == SOFIE_I8OUT_I32 || OUT == SOFIE_I8OUT_F32) ? 4 : 1;
   }
   static constexpr bool kCanSumRows = true;
   __device__ __forceinline__ bool sums_rows() const { return rows_per_plane != 0; }
   // sums of columns n..n+3 over a wave tile's rows, which start at row m and lie in one plane: integer additions, so the
   // order in which the tiles arrive does not matter
   __device__ __forceinline__ void add_row_sums(int m, int n, int N_, const int (&s)[4]) const
   {
      int *dst = (int *)Y + (size_t)(m / rows_per_plane) * (size_t)ldy + n + n_offset;
#pragma unroll
      for (int e = 0; e < 4; ++e)
         if (n + e < N_)
            atomicAdd(dst + e, s[e]);
   }
   __device__ __forceinline__ bool rows_vectorizable() const { return stage_ok != 0; }
   // row-major output with 16-byte aligned rows, every element stored (what the register tile store handles)
   // (and, for SOFIE_I8OUT_I8_DQQ, a q_scale against which the largest finite float still saturates: see
   // load_column_for_registers)
   bool stores_plain_rows() const
   {
      return stage_ok != 0 && nchw_ohw == 0 && rows_per_plane == 0 && q_scale_saturates();
   }
   // 1-byte elements stored as rows: the store from registers then issues one 16-byte store per lane and 16-row block
   __device__ __forceinline__ bool stores_one_byte_rows() const { return out != SOFIE_I8OUT_I32 && out != SOFIE_I8OUT_F32 && rows_per_plane == 0; }
   // output elements per 16 bytes (the unit of the vector stores)
   int elements_per_16_bytes() const { return (out == SOFIE_I8OUT_I32 || out == SOFIE_I8OUT_F32) ? 4 : 16; }
   bool q_scale_saturates() const { return out != SOFIE_I8OUT_I8_DQQ || (q_scale > -1e30f && q_scale < 1e30f); }
   // plane sums (of int8 results) whose planes are made of whole groups of `rows` GEMM rows
   bool sums_rows_of_whole_wave_tiles(int rows) const
   {
      return rows_per_plane != 0 && rows_per_plane % rows == 0 && (out == SOFIE_I8OUT_I8 || out == SOFIE_I8OUT_I8_DQQ) && nchw_ohw == 0 &&
             q_scale_saturates();
   }
   __device__ __forceinline__ char *out_base() const { return (char *)Y; }
   __device__ __forceinline__ size_t out_index(int m, int n) const
   {
      if (nchw_ohw) {
         const int img = m / nchw_ohw, pix = m - img * nchw_ohw;
         return ((size_t)img * ldy + (n + n_offset)) * nchw_ohw + pix;
      }
      return (size_t)m * (size_t)ldy + n + n_offset;
   }

   // the same for a store that only exists for row-major outputs (stores_plain_rows()): no case to tell apart per element
   __device__ __forceinline__ size_t out_index_of_plain_rows(int m, int n) const { return (size_t)m * (size_t)ldy + n + n_offset; }

   // DequantizeLinear of one accumulator: one fp32 multiply, then max(.,0) if relu_out
   __device__ __forceinline__ float to_f32(int acc, float s) const
   {
      float v = mul_nofma((float)acc, s);
      if (relu_out)
         v = v > 0.0f ? v : 0.0f;
      return v;
   }
   // requantisation: sat8(rne(float(acc)*s)) then relu, or sat8(rne((float(acc)*s)/q_scale))
   template <int OUT>
   __device__ __forceinline__ int to_i8(int acc, float s) const
   {
      if (requantizes<OUT>())
         return quantize_rne_clamp(mul_nofma((float)acc, s), relu_out ? 0 : -128);
      if (OUT == kOutDqqByRcp) // a finite per-tensor scale (the condition of this mode): no NaN to keep out of the short conversion
         return (int)i8_bits(quotient<OUT>(mul_nofma((float)acc, s)), -128.0f);
      return quantize_rne_clamp(quotient<OUT>(mul_nofma((float)acc, s)), -128);
   }

   // bias and scale of C consecutive columns
   template <int C>
   struct col_params {
      int b[C];
      float s[C];
   };
   template <int C>
   __device__ __forceinline__ void load_params(int n, col_params<C> &p) const
   {
      if (vec_param && n + C <= N) {
#pragma unroll
         for (int q = 0; q < C / 4; ++q) {
            v4i b = {0, 0, 0, 0};
            if (bias)
               b = *(const v4i *)(bias + n + n_offset + 4 * q);
            float4 f = make_float4(scale_scalar, scale_scalar, scale_scalar, scale_scalar);
            if (scale)
               f = *(const float4 *)(scale + n + n_offset + 4 * q);
            p.b[4 * q + 0] = b[0], p.b[4 * q + 1] = b[1], p.b[4 * q + 2] = b[2], p.b[4 * q + 3] = b[3];
            p.s[4 * q + 0] = f.x, p.s[4 * q + 1] = f.y, p.s[4 * q + 2] = f.z, p.s[4 * q + 3] = f.w;
         }
      } else {
#pragma unroll
         for (int i = 0; i < C; ++i) {
            const int nn = (n + i < N ? n + i : N - 1) + n_offset;
            p.b[i] = bias ? bias[nn] : 0;
            p.s[i] = scale ? scale[nn] : scale_scalar;
         }
      }
   }

   // The constants of ONE column as 32-bit words (what the register tile store hands from lane to lane): bias, scale.
   static constexpr int kColWords = 2;
   // The persistent kernel starts a tile's accumulators at the bias of their columns (word kBiasWord) instead of zero: the
   // sums are exact integers, so the result is that of adding the bias afterwards, and its store (the template argument
   // BIAS_DONE of the conversions below) saves that addition per element.
   static constexpr bool kBiasInAccumulator = true;
   static constexpr int kBiasWord = 0;
   __device__ __forceinline__ void load_column(int n, uint32_t (&w)[kColWords]) const
   {
      w[0] = (uint32_t)(bias ? bias[n + n_offset] : 0);
      w[1] = __float_as_uint(scale ? scale[n + n_offset] : scale_scalar);
   }
   template <int C>
   static __device__ __forceinline__ void set_column(col_params<C> &p, int i, const uint32_t (&w)[kColWords])
   {
      p.b[i] = (int)w[0];
      p.s[i] = __uint_as_float(w[1]);
   }

   // the int8 results of columns 4q..4q+3 as integers (what the plane sums of a convolution add up), each with kI8BitsBias
   // added (the word i8_bits() returns): sums of such words are taken as they are, modulo 2^32, and the bias is subtracted
   // once per sum instead of once per element
   static constexpr uint32_t kI8BitsBias = 0x4B400000u;
   template <int OUT, int C, bool BIAS_DONE = false>
   __device__ __forceinline__ void quantize4_biased(const col_params<C> &p, int q, int a0, int a1, int a2, int a3, uint32_t (&r)[4]) const
   {
      int acc[4] = {a0, a1, a2, a3};
      int acc_floor = relu_acc ? 0 : (int)0x80000000;
      asm volatile("" : "+s"(acc_floor)); // kept a number (see pack4)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
         if (!BIAS_DONE)
            acc[i] += p.b[4 * q + i];
         if (OUT != kOutI8NoFloor)
            acc[i] = acc[i] > acc_floor ? acc[i] : acc_floor;
         float v = mul_nofma((float)acc[i], p.s[4 * q + i]);
         if (divides<OUT>())
            v = quotient<OUT>(v);
         r[i] = i8_bits(v, (requantizes<OUT>() && relu_out) ? 0.0f : -128.0f); // needs the tamed scale, like pack4_short
      }
   }

   // sat8(rne(v)), clamped below at lo (-128, or 0 when a relu follows): the low byte of the returned word.  v is clamped to
   // [lo, 127] first (the bounds are integers: clamping commutes with the rounding), then 1.5 * 2^23 is added: the sum lies
   // in [2^23, 2^24), where floats are the integers, so the addition itself rounds to the nearest integer, ties to even (the
   // constant is even), and leaves that integer in the low mantissa bits.  Two instructions instead of the four of
   // quantize_rne_clamp.  NaN is clamped to lo by v_med3_f32 where quantize_rne_clamp gives 0: the caller keeps NaN out.
   static __device__ __forceinline__ uint32_t i8_bits(float v, float lo)
   {
      const float c = __builtin_amdgcn_fmed3f(v, lo, 127.0f);
      return __float_as_uint(c + 12582912.0f);
   }
   // One element of pack4_short: bias (unless it sits in the accumulator), floor, scale, quotient, clamp to [lo, 127].
   template <int OUT, bool BIAS_DONE>
   __device__ __forceinline__ float clamp1_short(int acc, int b, float s) const
   {
      static_assert(requantizes<OUT>() || divides<OUT>(), "1-byte outputs");
      int acc_floor = relu_acc ? 0 : (int)0x80000000;
      asm volatile("" : "+s"(acc_floor)); // kept a number (see pack4)
      const float lo = (requantizes<OUT>() && relu_out) ? 0.0f : -128.0f;
      if (!BIAS_DONE)
         acc += b;
      if (OUT != kOutI8NoFloor)
         acc = acc > acc_floor ? acc : acc_floor;
      float v = mul_nofma((float)acc, s);
      if (divides<OUT>())
         v = quotient<OUT>(v);
      return __builtin_amdgcn_fmed3f(v, lo, 127.0f);
   }
   // i8_bits() of a clamped element, the addition writing its low byte straight into byte K of the dword (sub-dword
   // destination select): no byte permutes.  K = 0 starts the dword.
   template <int K>
   static __device__ __forceinline__ void place_i8_byte(uint32_t &r, float c)
   {
      const float magic = 12582912.0f;
      if constexpr (K == 0)
         asm("v_add_f32_sdwa %0, %1, %2 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:DWORD" : "=v"(r) : "v"(c), "v"(magic));
      else if constexpr (K == 1)
         asm("v_add_f32_sdwa %0, %1, %2 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD" : "+v"(r) : "v"(c), "v"(magic));
      else if constexpr (K == 2)
         asm("v_add_f32_sdwa %0, %1, %2 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD" : "+v"(r) : "v"(c), "v"(magic));
      else
         asm("v_add_f32_sdwa %0, %1, %2 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD" : "+v"(r) : "v"(c), "v"(magic));
   }
   // pack4 for the 1-byte outputs with the short conversion.  float(acc) * s is NaN only for a scale that is NaN, or
   // infinite against an accumulator of 0; load_column_for_registers() below replaces such scales by ones that give the same results
   // without NaN.
   template <int OUT, int C, bool BIAS_DONE = false>
   __device__ __forceinline__ void pack4_short(const col_params<C> &p, int q, int a0, int a1, int a2, int a3, uint32_t *w) const
   {
      const float c0 = clamp1_short<OUT, BIAS_DONE>(a0, p.b[4 * q + 0], p.s[4 * q + 0]);
      const float c1 = clamp1_short<OUT, BIAS_DONE>(a1, p.b[4 * q + 1], p.s[4 * q + 1]);
      const float c2 = clamp1_short<OUT, BIAS_DONE>(a2, p.b[4 * q + 2], p.s[4 * q + 2]);
      const float c3 = clamp1_short<OUT, BIAS_DONE>(a3, p.b[4 * q + 3], p.s[4 * q + 3]);
      uint32_t r;
      place_i8_byte<0>(r, c0);
      place_i8_byte<1>(r, c1);
      place_i8_byte<2>(r, c2);
      place_i8_byte<3>(r, c3);
      w[0] = r;
   }
   // load_column for the store from registers.  Its 1-byte conversions (pack4_short, quantize4) need the scale made safe:
   // NaN becomes 0 and +-inf the largest finite number.  The results are those of the plain scale: a NaN product is stored
   // as 0, and so is 0 * s; a non-zero accumulator times +-inf saturates like one times +-FLT_MAX (for SOFIE_I8OUT_I8_DQQ
   // as long as FLT_MAX / q_scale still saturates: stores_plain_rows() keeps larger q_scale away from this store).  The
   // 4-byte outputs keep the scale as it is: they hand NaN and infinities on.
   __device__ __forceinline__ void load_column_for_registers(int n, uint32_t (&w)[kColWords]) const
   {
      load_column(n, w);
      float s = __uint_as_float(w[1]);
      float t = (s == s) ? s : 0.0f;
      t = __builtin_amdgcn_fmed3f(t, -3.402823466e38f, 3.402823466e38f);
      w[1] = __float_as_uint((out == SOFIE_I8OUT_I32 || out == SOFIE_I8OUT_F32) ? s : t);
   }

   // converts columns 4q..4q+3 of the lane's columns (exact int32 dot products) into 4*out_bytes() bytes
   template <int OUT, int C, bool BIAS_DONE = false>
   __device__ __forceinline__ void pack4(const col_params<C> &p, int q, int a0, int a1, int a2, int a3, uint32_t *w) const
   {
      static_assert(OUT != kOutI8NoFloor, "the store without a floor on the accumulator exists for the short conversion only");
      int acc[4] = {a0, a1, a2, a3};
      float s[4];
      int acc_floor = relu_acc ? 0 : (int)0x80000000; // relu on the accumulator as one max
      asm volatile("" : "+s"(acc_floor));              // kept a number: as a known pair of cases it becomes a max AND a select per element
#pragma unroll
      for (int i = 0; i < 4; ++i) {
         if (!BIAS_DONE)
            acc[i] += p.b[4 * q + i];
         s[i] = p.s[4 * q + i];
         acc[i] = acc[i] > acc_floor ? acc[i] : acc_floor;
      }
      if (OUT == SOFIE_I8OUT_I32) {
#pragma unroll
         for (int i = 0; i < 4; ++i)
            w[i] = (uint32_t)acc[i];
      } else if (OUT == SOFIE_I8OUT_F32) {
#pragma unroll
         for (int i = 0; i < 4; ++i)
            w[i] = __float_as_uint(to_f32(acc[i], s[i]));
      } else {
         const int q0 = to_i8<OUT>(acc[0], s[0]), q1 = to_i8<OUT>(acc[1], s[1]), q2 = to_i8<OUT>(acc[2], s[2]),
                   q3 = to_i8<OUT>(acc[3], s[3]);
         // low bytes of q0..q3 into one dword: three byte permutes
         const uint32_t lo = __builtin_amdgcn_perm((uint32_t)q1, (uint32_t)q0, 0x0c0c0400u);
         const uint32_t hi = __builtin_amdgcn_perm((uint32_t)q3, (uint32_t)q2, 0x0c0c0400u);
         w[0] = __builtin_amdgcn_perm(hi, lo, 0x05040100u);
      }
   }
};

// Y = epilogue(A[M,K] * Bt[N,K]^T); fills the derived fields of ep.
int gemm_i8_nt(const LaunchCfg &lc, const int8_t *A, const int8_t *Bt, int M, int N, int K, int lda, int ldb, I8Epilogue ep);
// Convolution whose whole reduction fits one 64-byte slab (few input channels): rows gathered byte by byte, one launch.
int conv_i8_gather(const LaunchCfg &lc, const GatherConvRows &src, const int8_t *Wp, int M, int N, int Kp, I8Epilogue ep);
// The same for NCHW input with stride and dilation 1 in x, 64 output channels and rows stored as they are: windows of four
// bytes instead of single bytes.  *taken tells whether the shape was this kernel's (else nothing was launched).
int conv_i8_few_channels(const LaunchCfg &lc, const FewChannelConv &src, const int8_t *Wp, int M, int N, int Kp, I8Epilogue ep, bool *taken);
// Convolution as an implicit GEMM: rows of A come from `src`, Wp is [N][K] with K = taps * Cg.
int conv_i8_implicit(const LaunchCfg &lc, const ConvRows &src, int Cg, const int8_t *Wp, int M, int N, int K, I8Epilogue ep);

} // namespace sofie_hip
