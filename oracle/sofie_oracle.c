/* sofie_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A plain-C, CPU restatement of the reference's (ML4EP/SOFIE 1.0.1) generated inference code for
 * the Gemm / Conv / epilogue / memory-plan path, plus the frozen definitions of the quantised
 * operators the reference does not have.  Only the tests, the smoke check and the benchmark's
 * cpu_baseline leg may load this library, and only as the checker.  The HIP runtime never calls it.
 *
 * Build: see oracle/Makefile (gcc -O2 -ffp-contract=off: no fused multiply-add may be formed, so
 * that every fp32 operation rounds exactly as written).
 *
 * What pins each function (tests/test_oracle_*.py):
 *   gemm_f32 / gemm_call      golden outputs Linear_16/32/64, LinearWithSigmoid, LinearWithLeakyRelu
 *                             of the reference's own tests; literal cases of its constant-folding
 *                             tests; float64 brute force.
 *   im2col / conv_f32         golden outputs of the reference's 18 Conv* fixtures; 7-loop direct
 *                             convolution in float64.
 *   relu/sigmoid/gelu/...     Gelu / GeluTanh / LinearWithSelu golden outputs; closed forms.
 *   basic_unary, unary_chain  numpy's float32 routines (an independent implementation) and identities
 *                             (exp(log x) = x, sin^2 + cos^2 = 1, sinh(asinh x) = x, ...); Clip bounds; the golden
 *                             outputs Sqrt, Reciprocal, Exp, Log, Neg, Elu, SeluNonDefaultCoeffs, LinearWithSelu of the
 *                             reference's tests; Erf against scipy's erf.
 *   binary_broadcast          Add, AddBroadcast1..7, Sub, Mul, Div, Pow, Pow_broadcast and the Max / Min / Mean / Sum
 *                             MultidirectionalBroadcast golden outputs; numpy's broadcasting arithmetic.
 *   reduce                    ReduceMean, ReduceProd, ReduceL2, ReduceMax, ReduceMax_axis0, ReduceMax_mid golden outputs; numpy's
 *                             reductions in float64.
 *   layernorm                 LayerNormalization2d / 4d golden outputs; the float64 definition; rows of zero mean and unit
 *                             variance before scale and bias.
 *   global_avg_pool           GlobalAvgPool2d golden output.
 *   softmax                   Softmax1d / 2d / 3d / 4d golden outputs; scipy's softmax and log_softmax in float64; rows sum
 *                             to 1; invariance under a shift of the input.
 *   pool2d                    MaxPool1d, MaxPool2d, AvgPool, AvgPoolPad, AvgPoolCountIncludePad golden outputs;
 *                             a float64 restatement of the ONNX definition over random geometries (ceil_mode and
 *                             both divisor conventions included); torch's max_pool / avg_pool; window = image is
 *                             global_avg_pool.  The reference's ceil-mode and asymmetric-padding models come
 *                             without data files: those cases rest on the definition alone.
 *   organize_memory           the reference's MemoryPlanner.inc compiled as oracle/_ref and run on the
 *                             same lifetimes; known totals of the Linear_16 plan.
 *   quantize/dequantize, gemm_i8, conv_i8, e4m3 codec, gemm_fp8
 *                             PARITY UNPINNED BY THE REFERENCE: it has no quantised operator
 *                             (parsers/src/RModelParser_ONNX.cxx:279-367).  Pinned instead by what the
 *                             ONNX definitions fix: exhaustive tables (all 256 e4m3 codes, all int8
 *                             products), tie cases of round-half-even, int64 numpy matmul, identity /
 *                             one-hot special cases.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------------------------------------
 * fp32 path
 * ---------------------------------------------------------------------------------------------- */

/* Portable column-major SGEMM with the Fortran BLAS meaning of every argument; the reference leaves
 * this to whatever BLAS is linked (core/src/utils/SOFIE_common_helpers.cxx:32-38).  The dot product
 * runs over k in increasing order in fp32. */
static void oracle_sgemm(char transa, char transb, int m, int n, int k, float alpha, const float *A, int lda,
                         const float *B, int ldb, float beta, float *C, int ldc)
{
   const int ta = (transa == 't' || transa == 'T');
   const int tb = (transb == 't' || transb == 'T');
   for (int j = 0; j < n; ++j) {
      for (int i = 0; i < m; ++i) {
         float sum = 0.0f;
         for (int p = 0; p < k; ++p) {
            float a = ta ? A[(size_t)i * lda + p] : A[(size_t)p * lda + i];
            float b = tb ? B[(size_t)p * ldb + j] : B[(size_t)j * ldb + p];
            sum += a * b;
         }
         float *c = &C[(size_t)j * ldc + i];
         *c = (beta == 0.0f) ? alpha * sum : alpha * sum + beta * *c;
      }
   }
}

/* Gemm_Call of the generated code (core/src/utils/SOFIE_common_helpers.cxx:296-310): optional copy of
 * C into the output, then sgemm_ with lda = transa ? k : m, ldb = transb ? n : k, ldc = m. */
ORACLE_API void oracle_gemm_call(float *output, int transa, int transb, int m, int n, int k, float alpha, const float *A,
                                 const float *B, float beta, const float *C)
{
   int lda = transa ? k : m;
   int ldb = transb ? n : k;
   if (C != NULL)
      memcpy(output, C, sizeof(float) * (size_t)m * (size_t)n);
   oracle_sgemm(transa ? 't' : 'n', transb ? 't' : 'n', m, n, k, alpha, A, lda, B, ldb, beta, output, m);
}

/* Relu helper (SOFIE_common_helpers.cxx:325-332): NaN -> 0, -0 -> +0. */
ORACLE_API void oracle_relu(float *out, const float *in, size_t n)
{
   for (size_t i = 0; i < n; ++i)
      out[i] = (in[i] > 0.0f) ? in[i] : 0.0f;
}
/* LeakyRelu as fused by the Gemm emitter (ROperator_Gemm.hxx:729-738). */
ORACLE_API void oracle_leaky_relu(float *out, const float *in, size_t n, float alpha)
{
   for (size_t i = 0; i < n; ++i)
      out[i] = in[i] >= 0.0f ? in[i] : alpha * in[i];
}
/* ROperator_Sigmoid.hxx:43-59 */
ORACLE_API void oracle_sigmoid(float *out, const float *in, size_t n)
{
   for (size_t i = 0; i < n; ++i)
      out[i] = 1.0f / (1.0f + expf(-in[i]));
}
/* ROperator_Gelu.hxx:42-71, erf form */
ORACLE_API void oracle_gelu(float *out, const float *in, size_t n)
{
   for (size_t i = 0; i < n; ++i)
      out[i] = 0.5f * in[i] * (1.0f + erff(in[i] * 0.7071067811865475f));
}
/* ROperator_Gelu.hxx:42-71, tanh form */
ORACLE_API void oracle_gelu_tanh(float *out, const float *in, size_t n)
{
   for (size_t i = 0; i < n; ++i) {
      float x = in[i];
      out[i] = 0.5f * x * (1.0f + tanhf(0.7978845608028654f * (x + 0.044715f * x * x * x)));
   }
}
ORACLE_API void oracle_tanh(float *out, const float *in, size_t n)
{
   for (size_t i = 0; i < n; ++i)
      out[i] = tanhf(in[i]);
}

/* The reference's remaining one-to-one float operators, codes 7..21 of include/sofie_hip.h:
 * UnaryOpTraits<T, ...>::Op (core/inc/SOFIE/operators/ROperator_BasicUnary.hxx:17-103: 1/x, std::sqrt, -x, std::exp,
 * std::log, std::sin, std::cos, std::abs, Softplus as x >= 20 ? x : log1p(exp(x)), std::atan, std::floor, std::asinh,
 * std::acosh, std::atanh) and Clip, Y = max(min_val, min(max_val, X)) (ROperator_Clip.hxx:18). */
ORACLE_API void oracle_basic_unary(float *out, const float *in, size_t n, int op, float alpha, float beta)
{
   for (size_t i = 0; i < n; ++i) {
      const float x = in[i];
      float y = x;
      switch (op) {
      case 7: y = 1.0f / x; break;
      case 8: y = sqrtf(x); break;
      case 9: y = -x; break;
      case 10: y = expf(x); break;
      case 11: y = logf(x); break;
      case 12: y = sinf(x); break;
      case 13: y = cosf(x); break;
      case 14: y = fabsf(x); break;
      case 15: y = (x >= 20.0f) ? x : log1pf(expf(x)); break;
      case 16: y = atanf(x); break;
      case 17: y = floorf(x); break;
      case 18: y = asinhf(x); break;
      case 19: y = acoshf(x); break;
      case 20: y = atanhf(x); break;
      case 21: y = fmaxf(alpha, fminf(beta, x)); break;
      case 22: y = beta * (fmaxf(0.0f, x) + fminf(0.0f, alpha * (expf(x) - 1.0f))); break; /* Selu, ROperator_Selu.hxx:56-62; beta = gamma */
      case 23: y = x >= 0.0f ? x : alpha * (expf(x) - 1.0f); break; /* Elu, ROperator_Elu.hxx:69-74 */
      case 24: y = erff(x); break;                                  /* Erf, ROperator_Erf.hxx: std::erf */
      case 25: y = fmaxf(0.0f, fminf(1.0f, alpha * x + beta)); break; /* HardSigmoid, ROperator_HardSigmoid.hxx:71-74 */
      case 26: {                                                    /* HardSwish, ROperator_HardSwish.hxx:56-60 */
         float h = 0x1.5555555555555p-3f * x + 0x1p-1f;
         y = x * fmaxf(0.0f, fminf(1.0f, h));
         break;
      }
      case 27: y = x / (1 + expf(-x)); break;                       /* Swish, ROperator_Swish.hxx:54-56 */
      default: break;
      }
      out[i] = y;
   }
}

/* activation codes of include/sofie_hip.h */
ORACLE_API void oracle_unary(float *out, const float *in, size_t n, int act, float alpha)
{
   switch (act) {
   case 1: oracle_relu(out, in, n); break;
   case 2: oracle_leaky_relu(out, in, n, alpha); break;
   case 3: oracle_sigmoid(out, in, n); break;
   case 4: oracle_gelu(out, in, n); break;
   case 5: oracle_gelu_tanh(out, in, n); break;
   case 6: oracle_tanh(out, in, n); break;
   default:
      if (act >= 7 && act <= 27)
         oracle_basic_unary(out, in, n, act, alpha, 0.0f);
      else if (out != in)
         memmove(out, in, n * sizeof(float));
   }
}

/* a chain of one-to-one operators, applied in order (codes, alpha, beta as in sofie_post_ops) */
ORACLE_API void oracle_unary_chain(float *out, const float *in, size_t n, int count, const int *op, const float *alpha, const float *beta)
{
   if (out != in)
      memmove(out, in, n * sizeof(float));
   for (int i = 0; i < count; ++i) {
      if (op[i] >= 7 && op[i] <= 27)
         oracle_basic_unary(out, out, n, op[i], alpha[i], beta[i]);
      else
         oracle_unary(out, out, n, op[i], alpha[i]);
   }
}

/* ROperator_Gemm<float>::Generate, CPU form (core/inc/SOFIE/operators/ROperator_Gemm.hxx:419-741):
 * row-major A[M,K] (or [K,M] with transA), B[K,N] (or [N,K] with transB).
 *   - a bias that is not Y-shaped is written into Y row by row (Copy for [N]/[1,N], Fill for [M,1] and
 *     scalars) and beta becomes 1 (:578-617); a Y-shaped bias is passed to Gemm_Call as C with the
 *     operator's beta; no bias forces beta = 0 (:491-499);
 *   - the row-major product is obtained from the column-major BLAS by swapping the operands:
 *     Gemm_Call(Y, transB, transA, n, m, k, alpha, B, A, beta, C) (:685-709);
 *   - fused Relu / LeakyRelu run over Y afterwards (:724-738).
 * bias_mode: 0 none, 1 row [N], 2 column [M,1], 3 scalar, 4 full [M,N]. act as in oracle_unary. */
ORACLE_API void oracle_gemm_f32(int M, int N, int K, int transA, int transB, float alpha, float beta, const float *A,
                                const float *B, const float *C, int bias_mode, int act, float act_alpha, float *Y)
{
   const float *c_arg = NULL;
   if (bias_mode == 0) {
      beta = 0.0f;
   } else if (bias_mode == 4) {
      c_arg = C;
   } else {
      beta = 1.0f;
      for (int j = 0; j < M; ++j) {
         float *row = Y + (size_t)N * j;
         if (bias_mode == 1)
            memcpy(row, C, sizeof(float) * (size_t)N);
         else
            for (int i = 0; i < N; ++i)
               row[i] = (bias_mode == 2) ? C[j] : C[0];
      }
   }
   oracle_gemm_call(Y, transB, transA, N, M, K, alpha, B, A, beta, c_arg);
   oracle_unary(Y, Y, (size_t)M * (size_t)N, act, act_alpha);
}

/* ROperator_BasicBinary<float,Add>::Generate (core/inc/SOFIE/operators/ROperator_BasicBinary.hxx:380-510):
 * nested loops over the output dims, a broadcast dim is read at index 0.  Shapes right-aligned, rank<=6. */
ORACLE_API void oracle_add_broadcast(int rank, const int64_t *yshape, const int64_t *ashape, const int64_t *bshape,
                                     const float *A, const float *B, float *Y)
{
   int64_t sa[6], sb[6], n = 1, ca = 1, cb = 1;
   for (int d = rank - 1; d >= 0; --d) {
      sa[d] = (ashape[d] == 1 && yshape[d] != 1) ? 0 : ca;
      sb[d] = (bshape[d] == 1 && yshape[d] != 1) ? 0 : cb;
      ca *= ashape[d];
      cb *= bshape[d];
      n *= yshape[d];
   }
   for (int64_t i = 0; i < n; ++i) {
      int64_t rest = i, ia = 0, ib = 0;
      for (int d = rank - 1; d >= 0; --d) {
         int64_t idx = rest % yshape[d];
         rest /= yshape[d];
         ia += idx * sa[d];
         ib += idx * sb[d];
      }
      Y[i] = A[ia] + B[ib];
   }
}

/* The other binary operators with the same loops (BinaryOperatorTrait<T, Op>::Op, ROperator_BasicBinary.hxx:22-53) and the
 * pairwise steps of the n-ary ones (NaryOperatorTraits, ROperator_BasicNary.hxx:19-100: std::max({..}) / std::min({..}) are
 * left folds that keep the first of equal elements; Sum adds left to right; Mean divides that sum by T(count)).
 * op: 0 a+b, 1 a-b, 2 a*b, 3 a/b, 4 powf(a,b), 5 std::max(a,b), 6 std::min(a,b), 7 (a+b)/param. */
ORACLE_API void oracle_binary_broadcast(int rank, const int64_t *yshape, const int64_t *ashape, const int64_t *bshape, const float *A,
                                        const float *B, float *Y, int op, float param)
{
   int64_t sa[6], sb[6], n = 1, ca = 1, cb = 1;
   for (int d = rank - 1; d >= 0; --d) {
      sa[d] = (ashape[d] == 1 && yshape[d] != 1) ? 0 : ca;
      sb[d] = (bshape[d] == 1 && yshape[d] != 1) ? 0 : cb;
      ca *= ashape[d];
      cb *= bshape[d];
      n *= yshape[d];
   }
   for (int64_t i = 0; i < n; ++i) {
      int64_t rest = i, ia = 0, ib = 0;
      for (int d = rank - 1; d >= 0; --d) {
         int64_t idx = rest % yshape[d];
         rest /= yshape[d];
         ia += idx * sa[d];
         ib += idx * sb[d];
      }
      const float a = A[ia], b = B[ib];
      float y;
      switch (op) {
      case 1: y = a - b; break;
      case 2: y = a * b; break;
      case 3: y = a / b; break;
      case 4: y = powf(a, b); break;
      case 5: y = a < b ? b : a; break;
      case 6: y = b < a ? b : a; break;
      case 7: y = (a + b) / param; break;
      default: y = a + b; break;
      }
      Y[i] = y;
   }
}

/* UTILITY::Im2col (core/src/utils/SOFIE_common_helpers.cxx:47-83): rows (c,kh,kw), columns (oh,ow),
 * zero outside the image; the unsigned-compare bounds test of :40-45. */
static int in_range(int a, int b)
{
   return (unsigned)a < (unsigned)b;
}
ORACLE_API void oracle_im2col(const float *data_im, int channels, int height, int width, int kernel_h, int kernel_w,
                              int pad_h_begin, int pad_h_end, int pad_w_begin, int pad_w_end, int stride_h, int stride_w,
                              int dilation_h, int dilation_w, float *data_col)
{
   const int output_h = (height + pad_h_begin + pad_h_end - (dilation_h * (kernel_h - 1) + 1)) / stride_h + 1;
   const int output_w = (width + pad_w_begin + pad_w_end - (dilation_w * (kernel_w - 1) + 1)) / stride_w + 1;
   const int channel_size = height * width;
   for (int channel = 0; channel < channels; ++channel, data_im += channel_size) {
      for (int kr = 0; kr < kernel_h; ++kr) {
         for (int kc = 0; kc < kernel_w; ++kc) {
            int input_row = -pad_h_begin + kr * dilation_h;
            for (int orow = 0; orow < output_h; ++orow, input_row += stride_h) {
               if (!in_range(input_row, height)) {
                  for (int oc = 0; oc < output_w; ++oc)
                     *(data_col++) = 0.0f;
               } else {
                  int input_col = -pad_w_begin + kc * dilation_w;
                  for (int oc = 0; oc < output_w; ++oc, input_col += stride_w)
                     *(data_col++) = in_range(input_col, width) ? data_im[input_row * width + input_col] : 0.0f;
               }
            }
         }
      }
   }
}

/* ROperator_Conv<float>::Generate for 1-D/2-D convolutions (core/inc/SOFIE/operators/ROperator_Conv.hxx:406-642):
 *   1. the kernel is copied into the dilated layout tensor_<Y>_f, zero between the taps (:442-476);
 *      from then on the convolution runs with kernel size k + (d-1)(k-1) and dilation 1 (:478);
 *   2. for every image (and group): Im2col, then Gemm_Call(y, false,false, m=OH*OW, n=Cout/g,
 *      k=Cin/g*KH*KW, 1, xcol, f, beta, bias) with the bias pre-broadcast to [Cout,OH,OW] and beta=1,
 *      or beta=0 without a bias (:487-552, 560-616).
 * X [N,C,H,W]; W [Cout, C/group, kh, kw]; pads {h_begin, w_begin, h_end, w_end}; Y [N,Cout,OH,OW].
 * For a 1-D convolution pass H=1, kh=1, pads (0,p0,0,p1), stride_h=1, dil_h=1 (:517-523).
 * `act`/`act_alpha`: an activation applied afterwards (a separate operator in the reference). */
ORACLE_API int oracle_conv_f32(int N, int C, int H, int W, int Cout, int kh, int kw, int pad_h0, int pad_w0, int pad_h1,
                               int pad_w1, int stride_h, int stride_w, int dil_h, int dil_w, int group, const float *X,
                               const float *Wt, const float *bias, int act, float act_alpha, float *Y)
{
   const int Cg = C / group, Cout_g = Cout / group;
   const int ekh = kh + (dil_h - 1) * (kh - 1), ekw = kw + (dil_w - 1) * (kw - 1);
   const int OH = (H + pad_h0 + pad_h1 - ekh) / stride_h + 1;
   const int OW = (W + pad_w0 + pad_w1 - ekw) / stride_w + 1;
   const int m = OH * OW, k = Cg * ekh * ekw;
   float *f = (float *)calloc((size_t)Cout * Cg * ekh * ekw, sizeof(float));
   float *xcol = (float *)malloc(sizeof(float) * (size_t)k * (size_t)m);
   float *bcast = bias ? (float *)malloc(sizeof(float) * (size_t)Cout * m) : NULL;
   if (!f || !xcol || (bias && !bcast)) {
      free(f);
      free(xcol);
      free(bcast);
      return 1;
   }
   for (int oc = 0; oc < Cout; ++oc)
      for (int ic = 0; ic < Cg; ++ic)
         for (int y = 0; y < kh; ++y)
            for (int x = 0; x < kw; ++x)
               f[(size_t)oc * Cg * ekh * ekw + (size_t)ic * ekh * ekw + (size_t)y * dil_h * ekw + (size_t)x * dil_w] =
                  Wt[(size_t)oc * Cg * kh * kw + (size_t)ic * kh * kw + (size_t)y * kw + x];
   if (bias)
      for (int oc = 0; oc < Cout; ++oc)
         for (int i = 0; i < m; ++i)
            bcast[(size_t)oc * m + i] = bias[oc];
   const float beta = bias ? 1.0f : 0.0f;
   for (int n = 0; n < N; ++n) {
      for (int g = 0; g < group; ++g) {
         size_t x_offset = (size_t)n * C * H * W + (size_t)g * Cg * H * W;
         size_t g_offset = (size_t)g * Cout_g * m;
         size_t out_offset = (size_t)n * Cout * m + g_offset;
         oracle_im2col(X + x_offset, Cg, H, W, ekh, ekw, pad_h0, pad_h1, pad_w0, pad_w1, stride_h, stride_w, 1, 1, xcol);
         oracle_gemm_call(Y + out_offset, 0, 0, m, Cout_g, k, 1.0f, xcol, f + (size_t)g * Cout_g * k, beta,
                          bias ? bcast + g_offset : NULL);
      }
   }
   oracle_unary(Y, Y, (size_t)N * Cout * m, act, act_alpha);
   free(f);
   free(xcol);
   free(bcast);
   return 0;
}

/* UTILITY::Im2col_3d (core/src/utils/SOFIE_common_helpers.cxx:85-139): rows (c, kd, kh, kw), columns (od, oh, ow), zero outside
 * the volume. */
ORACLE_API void oracle_im2col_3d(const float *data_im, int channels, int depth, int height, int width, int kernel_d, int kernel_h,
                                 int kernel_w, int pad_d_begin, int pad_d_end, int pad_h_begin, int pad_h_end, int pad_w_begin,
                                 int pad_w_end, int stride_d, int stride_h, int stride_w, int dilation_d, int dilation_h,
                                 int dilation_w, float *data_col)
{
   const int output_h = (height + pad_h_begin + pad_h_end - (dilation_h * (kernel_h - 1) + 1)) / stride_h + 1;
   const int output_w = (width + pad_w_begin + pad_w_end - (dilation_w * (kernel_w - 1) + 1)) / stride_w + 1;
   const int output_d = (depth + pad_d_begin + pad_d_end - (dilation_d * (kernel_d - 1) + 1)) / stride_d + 1;
   const int channel_size = height * width * depth;
   for (int channel = 0; channel < channels; ++channel, data_im += channel_size)
      for (int kd = 0; kd < kernel_d; ++kd)
         for (int kr = 0; kr < kernel_h; ++kr)
            for (int kc = 0; kc < kernel_w; ++kc) {
               int input_dep = -pad_d_begin + kd * dilation_d;
               for (int od = 0; od < output_d; ++od, input_dep += stride_d) {
                  int input_row = -pad_h_begin + kr * dilation_h;
                  for (int orow = 0; orow < output_h; ++orow, input_row += stride_h) {
                     int input_col = -pad_w_begin + kc * dilation_w;
                     for (int oc = 0; oc < output_w; ++oc, input_col += stride_w)
                        *(data_col++) = (in_range(input_dep, depth) && in_range(input_row, height) && in_range(input_col, width))
                                           ? data_im[input_dep * width * height + input_row * width + input_col]
                                           : 0.0f;
                  }
               }
            }
}

/* ROperator_Conv<float>::Generate for 3-D convolutions (core/inc/SOFIE/operators/ROperator_Conv.hxx:406-642): as in 1-D / 2-D the
 * kernel goes into the dilated layout (:442-476, zero between the taps, effective size k + (d-1)(k-1) per axis, dilation 1 from then
 * on), then per image and group Im2col_3d with the pads in the order {d_begin, d_end, h_begin, h_end, w_begin, w_end} taken from
 * the attribute {d_begin, h_begin, w_begin, d_end, h_end, w_end} (:533-541) and Gemm_Call(y, false, false, m = OD*OH*OW, n = Cout/g,
 * k = Cin/g*KD*KH*KW, 1, xcol, f, beta, bias).
 * X [N,C,D,H,W]; W [Cout, C/group, kd, kh, kw]; pads[6] = {d0,h0,w0,d1,h1,w1}; strides[3], dils[3]; Y [N,Cout,OD,OH,OW]. */
ORACLE_API int oracle_conv3d_f32(int N, int C, int D, int H, int W, int Cout, int kd, int kh, int kw, const int *pads, const int *strides,
                                 const int *dils, int group, const float *X, const float *Wt, const float *bias, int act, float act_alpha,
                                 float *Y)
{
   const int Cg = C / group, Cout_g = Cout / group;
   const int ekd = kd + (dils[0] - 1) * (kd - 1), ekh = kh + (dils[1] - 1) * (kh - 1), ekw = kw + (dils[2] - 1) * (kw - 1);
   const int OD = (D + pads[0] + pads[3] - ekd) / strides[0] + 1;
   const int OH = (H + pads[1] + pads[4] - ekh) / strides[1] + 1;
   const int OW = (W + pads[2] + pads[5] - ekw) / strides[2] + 1;
   const int m = OD * OH * OW, k = Cg * ekd * ekh * ekw;
   float *f = (float *)calloc((size_t)Cout * k, sizeof(float));
   float *xcol = (float *)malloc(sizeof(float) * (size_t)k * (size_t)m);
   float *bcast = bias ? (float *)malloc(sizeof(float) * (size_t)Cout * m) : NULL;
   if (!f || !xcol || (bias && !bcast)) {
      free(f);
      free(xcol);
      free(bcast);
      return 1;
   }
   for (int oc = 0; oc < Cout; ++oc)
      for (int ic = 0; ic < Cg; ++ic)
         for (int z = 0; z < kd; ++z)
            for (int y = 0; y < kh; ++y)
               for (int x = 0; x < kw; ++x)
                  f[(size_t)oc * k + (size_t)ic * ekd * ekh * ekw + (size_t)z * dils[0] * ekh * ekw + (size_t)y * dils[1] * ekw +
                    (size_t)x * dils[2]] = Wt[((((size_t)oc * Cg + ic) * kd + z) * kh + y) * kw + x];
   if (bias)
      for (int oc = 0; oc < Cout; ++oc)
         for (int i = 0; i < m; ++i)
            bcast[(size_t)oc * m + i] = bias[oc];
   const float beta = bias ? 1.0f : 0.0f;
   for (int n = 0; n < N; ++n)
      for (int g = 0; g < group; ++g) {
         const size_t x_offset = ((size_t)n * C + (size_t)g * Cg) * D * H * W;
         const size_t g_offset = (size_t)g * Cout_g * m;
         const size_t out_offset = (size_t)n * Cout * m + g_offset;
         oracle_im2col_3d(X + x_offset, Cg, D, H, W, ekd, ekh, ekw, pads[0], pads[3], pads[1], pads[4], pads[2], pads[5], strides[0],
                          strides[1], strides[2], 1, 1, 1, xcol);
         oracle_gemm_call(Y + out_offset, 0, 0, m, Cout_g, k, 1.0f, xcol, f + (size_t)g * Cout_g * k, beta, bias ? bcast + g_offset : NULL);
      }
   oracle_unary(Y, Y, (size_t)N * Cout * m, act, act_alpha);
   free(f);
   free(xcol);
   free(bcast);
   return 0;
}

/* GlobalAveragePool = AveragePool with kernel == image (core/inc/SOFIE/operators/ROperator_Pool.hxx:225-237):
 * sequential fp32 sum over the plane, then `value /= float(nsum)` (:362-368). */
ORACLE_API void oracle_global_avg_pool(float *Y, const float *X, int NC, int HW)
{
   for (int p = 0; p < NC; ++p) {
      float value = 0;
      for (int i = 0; i < HW; ++i)
         value += X[(size_t)p * HW + i];
      value /= (float)HW;
      Y[p] = value;
   }
}

/* MaxPool / AveragePool in 2-D (1-D: H = kh = 1; 3-D: oracle_pool3d below), the generated loops of core/inc/SOFIE/operators/ROperator_Pool.hxx:
 * bounds hmin = -pad_begin, hmax = H + pad_end - kh + 1 (ceil_mode: + stride instead of + 1, clipped to H) (:286-300);
 * window start walks hmin, hmin + stride, ... < hmax (:373-374); MaxPool keeps `xval > value` from -INFINITY (:376,
 * 394-396); AveragePool sums in window order and divides by float(nsum), nsum = kh*kw without padding and ceil_mode, else
 * the product of the per-axis extents min(i + kh, hi) - lo (:323-333, 379-384, 403-405).  Returns the number of outputs
 * written per plane (the caller's output shape must agree). */
static int oracle_pool_extent(int var, int kern, int size, int pad_end, int include_pad)
{
   int hi = include_pad ? size + pad_end : size;
   int lo = include_pad ? var : (var > 0 ? var : 0);
   return (var + kern < hi ? var + kern : hi) - lo;
}
ORACLE_API long oracle_pool2d(float *Y, const float *X, int planes, int H, int W, int kh, int kw, int pad_h0, int pad_w0, int pad_h1, int pad_w1,
                              int stride_h, int stride_w, int is_max, int ceil_mode, int count_include_pad)
{
   int hmin = -pad_h0, wmin = -pad_w0;
   int hmax = H + pad_h1 - kh + (ceil_mode ? stride_h : 1);
   int wmax = W + pad_w1 - kw + (ceil_mode ? stride_w : 1);
   if (ceil_mode && hmax > H)
      hmax = H;
   if (ceil_mode && wmax > W)
      wmax = W;
   int dynamic_divisor = ceil_mode || pad_h0 > 0 || pad_w0 > 0 || pad_h1 > 0 || pad_w1 > 0;
   size_t out = 0;
   for (int n = 0; n < planes; ++n) {
      const float *x = X + (size_t)n * H * W;
      for (int i = hmin; i < hmax; i += stride_h) {
         for (int j = wmin; j < wmax; j += stride_w) {
            float value = is_max ? -INFINITY : 0;
            int nsum = kh * kw;
            if (!is_max && dynamic_divisor)
               nsum = oracle_pool_extent(i, kh, H, pad_h1, count_include_pad) * oracle_pool_extent(j, kw, W, pad_w1, count_include_pad);
            for (int l = i; l < i + kh; l++) {
               if (l < 0 || l >= H)
                  continue;
               for (int m = j; m < j + kw; m++) {
                  if (m < 0 || m >= W)
                     continue;
                  float xval = x[l * W + m];
                  if (is_max) {
                     if (xval > value)
                        value = xval;
                  } else {
                     value += xval;
                  }
               }
            }
            if (!is_max)
               value /= (float)nsum;
            Y[out++] = value;
         }
      }
   }
   return planes ? (long)(out / (size_t)planes) : 0;
}

/* The same over three spatial axes (core/inc/SOFIE/operators/ROperator_Pool.hxx:293-300 bounds of the third axis, :421-475 the
 * generated loops): window starts i, j, k walk the three axes slowest first, the window is visited l, m, p in that order, the
 * divisor of an average is the product of the three extents (:433-438).  in/k/pad_begin/pad_end/stride are per axis. */
ORACLE_API long oracle_pool3d(float *Y, const float *X, int planes, const int *in, const int *k, const int *pad_begin, const int *pad_end,
                              const int *stride, int is_max, int ceil_mode, int count_include_pad)
{
   int lo[3], hi[3], dynamic_divisor = ceil_mode;
   for (int a = 0; a < 3; ++a) {
      lo[a] = -pad_begin[a];
      hi[a] = in[a] + pad_end[a] - k[a] + (ceil_mode ? stride[a] : 1);
      if (ceil_mode && hi[a] > in[a])
         hi[a] = in[a];
      dynamic_divisor |= pad_begin[a] > 0 || pad_end[a] > 0;
   }
   const size_t s0 = (size_t)in[1] * in[2], s1 = (size_t)in[2];
   size_t out = 0;
   for (int n = 0; n < planes; ++n) {
      const float *x = X + (size_t)n * in[0] * s0;
      for (int i = lo[0]; i < hi[0]; i += stride[0])
         for (int j = lo[1]; j < hi[1]; j += stride[1])
            for (int kk = lo[2]; kk < hi[2]; kk += stride[2]) {
               float value = is_max ? -INFINITY : 0;
               int nsum = k[0] * k[1] * k[2];
               if (!is_max && dynamic_divisor)
                  nsum = oracle_pool_extent(i, k[0], in[0], pad_end[0], count_include_pad) *
                         oracle_pool_extent(j, k[1], in[1], pad_end[1], count_include_pad) *
                         oracle_pool_extent(kk, k[2], in[2], pad_end[2], count_include_pad);
               for (int l = i; l < i + k[0]; l++) {
                  if (l < 0 || l >= in[0])
                     continue;
                  for (int m = j; m < j + k[1]; m++) {
                     if (m < 0 || m >= in[1])
                        continue;
                     for (int p = kk; p < kk + k[2]; p++) {
                        if (p < 0 || p >= in[2])
                           continue;
                        float xval = x[l * s0 + m * s1 + p];
                        if (is_max) {
                           if (xval > value)
                              value = xval;
                        } else {
                           value += xval;
                        }
                     }
                  }
               }
               if (!is_max)
                  value /= (float)nsum;
               Y[out++] = value;
            }
   }
   return planes ? (long)(out / (size_t)planes) : 0;
}

/* Softmax / LogSoftmax over the middle dimension of [outer, A, inner], the loops of ROperator_Softmax::Generate
 * (core/inc/SOFIE/operators/ROperator_Softmax.hxx): last axis (:92-119) y = exp(x - vmax), sum += y in order, then
 * y *= 1.0f / sum (or x - vmax - log(sum)); any other axis (:121-198) the same with y /= sum. */
ORACLE_API void oracle_softmax(float *Y, const float *X, long outer, int A, long inner, int log_softmax)
{
   for (long o = 0; o < outer; ++o) {
      for (long in = 0; in < inner; ++in) {
         const float *x = X + (size_t)o * A * inner + in;
         float *y = Y + (size_t)o * A * inner + in;
         float vmax = x[0];
         for (int i = 1; i < A; ++i)
            if (x[(size_t)i * inner] > vmax)
               vmax = x[(size_t)i * inner];
         float sum = 0.0f;
         for (int i = 0; i < A; ++i) {
            y[(size_t)i * inner] = expf(x[(size_t)i * inner] - vmax);
            sum += y[(size_t)i * inner];
         }
         if (log_softmax) {
            float log_sum = logf(sum);
            for (int i = 0; i < A; ++i)
               y[(size_t)i * inner] = x[(size_t)i * inner] - vmax - log_sum;
         } else if (inner == 1) {
            float inv_sum = 1.0f / sum;
            for (int i = 0; i < A; ++i)
               y[i] *= inv_sum;
         } else {
            for (int i = 0; i < A; ++i)
               y[(size_t)i * inner] /= sum;
         }
      }
   }
}

/* The Reduce family over the middle dimension of [outer, A, inner]: ROperator_Reduce<Op>::Generate
 * (core/inc/SOFIE/operators/ROperator_Reduce.hxx:349-400), whose three loop nests (reduced axes last, first, in the middle) all visit
 * the reduced elements of an output in increasing order.  op: 0 Sum, 1 Mean, 2 SumSquare, 3 Prod, 4 L2, 5 Max, 6 Min. */
ORACLE_API void oracle_reduce(float *Y, const float *X, long outer, int A, long inner, int op)
{
   for (long o = 0; o < outer; ++o) {
      for (long in = 0; in < inner; ++in) {
         const float *x = X + (size_t)o * A * inner + in;
         float y = op == 3 ? 1.0f : op == 5 ? -3.402823466e+38f : op == 6 ? 3.402823466e+38f : 0.0f;
         for (int a = 0; a < A; ++a) {
            float v = x[(size_t)a * inner];
            switch (op) {
            case 2:
            case 4: y += v * v; break;
            case 3: y *= v; break;
            case 5: y = y < v ? v : y; break; /* std::max(y, v) */
            case 6: y = v < y ? v : y; break; /* std::min(y, v) */
            default: y += v; break;
            }
         }
         if (op == 1)
            y /= (float)A;
         else if (op == 4)
            y = sqrtf(y);
         Y[(size_t)o * inner + in] = y;
      }
   }
}

/* LayerNormalization over [rows, L], the loops of ROperator_LayerNormalization::Generate
 * (core/inc/SOFIE/operators/ROperator_LayerNormalization.hxx:247-312): mean += x in order, mean /= L; sum += tmp*tmp with
 * tmp = x - mean; invStdDev = 1 / std::sqrt(sum / L + epsilon); Y = scale * invStdDev * (x - mean) [+ bias]. */
ORACLE_API void oracle_layernorm(float *Y, const float *X, const float *scale, const float *bias, long rows, int L, float epsilon, float *mean_out,
                                 float *inv_std_out)
{
   for (long r = 0; r < rows; ++r) {
      const float *x = X + (size_t)r * L;
      float mean = 0.0f;
      for (int j = 0; j < L; ++j)
         mean += x[j];
      mean /= (float)L;
      float sum = 0.0f;
      for (int j = 0; j < L; ++j) {
         float tmp = x[j] - mean;
         sum += tmp * tmp;
      }
      float invStdDev = 1 / sqrtf(sum / (float)L + epsilon);
      if (mean_out)
         mean_out[r] = mean;
      if (inv_std_out)
         inv_std_out[r] = invStdDev;
      for (int j = 0; j < L; ++j) {
         float v = scale[j] * invStdDev * (x[j] - mean);
         if (bias)
            v += bias[j];
         Y[(size_t)r * L + j] = v;
      }
   }
}

/* BatchNormalization at inference (core/inc/SOFIE/operators/ROperator_BatchNormalization.hxx:92-109, 139-148):
 * Initialize forms fused_scale[c] = scale[c] / sqrt(var[c] + eps) once; the generated loop computes
 * val = (x - mean[c]) * fused_scale[c] + bias[c], then `val > 0 ? val : 0` when a Relu was fused. */
ORACLE_API void oracle_batchnorm_fused_scale(float *fused, const float *scale, const float *var, int C, float eps)
{
   for (int c = 0; c < C; ++c)
      fused[c] = scale[c] / sqrtf(var[c] + eps);
}
ORACLE_API void oracle_batchnorm(float *Y, const float *X, const float *fused_scale, const float *mean, const float *bias, int N, int C,
                                 int spatial, int relu)
{
   size_t i = 0;
   for (int n = 0; n < N; ++n)
      for (int c = 0; c < C; ++c) {
         const float mean_val = mean[c], fused_scale_val = fused_scale[c], bias_val = bias[c];
         for (int sp = 0; sp < spatial; ++sp) {
            float val = (X[i] - mean_val) * fused_scale_val + bias_val;
            Y[i] = relu ? ((val > 0.0f) ? val : 0.0f) : val;
            i++;
         }
      }
}

/* ------------------------------------------------------------------------------------------------
 * Memory planner: OrganizeMemory (core/inc/SOFIE/utils/shared/MemoryPlanner.inc:33-132).
 * Tensor i lives in [begin[i], end[i]); events are swept in time order with frees (type 0) before
 * allocations (type 1) at the same time; an allocation takes the smallest free block that fits
 * (lowest offset among equals) from its start, else grows the pool; freed blocks merge with their
 * neighbours.  Events with equal (time,type) are taken in tensor order here (the reference leaves
 * that order to std::sort).  Returns 0, or 1 if some end <= begin, 2 if out of memory.
 * ---------------------------------------------------------------------------------------------- */
typedef struct {
   size_t off, size;
} free_block;
/* ---- the CPU path's pool planner -------------------------------------------------------------------------------
 * RModel::AllocateIntermediateMemory / CheckAndFlushIntermediateMemory (core/src/RModel.cxx:492-595, 597-674), driven
 * operator by operator as RModel::Generate does (:1474-1482): the outputs of an operator, largest first, each go into the
 * first free chunk that holds them (cut from the chunk's END), or grow the last chunk of the pool if that one is free, or
 * are appended; then every input whose last reader this operator is gives its chunk back, merging with free neighbours.
 * The pool is the end of the last chunk (GenerateIntermediateMemoryPool, :975-984).  The GPU backend plans with
 * OrganizeMemory (above), not with this; the function exists to pin the reference's other answer (Linear_16: 6400 B).
 *   ops: operator i produces tensors out_ids[out_ptr[i] .. out_ptr[i+1]) and reads in_ids[in_ptr[i] .. in_ptr[i+1]);
 *   last_use[t]: index of the operator after which t is released if t is among that operator's inputs, or -1 (a model
 *   output: never released). */
typedef struct {
   size_t off, size;
   int name; /* tensor id, or -1 for a free chunk */
} pool_chunk;
typedef struct {
   size_t off, size;
} free_chunk;

static int chunk_find(const pool_chunk *c, int n, size_t off)
{
   for (int i = 0; i < n; ++i)
      if (c[i].off == off)
         return i;
   return -1;
}
/* total_stack[off] = {name, size}: replaces the entry at off or inserts one, keeping the offsets ascending */
static void chunk_set(pool_chunk *c, int *n, size_t off, int name, size_t size)
{
   int i = chunk_find(c, *n, off);
   if (i < 0) {
      i = *n;
      while (i > 0 && c[i - 1].off > off) {
         c[i] = c[i - 1];
         --i;
      }
      ++*n;
   }
   c[i].off = off, c[i].name = name, c[i].size = size;
}
static void chunk_erase(pool_chunk *c, int *n, size_t off)
{
   int i = chunk_find(c, *n, off);
   if (i < 0)
      return;
   for (; i + 1 < *n; ++i)
      c[i] = c[i + 1];
   --*n;
}
static void free_insert(free_chunk *f, int *n, size_t off, size_t size)
{
   int i = *n;
   while (i > 0 && f[i - 1].off > off) {
      f[i] = f[i - 1];
      --i;
   }
   f[i].off = off, f[i].size = size;
   ++*n;
}
static void free_erase(free_chunk *f, int *n, int i)
{
   for (; i + 1 < *n; ++i)
      f[i] = f[i + 1];
   --*n;
}

ORACLE_API int oracle_plan_memory_greedy(int n_ops, const int *out_ptr, const int *out_ids, const int *in_ptr, const int *in_ids,
                                         int n_tensors, const size_t *size, const int *last_use, size_t *offset, size_t *pool_bytes)
{
   pool_chunk *total = (pool_chunk *)malloc(sizeof(pool_chunk) * (size_t)(2 * n_tensors + 2));
   free_chunk *avail = (free_chunk *)malloc(sizeof(free_chunk) * (size_t)(2 * n_tensors + 2));
   int *order = (int *)malloc(sizeof(int) * (size_t)(n_tensors + 1));
   if (!total || !avail || !order) {
      free(total), free(avail), free(order);
      return 1;
   }
   int nt = 0, na = 0;
   for (int op = 0; op < n_ops; ++op) {
      /* outputs ordered by size, largest first (:524-525; equal sizes keep their order here) */
      int no = 0;
      for (int k = out_ptr[op]; k < out_ptr[op + 1]; ++k) {
         int t = out_ids[k], i = no++;
         while (i > 0 && size[order[i - 1]] < size[t]) {
            order[i] = order[i - 1];
            --i;
         }
         order[i] = t;
      }
      for (int k = 0; k < no; ++k) {
         const int t = order[k];
         const size_t sz = size[t];
         int done = 0;
         for (int a = 0; a < na; ++a) {
            if (avail[a].size >= sz) {
               /* cut from the end of the free chunk (:540-547) */
               const size_t at = avail[a].off, loc = at + avail[a].size - sz;
               total[chunk_find(total, nt, at)].size -= sz;
               chunk_set(total, &nt, loc, t, sz);
               offset[t] = loc;
               avail[a].size -= sz;
               if (avail[a].size == 0)
                  free_erase(avail, &na, a);
               done = 1;
               break;
            } else if (a == na - 1 && total[nt - 1].off == avail[a].off) {
               /* the last free chunk is the last of the pool: it grows (:560-568) */
               chunk_set(total, &nt, avail[a].off, t, sz);
               offset[t] = avail[a].off;
               free_erase(avail, &na, a);
               done = 1;
               break;
            }
         }
         if (!done) {
            const size_t at = nt ? total[nt - 1].off + total[nt - 1].size : 0;
            chunk_set(total, &nt, at, t, sz);
            offset[t] = at;
         }
      }
      for (int k = in_ptr[op]; k < in_ptr[op + 1]; ++k) {
         const int t = in_ids[k];
         if (t < 0 || last_use[t] != op)
            continue;
         int c = -1;
         for (int i = 0; i < nt; ++i)
            if (total[i].name == t) {
               c = i;
               break;
            }
         if (c < 0)
            continue;
         const size_t coff = total[c].off, csz = total[c].size;
         int g = 0; /* first free chunk above coff */
         while (g < na && avail[g].off <= coff)
            ++g;
         const int sm = g - 1; /* last free chunk below */
         if (sm >= 0 && avail[sm].off + avail[sm].size == coff) {
            avail[sm].size += csz;
            total[chunk_find(total, nt, avail[sm].off)].size += csz;
            if (g < na && avail[sm].off + avail[sm].size == avail[g].off) {
               const size_t goff = avail[g].off;
               avail[sm].size += avail[g].size;
               total[chunk_find(total, nt, avail[sm].off)].size += total[chunk_find(total, nt, goff)].size;
               chunk_erase(total, &nt, goff);
               free_erase(avail, &na, g);
            }
            chunk_erase(total, &nt, coff);
         } else if (g < na && coff + csz == avail[g].off) {
            const size_t goff = avail[g].off, merged = csz + avail[g].size;
            free_erase(avail, &na, g);
            free_insert(avail, &na, coff, merged);
            total[c].size += total[chunk_find(total, nt, goff)].size;
            chunk_erase(total, &nt, goff);
            total[chunk_find(total, nt, coff)].name = -1;
         } else {
            free_insert(avail, &na, coff, csz);
            total[c].name = -1;
         }
      }
   }
   *pool_bytes = nt ? total[nt - 1].off + total[nt - 1].size : 0;
   free(total), free(avail), free(order);
   return 0;
}

typedef struct {
   int t, type, idx;
} mem_event;
static int cmp_event(const void *pa, const void *pb)
{
   const mem_event *a = (const mem_event *)pa, *b = (const mem_event *)pb;
   if (a->t != b->t)
      return a->t < b->t ? -1 : 1;
   if (a->type != b->type)
      return a->type < b->type ? -1 : 1;
   return (a->idx > b->idx) - (a->idx < b->idx);
}
ORACLE_API int oracle_organize_memory(int n, const int *begin, const int *end, const size_t *size, size_t *offsets,
                                      size_t *total_bytes, size_t *total_free_bytes, size_t *largest_free_block)
{
   for (int i = 0; i < n; ++i)
      if (!(end[i] > begin[i]))
         return 1;
   mem_event *ev = (mem_event *)malloc(sizeof(mem_event) * (size_t)(2 * n + 1));
   free_block *fl = (free_block *)malloc(sizeof(free_block) * (size_t)(n + 1)); /* sorted by offset */
   char *live = (char *)calloc((size_t)n + 1, 1);
   if (!ev || !fl || !live) {
      free(ev);
      free(fl);
      free(live);
      return 2;
   }
   for (int i = 0; i < n; ++i) {
      ev[2 * i] = (mem_event){end[i], 0, i};
      ev[2 * i + 1] = (mem_event){begin[i], 1, i};
   }
   qsort(ev, (size_t)(2 * n), sizeof(mem_event), cmp_event);
   int nfree = 0;
   size_t total = 0, tfree = 0, lfree = 0;
   for (int e = 0; e < 2 * n; ++e) {
      int idx = ev[e].idx;
      if (ev[e].type == 0) {
         if (!live[idx])
            continue;
         live[idx] = 0;
         free_block fb = {offsets[idx], size[idx]};
         int pos = 0;
         while (pos < nfree && fl[pos].off < fb.off)
            ++pos;
         memmove(&fl[pos + 1], &fl[pos], sizeof(free_block) * (size_t)(nfree - pos));
         fl[pos] = fb;
         ++nfree;
         if (pos > 0 && fl[pos - 1].off + fl[pos - 1].size == fl[pos].off) {
            fl[pos - 1].size += fl[pos].size;
            memmove(&fl[pos], &fl[pos + 1], sizeof(free_block) * (size_t)(nfree - pos - 1));
            --nfree;
            --pos;
         }
         if (pos + 1 < nfree && fl[pos].off + fl[pos].size == fl[pos + 1].off) {
            fl[pos].size += fl[pos + 1].size;
            memmove(&fl[pos + 1], &fl[pos + 2], sizeof(free_block) * (size_t)(nfree - pos - 2));
            --nfree;
         }
      } else {
         size_t need = size[idx];
         int best = -1;
         for (int i = 0; i < nfree; ++i)
            if (fl[i].size >= need && (best < 0 || fl[i].size < fl[best].size))
               best = i;
         size_t before = total, off;
         if (best >= 0) {
            off = fl[best].off;
            if (fl[best].size == need) {
               memmove(&fl[best], &fl[best + 1], sizeof(free_block) * (size_t)(nfree - best - 1));
               --nfree;
            } else {
               fl[best].off += need;
               fl[best].size -= need;
            }
         } else {
            off = total;
            total += need;
         }
         offsets[idx] = off;
         live[idx] = 1;
         if (total > before) {
            tfree = 0;
            lfree = 0;
            for (int i = 0; i < nfree; ++i) {
               tfree += fl[i].size;
               if (fl[i].size > lfree)
                  lfree = fl[i].size;
            }
         }
      }
   }
   *total_bytes = total;
   *total_free_bytes = tfree;
   *largest_free_block = lfree;
   free(ev);
   free(fl);
   free(live);
   return 0;
}

/* ------------------------------------------------------------------------------------------------
 * Quantised operators (ONNX definitions; no counterpart in the reference -- see the header)
 * ---------------------------------------------------------------------------------------------- */

/* sat8(rne(v)): nearbyintf under the default rounding mode is round-half-to-even; NaN -> 0. */
static inline int sat8_rne(float v)
{
   if (!(v == v))
      return 0;
   float r = nearbyintf(v);
   if (r < -128.0f)
      r = -128.0f;
   if (r > 127.0f)
      r = 127.0f;
   return (int)r;
}

/* QuantizeLinear, per tensor, zero point 0: q = sat8(rne(x / scale)), fp32 division. */
ORACLE_API void oracle_quantize_linear(int8_t *q, const float *x, size_t n, float scale)
{
   for (size_t i = 0; i < n; ++i)
      q[i] = (int8_t)sat8_rne(x[i] / scale);
}
/* DequantizeLinear: y = float(q) * scale. */
ORACLE_API void oracle_dequantize_linear_i8(float *y, const int8_t *q, size_t n, float scale)
{
   for (size_t i = 0; i < n; ++i)
      y[i] = (float)q[i] * scale;
}
ORACLE_API void oracle_dequantize_linear_i32(float *y, const int32_t *q, size_t n, float scale)
{
   for (size_t i = 0; i < n; ++i)
      y[i] = (float)q[i] * scale;
}

/* MatMulInteger: acc[m,n] = sum_k int32(A[m,k]) * int32(B[k,n]); A [M,K] row-major (or [K,M] with
 * transA), B [K,N] row-major (or [N,K] with transB).  Threads split the rows. */
ORACLE_API void oracle_matmul_integer(int M, int N, int K, int transA, int transB, const int8_t *A, const int8_t *B,
                                      int32_t *acc)
{
   /* re-lay B as [N,K] so the inner loop is contiguous; the sum is exact in any order */
   int8_t *bt = NULL, *at = NULL;
   if (!transB) {
      bt = (int8_t *)malloc((size_t)N * K + 1);
      for (int k = 0; k < K; ++k)
         for (int n = 0; n < N; ++n)
            bt[(size_t)n * K + k] = B[(size_t)k * N + n];
      B = bt;
   }
   if (transA) {
      at = (int8_t *)malloc((size_t)M * K + 1);
      for (int k = 0; k < K; ++k)
         for (int m = 0; m < M; ++m)
            at[(size_t)m * K + k] = A[(size_t)k * M + m];
      A = at;
   }
#ifdef _OPENMP
#pragma omp parallel for schedule(static)
#endif
   for (int m = 0; m < M; ++m) {
      const int8_t *a = A + (size_t)m * K;
      for (int n = 0; n < N; ++n) {
         const int8_t *b = B + (size_t)n * K;
         int32_t s = 0;
         for (int k = 0; k < K; ++k)
            s += (int32_t)a[k] * (int32_t)b[k];
         acc[(size_t)m * N + n] = s;
      }
   }
   free(bt);
   free(at);
}

/* The epilogue of the int8 Gemm, element by element (out kinds of include/sofie_hip.h):
 *   acc += bias[n]; acc = max(acc,0) if relu_acc;
 *   0: int32     1: float(acc)*s, then max(.,0) if relu_out     2: sat8(rne(float(acc)*s)), then max(.,0) if relu_out
 *   3: sat8(rne((float(acc)*s)/q_scale))
 * int32 -> fp32 conversion rounds to nearest even; one fp32 multiply, no fused multiply-add. */
ORACLE_API void oracle_gemm_i8_epilogue(int M, int N, const int32_t *acc, const int32_t *bias, const float *scale,
                                        float scale_scalar, float q_scale, int relu_acc, int relu_out, int out, void *Y)
{
   for (int m = 0; m < M; ++m) {
      for (int n = 0; n < N; ++n) {
         size_t i = (size_t)m * N + n;
         int32_t a = acc[i] + (bias ? bias[n] : 0);
         if (relu_acc && a < 0)
            a = 0;
         float s = scale ? scale[n] : scale_scalar;
         switch (out) {
         case 0: ((int32_t *)Y)[i] = a; break;
         case 1: {
            float v = (float)a * s;
            if (relu_out && !(v > 0.0f))
               v = 0.0f;
            ((float *)Y)[i] = v;
         } break;
         case 2: {
            int q = sat8_rne((float)a * s);
            if (relu_out && q < 0)
               q = 0;
            ((int8_t *)Y)[i] = (int8_t)q;
         } break;
         default: {
            float t = (float)a * s;
            ((int8_t *)Y)[i] = (int8_t)sat8_rne(t / q_scale);
         } break;
         }
      }
   }
}

ORACLE_API int oracle_gemm_i8(int M, int N, int K, int transA, int transB, const int8_t *A, const int8_t *B,
                              const int32_t *bias, const float *scale, float scale_scalar, float q_scale, int relu_acc,
                              int relu_out, int out, void *Y)
{
   int32_t *acc = (int32_t *)malloc(sizeof(int32_t) * ((size_t)M * N + 1));
   if (!acc)
      return 1;
   oracle_matmul_integer(M, N, K, transA, transB, A, B, acc);
   oracle_gemm_i8_epilogue(M, N, acc, bias, scale, scale_scalar, q_scale, relu_acc, relu_out, out, Y);
   free(acc);
   return 0;
}

/* int8 convolution, direct 7-loop form: acc = sum X_i8 * W_i8 (+ bias_i32[co]); the output is NCHW.
 * out: 0 int32, 1 float(acc)*scale[co] (then relu), 2 sat8(rne(float(acc)*scale[co])) then max(.,0) if relu. */
ORACLE_API void oracle_conv_i8(int N, int C, int H, int W, int Cout, int kh, int kw, int pad_h0, int pad_w0, int pad_h1,
                               int pad_w1, int stride_h, int stride_w, int dil_h, int dil_w, int group, const int8_t *X,
                               const int8_t *Wt, const int32_t *bias, const float *scale, int relu, int out, void *Y)
{
   const int Cg = C / group, Cout_g = Cout / group;
   const int OH = (H + pad_h0 + pad_h1 - (dil_h * (kh - 1) + 1)) / stride_h + 1;
   const int OW = (W + pad_w0 + pad_w1 - (dil_w * (kw - 1) + 1)) / stride_w + 1;
#ifdef _OPENMP
#pragma omp parallel for collapse(2) schedule(static)
#endif
   for (int n = 0; n < N; ++n) {
      for (int co = 0; co < Cout; ++co) {
         int g = co / Cout_g;
         for (int oh = 0; oh < OH; ++oh) {
            for (int ow = 0; ow < OW; ++ow) {
               int32_t a = bias ? bias[co] : 0;
               for (int ci = 0; ci < Cg; ++ci) {
                  for (int y = 0; y < kh; ++y) {
                     int ih = oh * stride_h - pad_h0 + y * dil_h;
                     if (!in_range(ih, H))
                        continue;
                     for (int x = 0; x < kw; ++x) {
                        int iw = ow * stride_w - pad_w0 + x * dil_w;
                        if (!in_range(iw, W))
                           continue;
                        a += (int32_t)X[(((size_t)n * C + g * Cg + ci) * H + ih) * W + iw] *
                             (int32_t)Wt[(((size_t)co * Cg + ci) * kh + y) * kw + x];
                     }
                  }
               }
               size_t i = (((size_t)n * Cout + co) * OH + oh) * OW + ow;
               if (out == 0) {
                  ((int32_t *)Y)[i] = (relu && a < 0) ? 0 : a;
               } else if (out == 1) {
                  float v = (float)a * scale[co];
                  ((float *)Y)[i] = relu ? ((v > 0.0f) ? v : 0.0f) : v;
               } else {
                  int q = sat8_rne((float)a * scale[co]);
                  if (relu && q < 0)
                     q = 0;
                  ((int8_t *)Y)[i] = (int8_t)q;
               }
            }
         }
      }
   }
}

/* Y = (float(sum_i32 over the plane) * scale) / float(HW) */
ORACLE_API void oracle_global_avg_pool_i8(float *Y, const int8_t *X, int NC, int HW, float scale)
{
   for (int p = 0; p < NC; ++p) {
      int32_t s = 0;
      for (int i = 0; i < HW; ++i)
         s += X[(size_t)p * HW + i];
      Y[p] = ((float)s * scale) / (float)HW;
   }
}

/* ------------------------------------------------------------------------------------------------
 * FP8 (OCP e4m3fn: 1 sign, 4 exponent (bias 7), 3 mantissa; no infinity; 0x7f/0xff are NaN; max 448)
 * ---------------------------------------------------------------------------------------------- */
ORACLE_API float oracle_e4m3_to_f32(uint8_t v)
{
   int sign = v >> 7, e = (v >> 3) & 15, m = v & 7;
   float r;
   if (e == 15 && m == 7)
      r = NAN;
   else if (e == 0)
      r = ldexpf((float)m, -9); /* subnormal: m/8 * 2^-6 */
   else
      r = ldexpf(1.0f + (float)m / 8.0f, e - 7);
   return sign ? -r : r;
}

/* fp32 -> e4m3fn, round to nearest even, saturating to +-448 (also for +-inf); NaN -> 0x7f. */
ORACLE_API uint8_t oracle_f32_to_e4m3(float x)
{
   if (x != x)
      return 0x7f;
   uint8_t sign = signbit(x) ? 0x80 : 0;
   float a = fabsf(x);
   if (a >= 448.0f)
      return sign | 0x7e; /* 448 and above, including values that would round up past 448 */
   int e;
   (void)frexpf(a, &e); /* a = f * 2^e, f in [0.5,1) -> exponent of the leading bit is e-1 */
   int exp = e - 1;
   if (exp < -6)
      exp = -6; /* subnormal range: fixed quantum 2^-9 */
   float quantum = ldexpf(1.0f, exp - 3);
   float q = nearbyintf(a / quantum); /* exact division by a power of two; ties to even */
   float r = q * quantum;
   if (r > 448.0f)
      return sign | 0x7e;
   /* encode r */
   if (r < ldexpf(1.0f, -6))
      return sign | (uint8_t)(r / ldexpf(1.0f, -9));
   int e2;
   float f2 = frexpf(r, &e2); /* r = f2 * 2^e2, f2 in [0.5,1) */
   int be = e2 - 1 + 7;
   int mant = (int)((f2 * 2.0f - 1.0f) * 8.0f);
   return sign | (uint8_t)(be << 3) | (uint8_t)mant;
}

ORACLE_API void oracle_quantize_fp8(uint8_t *q, const float *x, size_t n, float scale)
{
   for (size_t i = 0; i < n; ++i)
      q[i] = oracle_f32_to_e4m3(x[i] / scale);
}

/* fp32 -> bf16 bits, round to nearest even; NaN stays NaN. */
ORACLE_API uint16_t oracle_f32_to_bf16(float x)
{
   uint32_t u;
   memcpy(&u, &x, 4);
   if ((u & 0x7fffffffu) > 0x7f800000u)
      return (uint16_t)((u >> 16) | 0x40);
   u += 0x7fffu + ((u >> 16) & 1u);
   return (uint16_t)(u >> 16);
}

/* FP8 Gemm arbiter: products and sums in float64 (every e4m3 product is exact in fp32 and in fp64);
 * v = float(acc) * scale + bias[n]; activation in fp32; output fp32 (out=1) or bf16 bits (out=0).
 * Also returns sum_k |a*b| per element (fp32) when `abs_sum` is not NULL, for the error bound
 * K * 2^-24 * sum|a*b| * scale on the hardware's fp32 accumulation. */
ORACLE_API void oracle_gemm_fp8(int M, int N, int K, int transB, const uint8_t *A, const uint8_t *B, const float *bias,
                                float scale, int act, int out, void *Y, float *abs_sum)
{
   float lut[256];
   for (int i = 0; i < 256; ++i)
      lut[i] = oracle_e4m3_to_f32((uint8_t)i);
#ifdef _OPENMP
#pragma omp parallel for schedule(static)
#endif
   for (int m = 0; m < M; ++m) {
      for (int n = 0; n < N; ++n) {
         double s = 0.0, sa = 0.0;
         for (int k = 0; k < K; ++k) {
            double a = lut[A[(size_t)m * K + k]];
            double b = transB ? lut[B[(size_t)n * K + k]] : lut[B[(size_t)k * N + n]];
            s += a * b;
            sa += fabs(a * b);
         }
         float v = (float)s * scale;
         if (bias)
            v = v + bias[n];
         oracle_unary(&v, &v, 1, act, 0.0f);
         size_t i = (size_t)m * N + n;
         if (out == 1)
            ((float *)Y)[i] = v;
         else
            ((uint16_t *)Y)[i] = oracle_f32_to_bf16(v);
         if (abs_sum)
            abs_sum[i] = (float)sa;
      }
   }
}

ORACLE_API int oracle_num_threads(void)
{
#ifdef _OPENMP
   return omp_get_max_threads();
#else
   return 1;
#endif
}
ORACLE_API void oracle_set_num_threads(int n)
{
#ifdef _OPENMP
   omp_set_num_threads(n);
#else
   (void)n;
#endif
}
