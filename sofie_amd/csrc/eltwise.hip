// HBM-bound elementwise operators: QuantizeLinear / DequantizeLinear, the stand-alone activations,
// broadcast Add, GlobalAveragePool.  Each thread moves 16 bytes of the widest operand per step and
// the grid strides over the tensor, so the launches stay coalesced for any length.
#include "common.hpp"
#include <cfloat>

namespace sofie_hip {

static inline unsigned grid_for(size_t work_items, unsigned block = 256, unsigned max_blocks = 256 * 32)
{
   size_t b = (work_items + block - 1) / block;
   if (b < 1)
      b = 1;
   if (b > max_blocks)
      b = max_blocks;
   return (unsigned)b;
}

// q = sat8(rne(x / scale)), fp32 division (ONNX QuantizeLinear, zero point 0)
__global__ __launch_bounds__(256) void quantize_linear_kernel(int8_t *__restrict__ dst, const float *__restrict__ src,
                                                               size_t n, float scale, int vec)
{
   const size_t stride = (size_t)gridDim.x * blockDim.x;
   size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
   if (vec) {
      // four 16-byte loads per lane are issued before the first is used (a lane's pieces lie a workgroup's width apart, so every
      // wave instruction reads and writes whole lines): the kernel is a single round trip to memory, and a quarter of the waves run it
      const size_t n4 = n / 4;
      for (size_t base = blockIdx.x * (size_t)blockDim.x * 4 + threadIdx.x; base < n4; base += stride * 4) {
         float4 v[4];
#pragma unroll
         for (int j = 0; j < 4; ++j) {
            const size_t k = base + (size_t)j * blockDim.x;
            v[j] = k < n4 ? ((const float4 *)src)[k] : make_float4(0.f, 0.f, 0.f, 0.f);
         }
#pragma unroll
         for (int j = 0; j < 4; ++j) {
            const size_t k = base + (size_t)j * blockDim.x;
            int q0 = quantize_rne_sat8(__fdiv_rn(v[j].x, scale));
            int q1 = quantize_rne_sat8(__fdiv_rn(v[j].y, scale));
            int q2 = quantize_rne_sat8(__fdiv_rn(v[j].z, scale));
            int q3 = quantize_rne_sat8(__fdiv_rn(v[j].w, scale));
            if (k < n4)
               ((uint32_t *)dst)[k] = (uint32_t)(q0 & 0xff) | ((uint32_t)(q1 & 0xff) << 8) | ((uint32_t)(q2 & 0xff) << 16) | ((uint32_t)(q3 & 0xff) << 24);
         }
      }
      i = n4 * 4 + (blockIdx.x * (size_t)blockDim.x + threadIdx.x);
      if (i < n)
         dst[i] = (int8_t)quantize_rne_sat8(__fdiv_rn(src[i], scale));
   } else {
      for (; i < n; i += stride)
         dst[i] = (int8_t)quantize_rne_sat8(__fdiv_rn(src[i], scale));
   }
}

template <typename T>
__global__ __launch_bounds__(256) void dequantize_linear_kernel(float *__restrict__ dst, const T *__restrict__ src, size_t n,
                                                                 float scale)
{
   const size_t stride = (size_t)gridDim.x * blockDim.x;
   for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += stride)
      dst[i] = mul_nofma((float)src[i], scale);
}

__global__ __launch_bounds__(256) void unary_f32_kernel(float *dst, const float *src, size_t n, PostChain chain, int vec)
{
   const size_t stride = (size_t)gridDim.x * blockDim.x;
   size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
   if (vec) {
      const size_t n4 = n / 4;
      for (; i < n4; i += stride) {
         float4 v = ((const float4 *)src)[i];
         v.x = apply_chain(v.x, chain);
         v.y = apply_chain(v.y, chain);
         v.z = apply_chain(v.z, chain);
         v.w = apply_chain(v.w, chain);
         ((float4 *)dst)[i] = v;
      }
      i = n4 * 4 + (blockIdx.x * (size_t)blockDim.x + threadIdx.x);
      if (i < n)
         dst[i] = apply_chain(src[i], chain);
   } else {
      for (; i < n; i += stride)
         dst[i] = apply_chain(src[i], chain);
   }
}

// One output element per thread (grid-stride); neighbouring lanes take neighbouring outputs of the fastest axis, so the
// window rows they read overlap and lie next to each other in memory.  Three spatial axes, slowest first (a 2-D pooling has a
// first axis of extent 1): the window is visited axis 0, then 1, then 2, one fp32 addition at a time -- the order of the
// reference's generated loops, so an average has the bits of the reference's scalar loop.
__global__ __launch_bounds__(256) void pool_f32_kernel(float *__restrict__ Y, const float *__restrict__ X, sofie_pool3d_desc d, size_t total)
{
   const size_t stride = (size_t)gridDim.x * blockDim.x;
   const size_t s0 = (size_t)d.in[1] * (size_t)d.in[2], s1 = (size_t)d.in[2];
   for (size_t idx = blockIdx.x * (size_t)blockDim.x + threadIdx.x; idx < total; idx += stride) {
      const int o2 = (int)(idx % (size_t)d.out[2]);
      size_t t = idx / (size_t)d.out[2];
      const int o1 = (int)(t % (size_t)d.out[1]);
      t /= (size_t)d.out[1];
      const int o0 = (int)(t % (size_t)d.out[0]);
      const size_t plane = t / (size_t)d.out[0];
      const int i = o0 * d.stride[0] - d.pad_begin[0], j = o1 * d.stride[1] - d.pad_begin[1], k = o2 * d.stride[2] - d.pad_begin[2];
      const float *x = X + plane * (size_t)d.in[0] * s0;
      float value = d.mode == SOFIE_POOL_MAX ? -INFINITY : 0.0f;
      for (int l = i; l < i + d.k[0]; ++l) {
         if (l < 0 || l >= d.in[0])
            continue;
         for (int m = j; m < j + d.k[1]; ++m) {
            if (m < 0 || m >= d.in[1])
               continue;
            for (int p = k; p < k + d.k[2]; ++p) {
               if (p < 0 || p >= d.in[2])
                  continue;
               const float xv = x[(size_t)l * s0 + (size_t)m * s1 + p];
               if (d.mode == SOFIE_POOL_MAX) {
                  if (xv > value)
                     value = xv;
               } else {
                  value += xv;
               }
            }
         }
      }
      if (d.mode == SOFIE_POOL_AVERAGE) {
         int nsum = d.k[0] * d.k[1] * d.k[2];
         if (d.dynamic_divisor) {
            const int start[3] = {i, j, k};
            nsum = 1;
#pragma unroll
            for (int a = 0; a < 3; ++a) {
               const int hi = d.count_include_pad ? d.in[a] + d.pad_end[a] : d.in[a];
               const int lo = d.count_include_pad ? start[a] : (start[a] > 0 ? start[a] : 0);
               nsum *= (start[a] + d.k[a] < hi ? start[a] + d.k[a] : hi) - lo;
            }
         }
         value = __fdiv_rn(value, (float)nsum);
      }
      Y[idx] = value;
   }
}

struct AddShape {
   int rank;
   long long y[6], sa[6], sb[6]; // output dims, element strides of A and B (0 where broadcast)
};

struct TransposeShape {
   int rank;
   long long y[6], sx[6]; // output dims and, per OUTPUT axis, the element stride of the input axis it reads
};

// One output element per thread (grid-stride): writes are coalesced, reads are strided by the permutation.
__global__ __launch_bounds__(256) void transpose_f32_kernel(float *__restrict__ Y, const float *__restrict__ X, size_t n, TransposeShape sh)
{
   const size_t stride = (size_t)gridDim.x * blockDim.x;
   for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += stride) {
      size_t rest = i;
      long long ix = 0;
      for (int d = sh.rank - 1; d >= 0; --d) {
         ix += (long long)(rest % (size_t)sh.y[d]) * sh.sx[d];
         rest /= (size_t)sh.y[d];
      }
      Y[i] = X[ix];
   }
}

__global__ __launch_bounds__(256) void copy_rows_kernel(uint32_t *__restrict__ dst, size_t dst_pitch, const uint32_t *__restrict__ src, size_t src_pitch,
                                                         size_t rows, size_t row_words)
{
   const size_t n = rows * row_words, stride = (size_t)gridDim.x * blockDim.x;
   for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += stride) {
      const size_t r = i / row_words, c = i - r * row_words;
      dst[r * dst_pitch + c] = src[r * src_pitch + c];
   }
}

__device__ __forceinline__ float binary_op(float a, float b, int op, float param)
{
   switch (op) {
   case SOFIE_BINARY_SUB: return a - b;
   case SOFIE_BINARY_MUL: return mul_nofma(a, b);
   case SOFIE_BINARY_DIV: return __fdiv_rn(a, b);
   case SOFIE_BINARY_POW: return powf(a, b);
   case SOFIE_BINARY_MAX: return a < b ? b : a;
   case SOFIE_BINARY_MIN: return b < a ? b : a;
   case SOFIE_BINARY_ADD_DIV: return __fdiv_rn(a + b, param);
   default: return a + b;
   }
}

__global__ __launch_bounds__(256) void binary_f32_kernel(float *__restrict__ Y, const float *__restrict__ A, const float *__restrict__ B, size_t n,
                                                          AddShape sh, int op, float param)
{
   const size_t stride = (size_t)gridDim.x * blockDim.x;
   for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += stride) {
      size_t rest = i;
      long long ia = 0, ib = 0;
      for (int d = sh.rank - 1; d >= 0; --d) {
         long long idx = (long long)(rest % (size_t)sh.y[d]);
         rest /= (size_t)sh.y[d];
         ia += idx * sh.sa[d];
         ib += idx * sh.sb[d];
      }
      Y[i] = binary_op(A[ia], B[ib], op, param);
   }
}

__global__ __launch_bounds__(256) void add_f32_kernel(float *__restrict__ Y, const float *__restrict__ A,
                                                       const float *__restrict__ B, size_t n, AddShape sh)
{
   const size_t stride = (size_t)gridDim.x * blockDim.x;
   for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += stride) {
      size_t rest = i;
      long long ia = 0, ib = 0;
      for (int d = sh.rank - 1; d >= 0; --d) {
         long long idx = (long long)(rest % (size_t)sh.y[d]);
         rest /= (size_t)sh.y[d];
         ia += idx * sh.sa[d];
         ib += idx * sh.sb[d];
      }
      Y[i] = A[ia] + B[ib];
   }
}

// One wave per (n,c) plane: lanes stride over the plane, then a wave reduction.
template <typename T, typename ACC>
__global__ __launch_bounds__(256) void gap_kernel(float *__restrict__ Y, const T *__restrict__ X, int NC, int HW, float mul)
{
   const int plane = blockIdx.x * 4 + (threadIdx.x >> 6);
   const int lane = threadIdx.x & 63;
   if (plane >= NC)
      return;
   const T *p = X + (size_t)plane * HW;
   ACC s = 0;
   for (int i = lane; i < HW; i += 64)
      s += (ACC)p[i];
#pragma unroll
   for (int off = 32; off > 0; off >>= 1)
      s += __shfl_xor(s, off, 64);
   // fp32 input: sum / HW as the reference's pooling loop ends with `value /= float(nsum)`
   // (core/inc/SOFIE/operators/ROperator_Pool.hxx:362-368); int8 input: (float(sum) * scale) / HW
   if (lane == 0)
      Y[plane] = __fdiv_rn(mul_nofma((float)s, mul), (float)HW);
}

// NHWC int8 input, any channel count: one workgroup per image; thread c (strided) sums channel c over the
// pixels, so consecutive lanes read consecutive bytes.
__global__ __launch_bounds__(256) void gap_i8_nhwc_kernel(float *__restrict__ Y, const int8_t *__restrict__ X, int C, int HW,
                                                           float scale)
{
   const int8_t *p = X + (size_t)blockIdx.x * HW * C;
   for (int c = threadIdx.x; c < C; c += blockDim.x) {
      int s = 0;
      for (int i = 0; i < HW; ++i)
         s += (int)p[(size_t)i * C + c];
      Y[(size_t)blockIdx.x * C + c] = __fdiv_rn(mul_nofma((float)s, scale), (float)HW);
   }
}

// Softmax over the middle dimension of [outer, A, inner]: one wave per (outer, inner) line, lanes stride over the axis
// (consecutive lanes read consecutive elements when inner == 1), three passes over a line that stays in cache.
__global__ __launch_bounds__(256) void softmax_f32_kernel(float *__restrict__ Y, const float *__restrict__ X, long long lines, int A, long long inner,
                                                          int log_softmax)
{
   const int lane = threadIdx.x & 63;
   const long long wave = (long long)blockIdx.x * 4 + (threadIdx.x >> 6), nwaves = (long long)gridDim.x * 4;
   for (long long line = wave; line < lines; line += nwaves) {
      const long long o = line / inner, in = line - o * inner;
      const float *x = X + o * A * inner + in;
      float *y = Y + o * A * inner + in;
      float vmax = -INFINITY;
      for (int i = lane; i < A; i += 64) {
         const float v = x[i * inner];
         vmax = v > vmax ? v : vmax;
      }
#pragma unroll
      for (int off = 32; off >= 1; off >>= 1) {
         const float other = __shfl_xor(vmax, off, 64);
         vmax = other > vmax ? other : vmax;
      }
      float sum = 0.0f;
      for (int i = lane; i < A; i += 64)
         sum += expf(x[i * inner] - vmax);
#pragma unroll
      for (int off = 32; off >= 1; off >>= 1)
         sum += __shfl_xor(sum, off, 64);
      if (log_softmax) {
         const float log_sum = logf(sum);
         for (int i = lane; i < A; i += 64)
            y[i * inner] = x[i * inner] - vmax - log_sum;
      } else if (inner == 1) {
         const float inv_sum = 1.0f / sum;
         for (int i = lane; i < A; i += 64)
            y[i] = mul_nofma(expf(x[i] - vmax), inv_sum);
      } else {
         for (int i = lane; i < A; i += 64)
            y[i * inner] = __fdiv_rn(expf(x[i * inner] - vmax), sum);
      }
   }
}

__device__ __forceinline__ float reduce_start(int op)
{
   return op == SOFIE_REDUCE_PROD ? 1.0f : op == SOFIE_REDUCE_MAX ? -FLT_MAX : op == SOFIE_REDUCE_MIN ? FLT_MAX : 0.0f;
}
__device__ __forceinline__ float reduce_step(float y, float x, int op)
{
   switch (op) {
   case SOFIE_REDUCE_SUM_SQUARE:
   case SOFIE_REDUCE_L2: return y + mul_nofma(x, x);
   case SOFIE_REDUCE_PROD: return mul_nofma(y, x);
   case SOFIE_REDUCE_MAX: return y < x ? x : y;
   case SOFIE_REDUCE_MIN: return x < y ? x : y;
   default: return y + x;
   }
}
// folds two partial results (the tree form): partial sums of squares add, everything else combines as a step does
__device__ __forceinline__ float reduce_merge(float a, float b, int op)
{
   return (op == SOFIE_REDUCE_SUM_SQUARE || op == SOFIE_REDUCE_L2) ? a + b : reduce_step(a, b, op);
}
__device__ __forceinline__ float reduce_finish(float y, int A, int op)
{
   return op == SOFIE_REDUCE_MEAN ? __fdiv_rn(y, (float)A) : op == SOFIE_REDUCE_L2 ? sqrtf(y) : y;
}

// One output per thread, the reduced elements in increasing order: the reference's loop (neighbouring threads read neighbouring `inner`).
__global__ __launch_bounds__(256) void reduce_f32_kernel(float *__restrict__ Y, const float *__restrict__ X, size_t outputs, int A, long long inner, int op)
{
   const size_t stride = (size_t)gridDim.x * blockDim.x;
   for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < outputs; i += stride) {
      const size_t o = i / (size_t)inner, in = i - o * (size_t)inner;
      const float *x = X + o * (size_t)A * (size_t)inner + in;
      float y = reduce_start(op);
      for (int a = 0; a < A; ++a)
         y = reduce_step(y, x[(size_t)a * (size_t)inner], op);
      Y[i] = reduce_finish(y, A, op);
   }
}

// Long contiguous lines: one wave per line, lanes stride over it, then a shuffle tree.
__global__ __launch_bounds__(256) void reduce_lines_f32_kernel(float *__restrict__ Y, const float *__restrict__ X, long long lines, int A, int op)
{
   const int lane = threadIdx.x & 63;
   const long long wave = (long long)blockIdx.x * 4 + (threadIdx.x >> 6), nwaves = (long long)gridDim.x * 4;
   for (long long line = wave; line < lines; line += nwaves) {
      const float *x = X + line * A;
      float y = reduce_start(op);
      for (int a = lane; a < A; a += 64)
         y = reduce_step(y, x[a], op);
#pragma unroll
      for (int off = 32; off >= 1; off >>= 1)
         y = reduce_merge(y, __shfl_xor(y, off, 64), op);
      if (lane == 0)
         Y[line] = reduce_finish(y, A, op);
   }
}

// LayerNormalization: one wave per row of L elements, lanes stride over the row; mean, then the centred sum of squares, then the output.
__global__ __launch_bounds__(256) void layernorm_f32_kernel(float *__restrict__ Y, const float *__restrict__ X, const float *__restrict__ scale,
                                                            const float *__restrict__ bias, long long rows, int L, float epsilon,
                                                            float *__restrict__ mean_out, float *__restrict__ inv_std_out)
{
   const int lane = threadIdx.x & 63;
   const long long wave = (long long)blockIdx.x * 4 + (threadIdx.x >> 6), nwaves = (long long)gridDim.x * 4;
   for (long long row = wave; row < rows; row += nwaves) {
      const float *x = X + row * L;
      float *y = Y + row * L;
      float mean = 0.0f;
      for (int j = lane; j < L; j += 64)
         mean += x[j];
#pragma unroll
      for (int off = 32; off >= 1; off >>= 1)
         mean += __shfl_xor(mean, off, 64);
      mean = __fdiv_rn(mean, (float)L);
      float sum = 0.0f;
      for (int j = lane; j < L; j += 64) {
         const float tmp = x[j] - mean;
         sum += mul_nofma(tmp, tmp);
      }
#pragma unroll
      for (int off = 32; off >= 1; off >>= 1)
         sum += __shfl_xor(sum, off, 64);
      const float inv_std = __fdiv_rn(1.0f, sqrtf(__fdiv_rn(sum, (float)L) + epsilon));
      if (lane == 0) {
         if (mean_out)
            mean_out[row] = mean;
         if (inv_std_out)
            inv_std_out[row] = inv_std;
      }
      for (int j = lane; j < L; j += 64) {
         float v = mul_nofma(mul_nofma(scale[j], inv_std), x[j] - mean);
         if (bias)
            v += bias[j];
         y[j] = v;
      }
   }
}

// The last step of an average whose integer plane sums already exist (a convolution added them up in its store).
__global__ __launch_bounds__(256) void plane_sums_to_average_kernel(float *__restrict__ Y, const int32_t *__restrict__ sums, int NC, int HW,
                                                                    float scale)
{
   const int i = blockIdx.x * blockDim.x + threadIdx.x;
   if (i < NC)
      Y[i] = __fdiv_rn(mul_nofma((float)sums[i], scale), (float)HW);
}

// The same, and the sums are cleared behind the read: a buffer that starts out zero is zero again for the next convolution.
__global__ __launch_bounds__(256) void plane_sums_take_average_kernel(float *__restrict__ Y, int32_t *__restrict__ sums, int NC, int HW, float scale)
{
   const int i = blockIdx.x * blockDim.x + threadIdx.x;
   if (i < NC) {
      Y[i] = __fdiv_rn(mul_nofma((float)sums[i], scale), (float)HW);
      sums[i] = 0;
   }
}

// NHWC int8 input with C a multiple of 16 (and 16-byte aligned): one workgroup per (image, block of 256 channels).
// A thread owns 16 consecutive channels and every (256 / chunks)-th pixel, reads 16 bytes per pixel, and the
// per-thread int32 sums are added up through LDS (integer sums: exact in any order).
__global__ __launch_bounds__(256) void gap_i8_nhwc_vec_kernel(float *__restrict__ Y, const int8_t *__restrict__ X, int C, int HW,
                                                               float scale)
{
   __shared__ int part[256][17];
   const int cblocks = (C + 255) / 256;
   const int img = blockIdx.x / cblocks, cb = blockIdx.x % cblocks;
   const int c_first = cb * 256;
   const int chunks = ((C - c_first) < 256 ? (C - c_first) : 256) / 16; // 16-channel chunks in this block: 1..16
   // threads beyond groups*chunks idle: the pixel groups must not overlap
   const int groups = 256 / chunks;
   const int chunk = threadIdx.x % chunks, group = threadIdx.x / chunks;
   int s[16];
#pragma unroll
   for (int k = 0; k < 16; ++k)
      s[k] = 0;
   if (group < groups) {
      const int8_t *p = X + (size_t)img * HW * C + c_first + chunk * 16;
      typedef int int4v __attribute__((ext_vector_type(4)));
      auto add16 = [&](const int4v &v) {
#pragma unroll
         for (int d = 0; d < 4; ++d)
#pragma unroll
            for (int b = 0; b < 4; ++b)
               s[4 * d + b] += (int)(int8_t)(v[d] >> (8 * b));
      };
      int i = group;
      // eight pixels per round: eight independent 16-byte loads in flight per lane
      for (; i + 7 * groups < HW; i += 8 * groups) {
         int4v v[8];
#pragma unroll
         for (int u = 0; u < 8; ++u)
            v[u] = *(const int4v *)(p + (size_t)(i + u * groups) * C);
#pragma unroll
         for (int u = 0; u < 8; ++u)
            add16(v[u]);
      }
      for (; i < HW; i += groups)
         add16(*(const int4v *)(p + (size_t)i * C));
   }
#pragma unroll
   for (int k = 0; k < 16; ++k)
      part[threadIdx.x][k] = s[k];
   __syncthreads();
   // thread t < chunks*16 finishes channel c_first + t: add the `groups` partial sums of that channel
   if ((int)threadIdx.x < chunks * 16) {
      const int ch = threadIdx.x / 16, k = threadIdx.x % 16;
      int tot = 0;
      for (int g = 0; g < groups; ++g)
         tot += part[g * chunks + ch][k];
      Y[(size_t)img * C + c_first + threadIdx.x] = __fdiv_rn(mul_nofma((float)tot, scale), (float)HW);
   }
}

// Y = (X - mean[c]) * fused_scale[c] + bias[c] (+ relu); element i belongs to channel (i / spatial) % C
__global__ __launch_bounds__(256) void batchnorm_f32_kernel(float *__restrict__ Y, const float *__restrict__ X,
                                                             const float *__restrict__ fused, const float *__restrict__ mean,
                                                             const float *__restrict__ bias, size_t n, int C, int spatial, int relu)
{
   const size_t stride = (size_t)gridDim.x * blockDim.x;
   for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += stride) {
      const int c = (int)((i / (size_t)spatial) % (size_t)C);
      float v = __fmul_rn(X[i] - mean[c], fused[c]) + bias[c];
      if (relu)
         v = v > 0.0f ? v : 0.0f;
      Y[i] = v;
   }
}

} // namespace sofie_hip

using namespace sofie_hip;

extern "C" {

int sofie_hip_quantize_linear(sofie_hip_ctx *ctx, int8_t *dst, const float *src, size_t n, float scale)
{
   SOFIE_HIP_REQUIRE(ctx != nullptr, "sofie_hip_quantize_linear: ctx is NULL");
   if (n == 0)
      return SOFIE_HIP_OK;
   SOFIE_HIP_REQUIRE(dst && src, "sofie_hip_quantize_linear: NULL pointer");
   SOFIE_HIP_REQUIRE(scale > 0.0f, "sofie_hip_quantize_linear: scale must be positive");
   const int vec = (((uintptr_t)src & 15) == 0) && (((uintptr_t)dst & 3) == 0);
   hipLaunchKernelGGL(quantize_linear_kernel, dim3(grid_for(vec ? (n + 15) / 16 : n)), dim3(256), 0, ctx->stream, dst, src, n, scale, vec);
   return launch_status("quantize_linear_kernel");
}

int sofie_hip_dequantize_linear_i8(sofie_hip_ctx *ctx, float *dst, const int8_t *src, size_t n, float scale)
{
   SOFIE_HIP_REQUIRE(ctx != nullptr, "sofie_hip_dequantize_linear_i8: ctx is NULL");
   if (n == 0)
      return SOFIE_HIP_OK;
   SOFIE_HIP_REQUIRE(dst && src, "sofie_hip_dequantize_linear_i8: NULL pointer");
   hipLaunchKernelGGL(dequantize_linear_kernel<int8_t>, dim3(grid_for(n)), dim3(256), 0, ctx->stream, dst, src, n, scale);
   return launch_status("dequantize_linear_kernel");
}

int sofie_hip_dequantize_linear_i32(sofie_hip_ctx *ctx, float *dst, const int32_t *src, size_t n, float scale)
{
   SOFIE_HIP_REQUIRE(ctx != nullptr, "sofie_hip_dequantize_linear_i32: ctx is NULL");
   if (n == 0)
      return SOFIE_HIP_OK;
   SOFIE_HIP_REQUIRE(dst && src, "sofie_hip_dequantize_linear_i32: NULL pointer");
   hipLaunchKernelGGL(dequantize_linear_kernel<int32_t>, dim3(grid_for(n)), dim3(256), 0, ctx->stream, dst, src, n, scale);
   return launch_status("dequantize_linear_kernel");
}

static int launch_unary_chain(sofie_hip_ctx *ctx, float *dst, const float *src, size_t n, const PostChain &chain)
{
   const int vec = (((uintptr_t)src & 15) == 0) && (((uintptr_t)dst & 15) == 0);
   hipLaunchKernelGGL(unary_f32_kernel, dim3(grid_for(vec ? (n + 3) / 4 : n)), dim3(256), 0, ctx->stream, dst, src, n, chain, vec);
   return launch_status("unary_f32_kernel");
}

int sofie_hip_unary_f32(sofie_hip_ctx *ctx, float *dst, const float *src, size_t n, int32_t act, float act_alpha)
{
   SOFIE_HIP_REQUIRE(ctx != nullptr, "sofie_hip_unary_f32: ctx is NULL");
   PostChain chain;
   int bad = 0;
   SOFIE_HIP_REQUIRE(make_post_chain(chain, act, act_alpha, nullptr, bad), "sofie_hip_unary_f32: unknown activation %d", act);
   if (n == 0)
      return SOFIE_HIP_OK;
   SOFIE_HIP_REQUIRE(dst && src, "sofie_hip_unary_f32: NULL pointer");
   return launch_unary_chain(ctx, dst, src, n, chain);
}

int sofie_hip_unary_chain_f32(sofie_hip_ctx *ctx, float *dst, const float *src, size_t n, const sofie_post_ops *ops)
{
   SOFIE_HIP_REQUIRE(ctx != nullptr && ops != nullptr, "sofie_hip_unary_chain_f32: NULL argument");
   PostChain chain;
   int bad = 0;
   SOFIE_HIP_REQUIRE(make_post_chain(chain, SOFIE_ACT_NONE, 0.0f, ops, bad),
                     "sofie_hip_unary_chain_f32: unknown operator %d (or more than %d operators)", bad, SOFIE_MAX_POST_OPS);
   if (n == 0)
      return SOFIE_HIP_OK;
   SOFIE_HIP_REQUIRE(dst && src, "sofie_hip_unary_chain_f32: NULL pointer");
   return launch_unary_chain(ctx, dst, src, n, chain);
}

int sofie_hip_add_f32(sofie_hip_ctx *ctx, const sofie_add_desc *d)
{
   return sofie_hip_binary_f32(ctx, d, SOFIE_BINARY_ADD, 0.0f);
}

int sofie_hip_binary_f32(sofie_hip_ctx *ctx, const sofie_add_desc *d, int32_t op, float param)
{
   SOFIE_HIP_REQUIRE(ctx && d, "sofie_hip_add_f32: NULL argument");
   SOFIE_HIP_REQUIRE(op >= SOFIE_BINARY_ADD && op <= SOFIE_BINARY_LAST, "sofie_hip_binary_f32: unknown operator %d", op);
   SOFIE_HIP_REQUIRE(d->rank >= 0 && d->rank <= 6, "sofie_hip_add_f32: rank %d not in [0,6]", d->rank);
   AddShape sh;
   sh.rank = d->rank;
   size_t n = 1;
   long long stride_a = 1, stride_b = 1;
   for (int i = d->rank - 1; i >= 0; --i) {
      SOFIE_HIP_REQUIRE(d->y_shape[i] >= 0, "sofie_hip_add_f32: negative dimension");
      SOFIE_HIP_REQUIRE((d->a_shape[i] == d->y_shape[i] || d->a_shape[i] == 1) &&
                           (d->b_shape[i] == d->y_shape[i] || d->b_shape[i] == 1),
                        "sofie_hip_add_f32: operand dimension %d cannot be broadcast to the output", i);
      sh.y[i] = d->y_shape[i];
      sh.sa[i] = (d->a_shape[i] == 1 && d->y_shape[i] != 1) ? 0 : stride_a;
      sh.sb[i] = (d->b_shape[i] == 1 && d->y_shape[i] != 1) ? 0 : stride_b;
      stride_a *= d->a_shape[i];
      stride_b *= d->b_shape[i];
      n *= (size_t)d->y_shape[i];
   }
   if (n == 0)
      return SOFIE_HIP_OK;
   SOFIE_HIP_REQUIRE(d->A && d->B && d->Y, "sofie_hip_add_f32: NULL pointer");
   if (op == SOFIE_BINARY_ADD) {
      hipLaunchKernelGGL(add_f32_kernel, dim3(grid_for(n)), dim3(256), 0, ctx->stream, d->Y, d->A, d->B, n, sh);
      return launch_status("add_f32_kernel");
   }
   hipLaunchKernelGGL(binary_f32_kernel, dim3(grid_for(n)), dim3(256), 0, ctx->stream, d->Y, d->A, d->B, n, sh, op, param);
   return launch_status("binary_f32_kernel");
}

int sofie_hip_batchnorm_f32(sofie_hip_ctx *ctx, float *Y, const float *X, const float *fused_scale, const float *mean,
                            const float *bias, int32_t N, int32_t C, int32_t spatial, int32_t relu)
{
   SOFIE_HIP_REQUIRE(ctx != nullptr, "sofie_hip_batchnorm_f32: ctx is NULL");
   SOFIE_HIP_REQUIRE(N >= 0 && C > 0 && spatial > 0, "sofie_hip_batchnorm_f32: bad shape");
   if (N == 0)
      return SOFIE_HIP_OK;
   SOFIE_HIP_REQUIRE(Y && X && fused_scale && mean && bias, "sofie_hip_batchnorm_f32: NULL pointer");
   const size_t n = (size_t)N * (size_t)C * (size_t)spatial;
   hipLaunchKernelGGL(batchnorm_f32_kernel, dim3(grid_for(n)), dim3(256), 0, ctx->stream, Y, X, fused_scale, mean, bias, n, C, spatial, relu);
   return launch_status("batchnorm_f32_kernel");
}

int sofie_hip_pool3d_f32(sofie_hip_ctx *ctx, const sofie_pool3d_desc *d, float *Y, const float *X)
{
   SOFIE_HIP_REQUIRE(ctx && d, "sofie_hip_pool3d_f32: NULL argument");
   SOFIE_HIP_REQUIRE(d->planes >= 0, "sofie_hip_pool3d_f32: bad shape");
   SOFIE_HIP_REQUIRE(d->mode == SOFIE_POOL_MAX || d->mode == SOFIE_POOL_AVERAGE, "sofie_hip_pool3d_f32: unknown mode %d", d->mode);
   long long total = d->planes, in_total = d->planes;
   for (int a = 0; a < 3; ++a) {
      SOFIE_HIP_REQUIRE(d->in[a] > 0 && d->out[a] > 0 && d->k[a] > 0, "sofie_hip_pool3d_f32: bad shape");
      SOFIE_HIP_REQUIRE(d->stride[a] > 0, "sofie_hip_pool3d_f32: bad stride");
      SOFIE_HIP_REQUIRE(d->pad_begin[a] >= 0 && d->pad_end[a] >= 0, "sofie_hip_pool3d_f32: negative padding");
      // every window start must lie where the reference's loops put it: the last one begins inside the padded volume
      SOFIE_HIP_REQUIRE((long long)(d->out[a] - 1) * d->stride[a] - d->pad_begin[a] < d->in[a] + d->pad_end[a],
                        "sofie_hip_pool3d_f32: the output extent %d of axis %d does not fit the padded input", d->out[a], a);
      total *= d->out[a];
      in_total *= d->in[a];
      SOFIE_HIP_REQUIRE(total < (1LL << 40) && in_total < (1LL << 40), "sofie_hip_pool3d_f32: tensor too large");
   }
   if (total == 0)
      return SOFIE_HIP_OK;
   SOFIE_HIP_REQUIRE(Y && X, "sofie_hip_pool3d_f32: NULL pointer");
   hipLaunchKernelGGL(pool_f32_kernel, dim3(grid_for((size_t)total)), dim3(256), 0, ctx->stream, Y, X, *d, (size_t)total);
   return launch_status("pool_f32_kernel");
}

int sofie_hip_pool_f32(sofie_hip_ctx *ctx, const sofie_pool_desc *d, float *Y, const float *X)
{
   SOFIE_HIP_REQUIRE(ctx && d, "sofie_hip_pool_f32: NULL argument");
   SOFIE_HIP_REQUIRE(d->planes >= 0 && d->H > 0 && d->W > 0 && d->OH > 0 && d->OW > 0 && d->kh > 0 && d->kw > 0, "sofie_hip_pool_f32: bad shape");
   SOFIE_HIP_REQUIRE(d->stride_h > 0 && d->stride_w > 0, "sofie_hip_pool_f32: bad stride");
   SOFIE_HIP_REQUIRE(d->pad_h0 >= 0 && d->pad_w0 >= 0 && d->pad_h1 >= 0 && d->pad_w1 >= 0, "sofie_hip_pool_f32: negative padding");
   SOFIE_HIP_REQUIRE(d->mode == SOFIE_POOL_MAX || d->mode == SOFIE_POOL_AVERAGE, "sofie_hip_pool_f32: unknown mode %d", d->mode);
   // every window start must lie where the reference's loops put it: the last one begins inside the padded image
   SOFIE_HIP_REQUIRE((long long)(d->OH - 1) * d->stride_h - d->pad_h0 < d->H + d->pad_h1 &&
                        (long long)(d->OW - 1) * d->stride_w - d->pad_w0 < d->W + d->pad_w1,
                     "sofie_hip_pool_f32: the output shape %dx%d does not fit the padded input", d->OH, d->OW);
   // a volume of depth one
   sofie_pool3d_desc v{};
   v.planes = d->planes;
   v.in[0] = 1, v.in[1] = d->H, v.in[2] = d->W;
   v.out[0] = 1, v.out[1] = d->OH, v.out[2] = d->OW;
   v.k[0] = 1, v.k[1] = d->kh, v.k[2] = d->kw;
   v.pad_begin[0] = 0, v.pad_begin[1] = d->pad_h0, v.pad_begin[2] = d->pad_w0;
   v.pad_end[0] = 0, v.pad_end[1] = d->pad_h1, v.pad_end[2] = d->pad_w1;
   v.stride[0] = 1, v.stride[1] = d->stride_h, v.stride[2] = d->stride_w;
   v.mode = d->mode, v.count_include_pad = d->count_include_pad, v.dynamic_divisor = d->dynamic_divisor;
   return sofie_hip_pool3d_f32(ctx, &v, Y, X);
}

int sofie_hip_global_avg_pool_f32(sofie_hip_ctx *ctx, float *Y, const float *X, int32_t NC, int32_t HW)
{
   SOFIE_HIP_REQUIRE(ctx != nullptr, "sofie_hip_global_avg_pool_f32: ctx is NULL");
   SOFIE_HIP_REQUIRE(NC >= 0 && HW > 0, "sofie_hip_global_avg_pool_f32: bad shape");
   if (NC == 0)
      return SOFIE_HIP_OK;
   SOFIE_HIP_REQUIRE(Y && X, "sofie_hip_global_avg_pool_f32: NULL pointer");
   hipLaunchKernelGGL((gap_kernel<float, float>), dim3((NC + 3) / 4), dim3(256), 0, ctx->stream, Y, X, NC, HW, 1.0f);
   return launch_status("gap_kernel");
}

int sofie_hip_global_avg_pool_i8(sofie_hip_ctx *ctx, float *Y, const int8_t *X, int32_t N, int32_t C, int32_t HW,
                                 int32_t x_layout, float scale)
{
   SOFIE_HIP_REQUIRE(ctx != nullptr, "sofie_hip_global_avg_pool_i8: ctx is NULL");
   SOFIE_HIP_REQUIRE(N >= 0 && C > 0 && HW > 0, "sofie_hip_global_avg_pool_i8: bad shape");
   SOFIE_HIP_REQUIRE(x_layout == SOFIE_LAYOUT_NCHW || x_layout == SOFIE_LAYOUT_NHWC, "sofie_hip_global_avg_pool_i8: unknown layout");
   SOFIE_HIP_REQUIRE((long long)N * C < (1LL << 31), "sofie_hip_global_avg_pool_i8: too many planes");
   if (N == 0)
      return SOFIE_HIP_OK;
   SOFIE_HIP_REQUIRE(Y && X, "sofie_hip_global_avg_pool_i8: NULL pointer");
   if (x_layout == SOFIE_LAYOUT_NHWC) {
      if (C % 16 == 0 && (((uintptr_t)X & 15) == 0) && (long long)N * ((C + 255) / 256) < 0x7fffffffLL) {
         hipLaunchKernelGGL(gap_i8_nhwc_vec_kernel, dim3((unsigned)(N * ((C + 255) / 256))), dim3(256), 0, ctx->stream, Y, X, C, HW,
                            scale);
         return launch_status("gap_i8_nhwc_vec_kernel");
      }
      hipLaunchKernelGGL(gap_i8_nhwc_kernel, dim3((unsigned)N), dim3(256), 0, ctx->stream, Y, X, C, HW, scale);
      return launch_status("gap_i8_nhwc_kernel");
   }
   const int NC = N * C;
   hipLaunchKernelGGL((gap_kernel<int8_t, int>), dim3((NC + 3) / 4), dim3(256), 0, ctx->stream, Y, X, NC, HW, scale);
   return launch_status("gap_kernel");
}

int sofie_hip_transpose_f32(sofie_hip_ctx *ctx, float *Y, const float *X, int32_t rank, const int64_t *shape, const int32_t *perm)
{
   SOFIE_HIP_REQUIRE(ctx && shape && perm, "sofie_hip_transpose_f32: NULL argument");
   SOFIE_HIP_REQUIRE(rank >= 1 && rank <= 6, "sofie_hip_transpose_f32: rank %d not in [1,6]", rank);
   long long in_stride[6];
   size_t n = 1;
   unsigned seen = 0;
   for (int d = rank - 1; d >= 0; --d) {
      SOFIE_HIP_REQUIRE(shape[d] >= 0 && shape[d] < (1LL << 40), "sofie_hip_transpose_f32: bad dimension");
      in_stride[d] = (long long)n;
      n *= (size_t)shape[d];
      SOFIE_HIP_REQUIRE(n < (1ULL << 40), "sofie_hip_transpose_f32: tensor too large");
   }
   TransposeShape sh;
   sh.rank = rank;
   for (int k = 0; k < rank; ++k) {
      SOFIE_HIP_REQUIRE(perm[k] >= 0 && perm[k] < rank && !(seen & (1u << perm[k])), "sofie_hip_transpose_f32: perm is not a permutation of 0..%d", rank - 1);
      seen |= 1u << perm[k];
      sh.y[k] = shape[perm[k]];
      sh.sx[k] = in_stride[perm[k]];
   }
   if (n == 0)
      return SOFIE_HIP_OK;
   SOFIE_HIP_REQUIRE(Y && X, "sofie_hip_transpose_f32: NULL pointer");
   hipLaunchKernelGGL(transpose_f32_kernel, dim3(grid_for(n)), dim3(256), 0, ctx->stream, Y, X, n, sh);
   return launch_status("transpose_f32_kernel");
}

int sofie_hip_strided_gather_f32(sofie_hip_ctx *ctx, float *Y, const float *X, int32_t rank, const int64_t *out_shape, const int64_t *in_strides,
                                 int64_t in_offset, int64_t in_elements)
{
   SOFIE_HIP_REQUIRE(ctx && out_shape && in_strides, "sofie_hip_strided_gather_f32: NULL argument");
   SOFIE_HIP_REQUIRE(rank >= 1 && rank <= 6, "sofie_hip_strided_gather_f32: rank %d not in [1,6]", rank);
   SOFIE_HIP_REQUIRE(in_elements >= 0 && in_elements < (1LL << 40) && in_offset >= 0, "sofie_hip_strided_gather_f32: bad input size or offset");
   TransposeShape sh;
   sh.rank = rank;
   size_t n = 1;
   long long lo = in_offset, hi = in_offset; // the smallest and the largest input index the output reads
   for (int k = 0; k < rank; ++k) {
      SOFIE_HIP_REQUIRE(out_shape[k] >= 0 && out_shape[k] < (1LL << 40), "sofie_hip_strided_gather_f32: bad dimension");
      SOFIE_HIP_REQUIRE(in_strides[k] > -(1LL << 40) && in_strides[k] < (1LL << 40), "sofie_hip_strided_gather_f32: bad stride");
      n *= (size_t)out_shape[k];
      SOFIE_HIP_REQUIRE(n < (1ULL << 40), "sofie_hip_strided_gather_f32: tensor too large");
      sh.y[k] = out_shape[k];
      sh.sx[k] = in_strides[k];
   }
   if (n == 0)
      return SOFIE_HIP_OK;
   for (int k = 0; k < rank; ++k) {
      const double span = (double)(out_shape[k] - 1) * (double)in_strides[k];
      SOFIE_HIP_REQUIRE(span > -1.0e15 && span < 1.0e15, "sofie_hip_strided_gather_f32: axis %d reaches outside the input", k);
      (in_strides[k] < 0 ? lo : hi) += (long long)(out_shape[k] - 1) * in_strides[k];
   }
   SOFIE_HIP_REQUIRE(lo >= 0 && hi < in_elements, "sofie_hip_strided_gather_f32: reads elements %lld..%lld of an input of %lld", lo, hi, (long long)in_elements);
   SOFIE_HIP_REQUIRE(Y && X, "sofie_hip_strided_gather_f32: NULL pointer");
   hipLaunchKernelGGL(transpose_f32_kernel, dim3(grid_for(n)), dim3(256), 0, ctx->stream, Y, X + in_offset, n, sh);
   return launch_status("transpose_f32_kernel");
}

int sofie_hip_copy_rows(sofie_hip_ctx *ctx, void *dst, size_t dst_pitch_bytes, const void *src, size_t src_pitch_bytes, size_t rows, size_t row_bytes)
{
   SOFIE_HIP_REQUIRE(ctx != nullptr, "sofie_hip_copy_rows: ctx is NULL");
   SOFIE_HIP_REQUIRE(row_bytes % 4 == 0 && dst_pitch_bytes % 4 == 0 && src_pitch_bytes % 4 == 0, "sofie_hip_copy_rows: sizes must be multiples of 4 bytes");
   SOFIE_HIP_REQUIRE(dst_pitch_bytes >= row_bytes && src_pitch_bytes >= row_bytes, "sofie_hip_copy_rows: a pitch is smaller than the row");
   SOFIE_HIP_REQUIRE(rows < (1ULL << 40) && row_bytes < (1ULL << 40) && (double)rows * (double)row_bytes < 1.0e13, "sofie_hip_copy_rows: too large");
   if (rows == 0 || row_bytes == 0)
      return SOFIE_HIP_OK;
   SOFIE_HIP_REQUIRE(dst && src && (((uintptr_t)dst | (uintptr_t)src) & 3) == 0, "sofie_hip_copy_rows: NULL or misaligned pointer");
   hipLaunchKernelGGL(copy_rows_kernel, dim3(grid_for(rows * (row_bytes / 4))), dim3(256), 0, ctx->stream, (uint32_t *)dst, dst_pitch_bytes / 4,
                      (const uint32_t *)src, src_pitch_bytes / 4, rows, row_bytes / 4);
   return launch_status("copy_rows_kernel");
}

int sofie_hip_softmax_f32(sofie_hip_ctx *ctx, float *Y, const float *X, int64_t outer, int32_t axis_len, int64_t inner, int32_t log_softmax)
{
   SOFIE_HIP_REQUIRE(ctx != nullptr, "sofie_hip_softmax_f32: ctx is NULL");
   SOFIE_HIP_REQUIRE(outer >= 0 && axis_len > 0 && inner > 0, "sofie_hip_softmax_f32: bad shape");
   SOFIE_HIP_REQUIRE(outer < (1LL << 40) && inner < (1LL << 40) && (double)outer * axis_len * (double)inner < 1.0e12, "sofie_hip_softmax_f32: tensor too large");
   const long long lines = (long long)outer * inner;
   if (lines == 0)
      return SOFIE_HIP_OK;
   SOFIE_HIP_REQUIRE(Y && X, "sofie_hip_softmax_f32: NULL pointer");
   const long long blocks = (lines + 3) / 4;
   hipLaunchKernelGGL(softmax_f32_kernel, dim3((unsigned)(blocks < 256 * 64 ? blocks : 256 * 64)), dim3(256), 0, ctx->stream, Y, X, lines, axis_len,
                      (long long)inner, log_softmax);
   return launch_status("softmax_f32_kernel");
}

int sofie_hip_reduce_f32(sofie_hip_ctx *ctx, float *Y, const float *X, int64_t outer, int32_t A, int64_t inner, int32_t op)
{
   SOFIE_HIP_REQUIRE(ctx != nullptr, "sofie_hip_reduce_f32: ctx is NULL");
   SOFIE_HIP_REQUIRE(op >= SOFIE_REDUCE_SUM && op <= SOFIE_REDUCE_MIN, "sofie_hip_reduce_f32: unknown operator %d", op);
   SOFIE_HIP_REQUIRE(outer >= 0 && A > 0 && inner > 0 && outer < (1LL << 40) && inner < (1LL << 40) && (double)outer * A * (double)inner < 1.0e12,
                     "sofie_hip_reduce_f32: bad shape");
   const long long outputs = (long long)outer * inner;
   if (outputs == 0)
      return SOFIE_HIP_OK;
   SOFIE_HIP_REQUIRE(Y && X, "sofie_hip_reduce_f32: NULL pointer");
   if (inner == 1 && A >= 64 && outputs < 16384) {
      hipLaunchKernelGGL(reduce_lines_f32_kernel, dim3((unsigned)((outputs + 3) / 4)), dim3(256), 0, ctx->stream, Y, X, outputs, A, op);
      return launch_status("reduce_lines_f32_kernel");
   }
   hipLaunchKernelGGL(reduce_f32_kernel, dim3(grid_for((size_t)outputs)), dim3(256), 0, ctx->stream, Y, X, (size_t)outputs, A, (long long)inner, op);
   return launch_status("reduce_f32_kernel");
}

int sofie_hip_layernorm_f32(sofie_hip_ctx *ctx, float *Y, const float *X, const float *scale, const float *bias, int64_t rows, int32_t L, float epsilon,
                            float *mean_out, float *inv_std_out)
{
   SOFIE_HIP_REQUIRE(ctx != nullptr, "sofie_hip_layernorm_f32: ctx is NULL");
   SOFIE_HIP_REQUIRE(rows >= 0 && L > 0 && rows < (1LL << 40) && (double)rows * L < 1.0e12, "sofie_hip_layernorm_f32: bad shape");
   SOFIE_HIP_REQUIRE(epsilon >= 0.0f, "sofie_hip_layernorm_f32: epsilon is negative");
   if (rows == 0)
      return SOFIE_HIP_OK;
   SOFIE_HIP_REQUIRE(Y && X && scale, "sofie_hip_layernorm_f32: NULL pointer");
   const long long blocks = (rows + 3) / 4;
   hipLaunchKernelGGL(layernorm_f32_kernel, dim3((unsigned)(blocks < 256 * 64 ? blocks : 256 * 64)), dim3(256), 0, ctx->stream, Y, X, scale, bias, (long long)rows, L,
                      epsilon, mean_out, inv_std_out);
   return launch_status("layernorm_f32_kernel");
}

int sofie_hip_plane_sums_to_average(sofie_hip_ctx *ctx, float *Y, const int32_t *sums, int32_t NC, int32_t HW, float scale)
{
   SOFIE_HIP_REQUIRE(ctx != nullptr, "sofie_hip_plane_sums_to_average: ctx is NULL");
   SOFIE_HIP_REQUIRE(NC >= 0 && HW > 0, "sofie_hip_plane_sums_to_average: bad shape");
   if (NC == 0)
      return SOFIE_HIP_OK;
   SOFIE_HIP_REQUIRE(Y && sums, "sofie_hip_plane_sums_to_average: NULL pointer");
   hipLaunchKernelGGL(plane_sums_to_average_kernel, dim3((NC + 255) / 256), dim3(256), 0, ctx->stream, Y, sums, NC, HW, scale);
   return launch_status("plane_sums_to_average_kernel");
}

int sofie_hip_plane_sums_take_average(sofie_hip_ctx *ctx, float *Y, int32_t *sums, int32_t NC, int32_t HW, float scale)
{
   SOFIE_HIP_REQUIRE(ctx != nullptr, "sofie_hip_plane_sums_take_average: ctx is NULL");
   SOFIE_HIP_REQUIRE(NC >= 0 && HW > 0, "sofie_hip_plane_sums_take_average: bad shape");
   if (NC == 0)
      return SOFIE_HIP_OK;
   SOFIE_HIP_REQUIRE(Y && sums, "sofie_hip_plane_sums_take_average: NULL pointer");
   hipLaunchKernelGGL(plane_sums_take_average_kernel, dim3((NC + 255) / 256), dim3(256), 0, ctx->stream, Y, sums, NC, HW, scale);
   return launch_status("plane_sums_take_average_kernel");
}

} // extern "C"
