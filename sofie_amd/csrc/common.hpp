// Shared declarations of the gfx950 runtime behind include/sofie_hip.h.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include "sofie_hip.h"

struct sofie_hip_ctx {
   int device = 0;
   hipStream_t stream = nullptr;
   bool owns_stream = false;
   char *arena = nullptr;
   size_t arena_bytes = 0;
   bool owns_arena = false;
   hipEvent_t ev0 = nullptr, ev1 = nullptr;
};

namespace sofie_hip {

// Records the text returned by sofie_hip_last_error() for the calling thread and returns `code`.
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

#define SOFIE_HIP_CHECK(expr)                                                                         \
   do {                                                                                               \
      hipError_t e_ = (expr);                                                                         \
      if (e_ != hipSuccess)                                                                           \
         return ::sofie_hip::fail(SOFIE_HIP_ERR_RUNTIME, "%s failed: %s (%s:%d)", #expr,              \
                                  hipGetErrorString(e_), __FILE__, __LINE__);                         \
   } while (0)

#define SOFIE_HIP_REQUIRE(cond, ...)                                                                  \
   do {                                                                                               \
      if (!(cond))                                                                                    \
         return ::sofie_hip::fail(SOFIE_HIP_ERR_INVALID, __VA_ARGS__);                                \
   } while (0)

inline int launch_status(const char *what)
{
   hipError_t e = hipGetLastError();
   if (e != hipSuccess)
      return fail(SOFIE_HIP_ERR_RUNTIME, "launch of %s failed: %s", what, hipGetErrorString(e));
   return SOFIE_HIP_OK;
}

// ---- scalar formulas shared by every epilogue --------------------------------------------------

// Activation on fp32, the reference's CPU formulas (see sofie_hip.h for the citations).
__device__ __forceinline__ float apply_act(float v, int act, float alpha, float beta = 0.0f)
{
   switch (act) {
   case SOFIE_ACT_RELU: return (v > 0.0f) ? v : 0.0f;
   case SOFIE_ACT_LEAKYRELU: return (v >= 0.0f) ? v : alpha * v;
   case SOFIE_ACT_SIGMOID: return 1.0f / (1.0f + expf(-v));
   case SOFIE_ACT_GELU: return 0.5f * v * (1.0f + erff(v * 0.7071067811865475f));
   case SOFIE_ACT_GELU_TANH: return 0.5f * v * (1.0f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v)));
   case SOFIE_ACT_TANH: return tanhf(v);
   case SOFIE_ACT_RECIPROCAL: return 1.0f / v;
   case SOFIE_ACT_SQRT: return sqrtf(v);
   case SOFIE_ACT_NEG: return -v;
   case SOFIE_ACT_EXP: return expf(v);
   case SOFIE_ACT_LOG: return logf(v);
   case SOFIE_ACT_SIN: return sinf(v);
   case SOFIE_ACT_COS: return cosf(v);
   case SOFIE_ACT_ABS: return fabsf(v);
   case SOFIE_ACT_SOFTPLUS: return (v >= 20.0f) ? v : log1pf(expf(v));
   case SOFIE_ACT_ATAN: return atanf(v);
   case SOFIE_ACT_FLOOR: return floorf(v);
   case SOFIE_ACT_ASINH: return asinhf(v);
   case SOFIE_ACT_ACOSH: return acoshf(v);
   case SOFIE_ACT_ATANH: return atanhf(v);
   case SOFIE_ACT_CLIP: return fmaxf(alpha, fminf(beta, v));
   default: return v;
   }
}

// An operator's own activation followed by the caller's chain of one-to-one operators, by value in the kernel
// arguments; `count` is the same for every lane, so the loop does not diverge.
struct PostChain {
   int count = 0;
   int op[SOFIE_MAX_POST_OPS + 1];
   float alpha[SOFIE_MAX_POST_OPS + 1];
   float beta[SOFIE_MAX_POST_OPS + 1];
};

__device__ __forceinline__ float apply_chain(float v, const PostChain &c)
{
   for (int i = 0; i < c.count; ++i)
      v = apply_act(v, c.op[i], c.alpha[i], c.beta[i]);
   return v;
}

// Host side: checks the codes and builds the chain {act, post...}.  Returns false (with `bad` set to the offending
// code, or -1 for a bad count) if anything is out of range.
inline bool make_post_chain(PostChain &c, int act, float act_alpha, const sofie_post_ops *post, int &bad)
{
   c.count = 0;
   bad = act;
   if (act < SOFIE_ACT_NONE || act > SOFIE_ACT_LAST)
      return false;
   if (act != SOFIE_ACT_NONE) {
      c.op[0] = act;
      c.alpha[0] = act_alpha;
      c.beta[0] = 0.0f;
      c.count = 1;
   }
   if (!post)
      return true;
   bad = -1;
   if (post->count < 0 || post->count > SOFIE_MAX_POST_OPS)
      return false;
   for (int i = 0; i < post->count; ++i) {
      bad = post->op[i];
      if (post->op[i] < SOFIE_ACT_NONE || post->op[i] > SOFIE_ACT_LAST)
         return false;
      if (post->op[i] == SOFIE_ACT_NONE)
         continue;
      c.op[c.count] = post->op[i];
      c.alpha[c.count] = post->alpha[i];
      c.beta[c.count] = post->beta[i];
      ++c.count;
   }
   return true;
}

// sat8(rne(v)): round half to even, saturate to [-128,127]; NaN -> 0 (matches the CPU restatement,
// which clamps before converting and maps NaN to 0).
__device__ __forceinline__ int quantize_rne_sat8(float v)
{
   if (!(v == v))
      return 0;
   float r = __builtin_rintf(v); // v_rndne_f32
   r = fminf(fmaxf(r, -128.0f), 127.0f);
   return (int)r;
}

// The same function for the GEMM store, where it runs once per output element: v_rndne_f32, then
// v_cvt_i32_f32, which by itself saturates to the int32 range and turns NaN into 0, then an integer clamp
// to [lo, 127] (lo = -128, or 0 when a relu follows: max(sat8(x), 0) == clamp(x, 0, 127)).
__device__ __forceinline__ int quantize_rne_clamp(float v, int lo)
{
   const float r = __builtin_rintf(v);
   int q;
   asm("v_cvt_i32_f32 %0, %1" : "=v"(q) : "v"(r));
   int c;
   asm("v_med3_i32 %0, %1, %2, %3" : "=v"(c) : "v"(q), "s"(lo), "v"(127)); // lo <= 127: the median is the clamp
   return c;
}

// fp32 multiply that the compiler may not fuse with a neighbouring add.
__device__ __forceinline__ float mul_nofma(float a, float b)
{
   return __fmul_rn(a, b);
}

} // namespace sofie_hip
