// Shared declarations of the gfx950 runtime behind include/sofie_hip.h.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include "sofie_hip.h"

// Kernel-choice overrides of a context (tuning and tests).  Read from the environment ONCE, when the context is created
// (SOFIE_HIP_SWIZZLE, SOFIE_HIP_I8_TILE, SOFIE_HIP_F8_TILE, SOFIE_HIP_GEMM_VARIANT, SOFIE_HIP_CONV_EXPLICIT,
// SOFIE_HIP_F32_SKINNY, SOFIE_HIP_F32_CHAIN), afterwards changed only through sofie_hip_ctx_set_option.
struct sofie_hip_options {
   int swizzle = 4;       // tile order: XCD regrouping, bands of 4 tile rows
   int i8_tile = 0;       // 0 = heuristic
   int f8_tile = 0;
   int gemm_variant = 0;  // alternative pipelined kernel (1), general kernel only (-1)
   int conv_explicit = 0; // int8 convolution through a column matrix whenever the workspace holds one
   int f32_skinny = -1;   // -1 = heuristic
   int f32_chain = -1;
};

struct sofie_hip_ctx {
   sofie_hip_options opt;
   int device = 0;
   hipStream_t stream = nullptr;
   bool owns_stream = false;
   char *arena = nullptr;
   size_t arena_bytes = 0;
   bool owns_arena = false;
   hipEvent_t ev0 = nullptr, ev1 = nullptr;
};

namespace sofie_hip {

// What a launch of the int8 / FP8 GEMM kernels needs from the context: the stream and the kernel-choice overrides.
struct LaunchCfg {
   hipStream_t stream;
   int tile;    // forced tile configuration, 0 = heuristic
   int variant; // alternative of the pipelined kernel
   int swizzle; // tile order (tile_of_block)
};
inline LaunchCfg launch_cfg_i8(const sofie_hip_ctx *ctx) { return LaunchCfg{ctx->stream, ctx->opt.i8_tile, ctx->opt.gemm_variant, ctx->opt.swizzle}; }
inline LaunchCfg launch_cfg_f8(const sofie_hip_ctx *ctx) { return LaunchCfg{ctx->stream, ctx->opt.f8_tile, ctx->opt.gemm_variant, ctx->opt.swizzle}; }

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
__device__ __forceinline__ float apply_activation(float v, int act, float alpha)
{
   switch (act) {
   case SOFIE_ACT_RELU: return (v > 0.0f) ? v : 0.0f;
   case SOFIE_ACT_LEAKYRELU: return (v >= 0.0f) ? v : alpha * v;
   case SOFIE_ACT_SIGMOID: return 1.0f / (1.0f + expf(-v));
   case SOFIE_ACT_GELU: return 0.5f * v * (1.0f + erff(v * 0.7071067811865475f));
   case SOFIE_ACT_GELU_TANH: return 0.5f * v * (1.0f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v)));
   case SOFIE_ACT_TANH: return tanhf(v);
   default: return v;
   }
}

// The other one-to-one operators (codes above SOFIE_ACT_TANH).  Kept out of line: the kernels that carry an
// epilogue stay as small as they were with the six activations, and pay a call only when a model uses these.
static __device__ __noinline__ float apply_basic_unary(float v, int act, float alpha, float beta)
{
   switch (act) {
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
   case SOFIE_ACT_SELU: return beta * (fmaxf(0.0f, v) + fminf(0.0f, alpha * (expf(v) - 1.0f)));
   case SOFIE_ACT_ELU: return v >= 0.0f ? v : alpha * (expf(v) - 1.0f);
   case SOFIE_ACT_ERF: return erff(v);
   case SOFIE_ACT_HARDSIGMOID: return fmaxf(0.0f, fminf(1.0f, alpha * v + beta));
   case SOFIE_ACT_HARDSWISH: return v * fmaxf(0.0f, fminf(1.0f, 0x1.5555555555555p-3f * v + 0.5f));
   case SOFIE_ACT_SWISH: return v / (1.0f + expf(-v));
   default: return v;
   }
}

__device__ __forceinline__ float apply_act(float v, int act, float alpha, float beta = 0.0f)
{
   return act <= SOFIE_ACT_TANH ? apply_activation(v, act, alpha) : apply_basic_unary(v, act, alpha, beta);
}

// An operator's own activation followed by the caller's chain of one-to-one operators, by value in the kernel
// arguments.  The links are named fields, not arrays: every access has a fixed offset, so the chain stays in
// scalar registers (an array indexed by a loop counter would be copied to private memory).
struct PostChain {
   int count = 0;
   int op0 = 0, op1 = 0, op2 = 0, op3 = 0, op4 = 0;
   float a0 = 0, a1 = 0, a2 = 0, a3 = 0, a4 = 0;
   float b0 = 0, b1 = 0, b2 = 0, b3 = 0, b4 = 0;
};
static_assert(SOFIE_MAX_POST_OPS == 4, "PostChain holds the activation and four links");

// links 1..4, out of line (a model with more than one link behind an operator pays one call per element)
static __device__ __noinline__ float apply_chain_tail(float v, int count, int op1, float a1, float b1, int op2, float a2, float b2, int op3,
                                               float a3, float b3, int op4, float a4, float b4)
{
   v = apply_act(v, op1, a1, b1);
   if (count > 2)
      v = apply_act(v, op2, a2, b2);
   if (count > 3)
      v = apply_act(v, op3, a3, b3);
   if (count > 4)
      v = apply_act(v, op4, a4, b4);
   return v;
}

__device__ __forceinline__ float apply_chain(float v, const PostChain &c)
{
   if (c.count > 0)
      v = apply_act(v, c.op0, c.a0, c.b0);
   if (c.count > 1)
      v = apply_chain_tail(v, c.count, c.op1, c.a1, c.b1, c.op2, c.a2, c.b2, c.op3, c.a3, c.b3, c.op4, c.a4, c.b4);
   return v;
}

// Host side: checks the codes and builds the chain {act, post...}.  Returns false (with `bad` set to the offending
// code, or -1 for a bad count) if anything is out of range.
inline bool make_post_chain(PostChain &c, int act, float act_alpha, const sofie_post_ops *post, int &bad)
{
   c = PostChain();
   int ops[SOFIE_MAX_POST_OPS + 1];
   float al[SOFIE_MAX_POST_OPS + 1], be[SOFIE_MAX_POST_OPS + 1];
   int n = 0;
   bad = act;
   if (act < SOFIE_ACT_NONE || act > SOFIE_ACT_LAST)
      return false;
   if (act != SOFIE_ACT_NONE) {
      ops[n] = act;
      al[n] = act_alpha;
      be[n] = 0.0f;
      ++n;
   }
   if (post) {
      bad = -1;
      if (post->count < 0 || post->count > SOFIE_MAX_POST_OPS)
         return false;
      for (int i = 0; i < post->count; ++i) {
         bad = post->op[i];
         if (post->op[i] < SOFIE_ACT_NONE || post->op[i] > SOFIE_ACT_LAST)
            return false;
         if (post->op[i] == SOFIE_ACT_NONE)
            continue;
         ops[n] = post->op[i];
         al[n] = post->alpha[i];
         be[n] = post->beta[i];
         ++n;
      }
   }
   for (int i = n; i <= SOFIE_MAX_POST_OPS; ++i) {
      ops[i] = SOFIE_ACT_NONE;
      al[i] = be[i] = 0.0f;
   }
   c.count = n;
   c.op0 = ops[0]; c.op1 = ops[1]; c.op2 = ops[2]; c.op3 = ops[3]; c.op4 = ops[4];
   c.a0 = al[0]; c.a1 = al[1]; c.a2 = al[2]; c.a3 = al[3]; c.a4 = al[4];
   c.b0 = be[0]; c.b1 = be[1]; c.b2 = be[2]; c.b3 = be[3]; c.b4 = be[4];
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
