/* sofie_hip.h -- C-ABI of the gfx950 (MI355X) runtime that SOFIE-emitted Session code calls.
 *
 * Every entry point is plain C: pointers, sizes, POD descriptors.  No C++ or torch types cross
 * this boundary.  All functions return 0 on success and a non-zero status on failure; the text
 * of the last failure on the calling thread is returned by sofie_hip_last_error().  The emitted
 * C++ Session turns a non-zero status into std::runtime_error, which is the error convention of
 * the reference's generated code (core/src/RModel.cxx:1839-1841, 1386-1389).
 *
 * Threading: a context is used by one thread at a time (the reference's rule is one Session per
 * thread, core/inc/SOFIE/utils/SOFIEHelpers.hxx:31-51).  Different contexts are independent.
 *
 * Pointers in descriptors are DEVICE pointers unless the parameter says "host".  A Session
 * normally forms them as arena base + planned offset (sofie_hip_arena_ptr).
 */
#ifndef SOFIE_HIP_H
#define SOFIE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Version of this interface: raised whenever an entry point is added, removed or changes its meaning (3: the kernel-choice
 * options are read from the environment once, when a context is created, and changed through sofie_hip_ctx_set_option; entry
 * points added for 3-D operators and for callers that cannot allocate; 4: sofie_hip_plane_sums_take_average added).  An
 * emitted Session compares the value it was compiled with against sofie_hip_abi_version() of the library it finds at run
 * time, and refuses to run on a different one. */
#define SOFIE_HIP_ABI_VERSION 4

typedef struct sofie_hip_ctx sofie_hip_ctx;

/* ---- status codes ------------------------------------------------------------------------- */
enum {
   SOFIE_HIP_OK = 0,
   SOFIE_HIP_ERR_INVALID = 1,  /* bad argument / unsupported combination (nothing was launched) */
   SOFIE_HIP_ERR_RUNTIME = 2,  /* a HIP call failed                                              */
   SOFIE_HIP_ERR_NOMEM = 3     /* arena allocation failed or offset outside the arena            */
};

/* ---- context, stream, arena --------------------------------------------------------------- */

/* Replaces the alpaka Session's devAcc/queue members and its unified pool allocation
 * (core/src/RModel_ALPAKA.cxx:1090-1141, 443-540).  `external_stream` is a hipStream_t (or NULL
 * for a stream owned by the context): the kExternalStream option of the reference
 * (core/inc/SOFIE/RModel_Base.hxx:19-33). */
int sofie_hip_ctx_create(sofie_hip_ctx **out, int device, void *external_stream);
int sofie_hip_ctx_destroy(sofie_hip_ctx *ctx);
/* Kernel-choice overrides of one context, for tuning and for tests that must reach a particular kernel (no counterpart in the
 * reference, whose GPU path has no such choice): "i8_tile" / "f8_tile" (64, 128, 256; 258 and 512 ask for the two-per-CU and the
 * persistent kernel; 0 = heuristic), "gemm_variant" (1: alternative pipelined kernel, -1: general kernel only), "swizzle"
 * (tile order), "conv_explicit" (1: int8 convolutions through a column matrix whenever the workspace holds one), "f32_skinny",
 * "f32_chain" (0 / 1, -1 = heuristic).  Each is also read once, at sofie_hip_ctx_create, from the environment variable
 * SOFIE_HIP_<NAME IN CAPITALS>; nothing reads the environment after that. */
int sofie_hip_ctx_set_option(sofie_hip_ctx *ctx, const char *name, int32_t value);
const char *sofie_hip_last_error(void);
int sofie_hip_abi_version(void);

/* One hipMalloc for the whole Session: weights + planned intermediates (the reference allocates
 * one `allocBuf<uint8_t>` of poolTotalBytes, core/src/RModel_ALPAKA.cxx:477-498).  `align` must
 * be a power of two >= 256 (kPoolAlignBytes, core/src/RModel_ALPAKA.cxx:25). */
int sofie_hip_arena_create(sofie_hip_ctx *ctx, size_t bytes, size_t align);
/* kCustomMemory: adopt caller memory instead of allocating (MemoryProvider.assign,
 * core/src/utils/SOFIE_common_helpers.cxx:741-804). */
int sofie_hip_arena_adopt(sofie_hip_ctx *ctx, void *device_ptr, size_t bytes);
void *sofie_hip_arena_ptr(sofie_hip_ctx *ctx, size_t offset); /* NULL if offset out of range */
size_t sofie_hip_arena_bytes(sofie_hip_ctx *ctx);
void *sofie_hip_stream(sofie_hip_ctx *ctx); /* the hipStream_t every launch below goes to */

/* Host <-> arena copies (the user's alpaka::memcpy around infer, README.md:269-325; weight upload
 * MoveInitializedTensorsToBuffers_ALPAKA, core/src/RModel_ALPAKA.cxx:1695-1707). Asynchronous on
 * the context's stream; sofie_hip_sync waits. */
int sofie_hip_upload(sofie_hip_ctx *ctx, void *dst_device, const void *src_host, size_t bytes);
int sofie_hip_download(sofie_hip_ctx *ctx, void *dst_host, const void *src_device, size_t bytes);
int sofie_hip_copy(sofie_hip_ctx *ctx, void *dst_device, const void *src_device, size_t bytes);
int sofie_hip_fill_zero(sofie_hip_ctx *ctx, void *dst_device, size_t bytes); /* resetState, RModel_ALPAKA.cxx:1546-1568 */
int sofie_hip_sync(sofie_hip_ctx *ctx);                                      /* alpaka::wait(queue) */

/* Data movement of the shape operators.  Transpose (ROperator_Transpose::Generate, core/inc/SOFIE/operators/ROperator_Transpose.hxx):
 * Y[i_perm[0], ..., i_perm[r-1]] = X[i_0, ..., i_{r-1}], i.e. output axis k is input axis perm[k]; `shape` is the INPUT shape, rank <= 6,
 * 4-byte elements.  copy_rows moves `rows` pieces of `row_bytes` bytes from a pitched source to a pitched destination (Concat
 * along an inner axis, ROperator_Concat.hxx: each input contributes one piece per outer index); pitches and row_bytes multiples of 4. */
int sofie_hip_transpose_f32(sofie_hip_ctx *ctx, float *Y, const float *X, int32_t rank, const int64_t *shape, const int32_t *perm);
/* The same kernel with the strides spelled out: Y[i_0, ..., i_{r-1}] = X[in_offset + sum_k i_k * in_strides[k]], Y dense of shape out_shape,
 * rank <= 6, strides in elements (0 repeats an axis, a negative one walks it backwards).  It carries Slice (ROperator_Slice::Generate,
 * core/inc/SOFIE/operators/ROperator_Slice.hxx: offset = sum start * stride, stride = step * stride), Split (ROperator_Split.hxx: one slice
 * per output), Expand (ROperator_Expand.hxx: stride 0 on the broadcast axes) and Tile (ROperator_Tile.hxx: every axis seen as [repeat, length]
 * with strides [0, stride]).  Every element read must lie inside [0, in_elements): checked on the host before the launch. */
int sofie_hip_strided_gather_f32(sofie_hip_ctx *ctx, float *Y, const float *X, int32_t rank, const int64_t *out_shape, const int64_t *in_strides,
                                 int64_t in_offset, int64_t in_elements);
int sofie_hip_copy_rows(sofie_hip_ctx *ctx, void *dst_device, size_t dst_pitch_bytes, const void *src_device, size_t src_pitch_bytes, size_t rows,
                        size_t row_bytes);

/* ---- activation / epilogue vocabulary ------------------------------------------------------ */
/* Scalar formulas follow the reference's CPU emitters:
 *   RELU      x > 0 ? x : 0            core/src/utils/SOFIE_common_helpers.cxx:325-332
 *   LEAKYRELU x >= 0 ? x : alpha*x     core/inc/SOFIE/operators/ROperator_Gemm.hxx:729-738
 *   SIGMOID   1/(1+exp(-x))            core/inc/SOFIE/operators/ROperator_Sigmoid.hxx:43-59
 *   GELU      0.5 x (1+erf(x/sqrt2))   core/inc/SOFIE/operators/ROperator_Gelu.hxx:42-71
 *   GELU_TANH 0.5 x (1+tanh(0.7978845608028654 (x+0.044715 x^3)))   (same file)
 *   TANH      std::tanh                core/inc/SOFIE/operators/ROperator_Tanh.hxx */
enum {
   SOFIE_ACT_NONE = 0,
   SOFIE_ACT_RELU = 1,
   SOFIE_ACT_LEAKYRELU = 2,
   SOFIE_ACT_SIGMOID = 3,
   SOFIE_ACT_GELU = 4,
   SOFIE_ACT_GELU_TANH = 5,
   SOFIE_ACT_TANH = 6,
   /* The reference's other one-to-one float operators (formulas of core/inc/SOFIE/operators/ROperator_BasicUnary.hxx:17-103
    * and ROperator_Clip.hxx:18), usable wherever an activation code is:                                              */
   SOFIE_ACT_RECIPROCAL = 7, /* 1/x                                   */
   SOFIE_ACT_SQRT = 8,
   SOFIE_ACT_NEG = 9,
   SOFIE_ACT_EXP = 10,
   SOFIE_ACT_LOG = 11,
   SOFIE_ACT_SIN = 12,
   SOFIE_ACT_COS = 13,
   SOFIE_ACT_ABS = 14,
   SOFIE_ACT_SOFTPLUS = 15,  /* x >= 20 ? x : log1p(exp(x))           */
   SOFIE_ACT_ATAN = 16,
   SOFIE_ACT_FLOOR = 17,
   SOFIE_ACT_ASINH = 18,
   SOFIE_ACT_ACOSH = 19,
   SOFIE_ACT_ATANH = 20,
   SOFIE_ACT_CLIP = 21,      /* max(alpha, min(beta, x))              */
   SOFIE_ACT_SELU = 22,      /* beta * (max(0,x) + min(0, alpha*(exp(x)-1))), beta = gamma; core/inc/SOFIE/operators/ROperator_Selu.hxx:56-62 */
   SOFIE_ACT_ELU = 23,       /* x >= 0 ? x : alpha * (exp(x) - 1); core/inc/SOFIE/operators/ROperator_Elu.hxx:69-74 */
   SOFIE_ACT_ERF = 24,       /* std::erf(x); core/inc/SOFIE/operators/ROperator_Erf.hxx */
   SOFIE_ACT_HARDSIGMOID = 25, /* max(0, min(1, alpha * x + beta)); core/inc/SOFIE/operators/ROperator_HardSigmoid.hxx:71-74 */
   SOFIE_ACT_HARDSWISH = 26,   /* x * fmax(0, fmin(1, (1/6) * x + 1/2)), 1/6 rounded to float; core/inc/SOFIE/operators/ROperator_HardSwish.hxx:56-60 */
   SOFIE_ACT_SWISH = 27,       /* x / (1 + exp(-x)); core/inc/SOFIE/operators/ROperator_Swish.hxx:54-56 */
   SOFIE_ACT_LAST = 27
};

/* A chain of one-to-one operators applied, in order, to every element an operator stores: what the reference's
 * elementwise fusion builds from GetElementwiseExpr (core/inc/SOFIE/operators/ROperator_ALPAKA.hxx:57-76) when
 * such operators follow a Gemm or a Conv.  op[i] is a SOFIE_ACT_* code, alpha[i] / beta[i] its parameters
 * (LeakyRelu slope; Clip bounds). */
#define SOFIE_MAX_POST_OPS 4
typedef struct sofie_post_ops {
   int32_t count; /* 0..SOFIE_MAX_POST_OPS */
   int32_t op[SOFIE_MAX_POST_OPS];
   float alpha[SOFIE_MAX_POST_OPS];
   float beta[SOFIE_MAX_POST_OPS];
} sofie_post_ops;

/* How a bias (the Gemm operand C) is broadcast onto Y[M,N]; the four cases the reference's Gemm
 * emitter distinguishes (core/inc/SOFIE/operators/ROperator_Gemm.hxx:578-617). */
enum {
   SOFIE_BIAS_NONE = 0,
   SOFIE_BIAS_ROW = 1,    /* C is [N] or [1,N]: Copy(Y + N*j, C, N) for every row j            */
   SOFIE_BIAS_COL = 2,    /* C is [M,1]:        Fill(Y + N*j, C[j], N)                          */
   SOFIE_BIAS_SCALAR = 3, /* C is [1,1]/[1]:    Fill(Y + N*j, C[0], N)                          */
   SOFIE_BIAS_FULL = 4    /* C is [M,N]: passed to Gemm_Call as C, Y = alpha*A*B + beta*C       */
};

/* ---- fp32 Gemm / MatMul -------------------------------------------------------------------- */
/* Replaces ROperator_Gemm<float>::Generate + Gemm_Call + BLAS::sgemm_ + Relu
 * (core/inc/SOFIE/operators/ROperator_Gemm.hxx:419-741, core/src/utils/SOFIE_common_helpers.cxx:296-332)
 * and, on the alpaka path, blas.gemm / blas.gemmrelu / blas.gemmStridedBatched + GemmBiasAddKernel
 * (ROperator_Gemm.hxx:743-764, 931-1103).
 *   Y[b] = post( act( alpha * op(A[b]) * op(B[b]) + beta_eff * broadcast(C) + residual[b] ) ),  b < batch
 * Tensors are row-major as ONNX defines them: op(A) is [M,K], op(B) is [K,N], Y is [M,N].
 * transA: A is stored [K,M]; transB: B is stored [N,K].  beta_eff is 1 for the broadcast cases and
 * `beta` for SOFIE_BIAS_FULL, which is the reference's behaviour (ROperator_Gemm.hxx:580). */
typedef struct sofie_gemm_f32_desc {
   int32_t M, N, K;
   int32_t transA, transB;
   int32_t lda, ldb, ldy; /* row strides in elements of the STORED matrices; 0 = dense default */
   float alpha, beta;
   const float *A;
   const float *B;
   const float *C; /* bias or NULL */
   int32_t bias_mode;
   int32_t act;
   float act_alpha; /* LeakyRelu slope */
   float *Y;
   int32_t batch; /* stacked MatMul count (>=1); strides in elements, 0 = operand shared */
   int64_t strideA, strideB, strideC, strideY;
   const sofie_post_ops *post; /* applied after `act`; NULL = none */
   /* A tensor of Y's shape (same ldy and strideY) added before `act`: an Add of another activation tensor behind the product
    * (a residual connection), which the reference runs as a separate ROperator_BasicBinary.  NULL = none. */
   const float *residual;
} sofie_gemm_f32_desc;
int sofie_hip_gemm_f32(sofie_hip_ctx *ctx, const sofie_gemm_f32_desc *d);
/* `count` products of which each reads what the one before wrote (layers[l].A == layers[l-1].Y): the Gemm + activation
 * sequence the reference emits for an MLP, one blas call and one Relu pass per layer (ROperator_Gemm.hxx:685-741).  The
 * results are those of `count` calls of sofie_hip_gemm_f32 in order, every Y written.  At small M (up to 256 rows, no transA,
 * no stacking, rows of at most 2048 to 8192 floats) the whole chain is ONE launch, the activations passing from layer to
 * layer through LDS; otherwise the call is the loop over the layers. */
#define SOFIE_MAX_GEMM_CHAIN 16
int sofie_hip_gemm_chain_f32(sofie_hip_ctx *ctx, const sofie_gemm_f32_desc *layers, int32_t count);

/* ---- int8 Gemm (MatMulInteger + fused requantisation) -------------------------------------- */
/* No counterpart exists in the reference (ROperator_Gemm is float only,
 * core/inc/SOFIE/operators/ROperator_Gemm.hxx:67; no quantised operator is registered,
 * parsers/src/RModelParser_ONNX.cxx:279-367).  The semantics are the ONNX ones:
 *   acc[m,n]  = sum_k int32(A[m,k]) * int32(B[k,n])              (exact)
 *   acc      += bias_i32[n]                                      (if bias)
 *   acc       = max(acc,0)                                       (if relu_acc)
 * then by `out`:
 *   SOFIE_I8OUT_I32    Y_i32 = acc
 *   SOFIE_I8OUT_F32    Y_f32 = float(acc) * s              (DequantizeLinear; s = scale[n] or scale_scalar),
 *                              then max(.,0) if relu_out
 *   SOFIE_I8OUT_I8     Y_i8  = sat8(rne(float(acc) * s))   (requant), then max(.,0) if relu_out
 *   SOFIE_I8OUT_I8_DQQ Y_i8  = sat8(rne((float(acc) * s) / q_scale))   (DequantizeLinear followed by the
 *                              next layer's QuantizeLinear, same fp32 operations in the same order)
 * One fp32 multiply (no fused multiply-add), round-half-to-even, saturation to [-128,127].
 * A is [M,K] int8 row-major (lda), B is [K,N] row-major (ldb) or, with transB, stored [N,K].
 * The MFMA kernel wants both operands K-contiguous; a B given as [K,N] is transposed into
 * `workspace` (K*N bytes, 256-B aligned) on every call.  A constant B (a weight) is better re-laid
 * out once at Session construction with sofie_hip_transpose_i8 and then passed with transB = 1. */
enum { SOFIE_I8OUT_I32 = 0, SOFIE_I8OUT_F32 = 1, SOFIE_I8OUT_I8 = 2, SOFIE_I8OUT_I8_DQQ = 3,
       SOFIE_I8OUT_I8_PLANE_SUMS = 4 /* sofie_hip_conv_i8 only, see there */ };
typedef struct sofie_gemm_i8_desc {
   int32_t M, N, K;
   int32_t transA, transB;
   int32_t lda, ldb, ldy; /* 0 = dense default */
   const int8_t *A;
   const int8_t *B;
   const int32_t *bias; /* [N] or NULL */
   const float *scale;  /* [N] per output channel, or NULL -> scale_scalar */
   float scale_scalar;
   float q_scale; /* SOFIE_I8OUT_I8_DQQ only */
   int32_t relu_acc, relu_out;
   int32_t out;
   void *Y;
   void *workspace; /* device scratch for operand re-layout, may be NULL if not needed */
   size_t workspace_bytes;
} sofie_gemm_i8_desc;
int sofie_hip_gemm_i8(sofie_hip_ctx *ctx, const sofie_gemm_i8_desc *d);
/* Bytes of workspace sofie_hip_gemm_i8 needs for this descriptor (0 if none). */
size_t sofie_hip_gemm_i8_workspace(const sofie_gemm_i8_desc *d);
/* sofie_hip_gemm_i8 for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  It has no counterpart in the reference.  The scratch for the operand re-layout (B given
 * as [K,N], A given as [K,M]) is a static device array of SOFIE_HIP_GEMM_I8_NOALLOC_SCRATCH_BYTES that every GPU the library
 * runs on holds until the process ends; `workspace` / `workspace_bytes` of the descriptor are ignored.  A descriptor whose
 * re-layout needs more (sofie_hip_gemm_i8_workspace) is refused with an error.  The call allocates and frees nothing.  All
 * calls on one GPU share that GPU's array: calls that overlap in time on one GPU (two streams, two threads) race. */
#define SOFIE_HIP_GEMM_I8_NOALLOC_SCRATCH_BYTES (8u << 20)
int sofie_hip_gemm_i8_noalloc(sofie_hip_ctx *ctx, const sofie_gemm_i8_desc *d);
/* Re-layout of a [K,N] int8 matrix into [N,K] (weights, once, at Session construction; the
 * analogue of the Conv weight re-layout into tensor_<Y>_f, ROperator_Conv.hxx:456-476). */
int sofie_hip_transpose_i8(sofie_hip_ctx *ctx, int8_t *dst, const int8_t *src, int32_t rows, int32_t cols,
                           int32_t ld_src, int32_t ld_dst);

/* ---- FP8 (OCP e4m3fn) Gemm ------------------------------------------------------------------ */
/* No counterpart in the reference (ETensorType ends at BFLOAT16, core/inc/SOFIE/utils/SOFIE_common.hxx:29-54).
 *   acc[m,n] = sum_k f32(A[m,k]) * f32(B[k,n])   (fp32 accumulate, hardware summation order)
 *   v        = acc * (scale_a*scale_b) + bias[n];   v = act(v);   Y = bf16_rne(v) or fp32
 * A [M,K] e4m3fn bytes; B [K,N] or, with transB, [N,K]; same workspace rule as the int8 Gemm.
 *
 * Per-element bound.  The matrix cores do not add the products of a K step in IEEE fp32 order, so the result is not
 * bit-defined; it is held to the exactly accumulated one.  With S = sum_k |a_k b_k| (exact products), v0 the value before
 * the activation and y0 the result when the sum is exact and every later step is one correctly rounded fp32 operation:
 *   |Y - y0| <= L * (2^-14 * S * scale  +  2^-22 * (|v0| + |bias[n]|))    accumulation; roundings of the scaling and the bias
 *             + g * |v0|                                                  SOFIE_ACT_GELU only: g = 1e-6 (fp32 output), 8e-5 (bf16 output)
 *             + 2^-21 * |y0|                                              the activation's own fp32 evaluation
 *             + half an ulp of bf16 at the result (at most 2^-8 * |Y|)    SOFIE_F8OUT_BF16 only
 * L = 1.13 for the two GELU forms (the largest slope of GELU), 1 otherwise.  SOFIE_ACT_GELU is evaluated in the store as
 * v * Phi(v).  For fp32 output Phi comes from the rational approximation 7.1.26 of Abramowitz and Stegun (|error of erfc| <=
 * 1.5e-7), the hardware's reciprocal and 2^x (one ulp each) and seven more fp32 operations: |error of Phi| <= 1e-6.  For bf16
 * output, whose half ulp is 2^-9 .. 2^-8 of the result, Phi - 1/2 is an odd polynomial of degree 15 in v clamped to [-4, 4]:
 * |error of Phi| <= 8e-5, a fiftieth of that half ulp, at half the instructions (the store of a tile is time the matrix cores
 * stand idle).
 * 2^-14 is four times the largest accumulation error measured (about 2^-16 * S per 64-element K step, not growing with K). */
enum { SOFIE_F8OUT_BF16 = 0, SOFIE_F8OUT_F32 = 1 };
typedef struct sofie_gemm_fp8_desc {
   int32_t M, N, K;
   int32_t transB;
   int32_t lda, ldb, ldy;
   const uint8_t *A;
   const uint8_t *B;
   const float *bias; /* [N] fp32 or NULL */
   float scale;       /* scale_a * scale_b, formed in fp32 by the caller */
   int32_t act;
   int32_t out;
   void *Y;
   void *workspace;
   size_t workspace_bytes;
} sofie_gemm_fp8_desc;
int sofie_hip_gemm_fp8(sofie_hip_ctx *ctx, const sofie_gemm_fp8_desc *d);
/* fp32 -> e4m3fn: q = sat(rne_e4m3(x / scale)); saturating at +-448, NaN -> 0x7f. */
int sofie_hip_quantize_fp8(sofie_hip_ctx *ctx, uint8_t *dst, const float *src, size_t n, float scale);

/* ---- QuantizeLinear / DequantizeLinear (per tensor, symmetric, zero point 0) ---------------- */
/* ONNX: q = sat8(rne(x / scale)) with fp32 division; y = float(q) * scale.  Not in the reference. */
int sofie_hip_quantize_linear(sofie_hip_ctx *ctx, int8_t *dst, const float *src, size_t n, float scale);
int sofie_hip_dequantize_linear_i8(sofie_hip_ctx *ctx, float *dst, const int8_t *src, size_t n, float scale);
int sofie_hip_dequantize_linear_i32(sofie_hip_ctx *ctx, float *dst, const int32_t *src, size_t n, float scale);

/* ---- stand-alone elementwise operators ------------------------------------------------------ */
/* Replaces the CPU loops / alpaka kernels of ROperator_Relu, _Sigmoid, _Gelu, _LeakyRelu, _Tanh
 * (core/inc/SOFIE/operators/ROperator_Relu.hxx:47-86 and siblings). dst may equal src. */
int sofie_hip_unary_f32(sofie_hip_ctx *ctx, float *dst, const float *src, size_t n, int32_t act, float act_alpha);
/* several of them in one pass over the data: dst[i] = op[count-1](... op[0](src[i])) */
int sofie_hip_unary_chain_f32(sofie_hip_ctx *ctx, float *dst, const float *src, size_t n, const sofie_post_ops *ops);
/* ROperator_BasicBinary<float,Add> with multidirectional broadcasting
 * (core/inc/SOFIE/operators/ROperator_BasicBinary.hxx:380-510).  Shapes are right-aligned, rank<=6;
 * a_shape/b_shape hold 1 where the operand is broadcast. */
typedef struct sofie_add_desc {
   int32_t rank;
   int64_t y_shape[6];
   int64_t a_shape[6];
   int64_t b_shape[6];
   const float *A;
   const float *B;
   float *Y;
} sofie_add_desc;
int sofie_hip_add_f32(sofie_hip_ctx *ctx, const sofie_add_desc *d);
/* The other members of the family, same broadcasting (BinaryOperatorTrait<T, Op>::Op, ROperator_BasicBinary.hxx:22-53: a - b,
 * a * b, a / b, std::pow(a, b)), and the pairwise steps of the n-ary operators (NaryOperatorTraits, ROperator_BasicNary.hxx:19-100:
 * std::max / std::min keep the FIRST operand unless the second is strictly larger / smaller, Sum adds left to right, Mean
 * divides that sum by float(count)): an n-ary operator is a left fold of these, ADD_DIV with `param` = count being Mean's last step.
 * Pow goes through the device's powf (a few ulp from the host library's); every other result is the IEEE one. */
enum {
   SOFIE_BINARY_ADD = 0, SOFIE_BINARY_SUB = 1, SOFIE_BINARY_MUL = 2, SOFIE_BINARY_DIV = 3, SOFIE_BINARY_POW = 4,
   SOFIE_BINARY_MAX = 5, /* a < b ? b : a */
   SOFIE_BINARY_MIN = 6, /* b < a ? b : a */
   SOFIE_BINARY_ADD_DIV = 7, /* (a + b) / param */
   SOFIE_BINARY_LAST = 7
};
int sofie_hip_binary_f32(sofie_hip_ctx *ctx, const sofie_add_desc *d, int32_t op, float param);

/* ---- Conv as GEMM --------------------------------------------------------------------------- */
/* Replaces ROperator_Conv<float>::Generate: weight re-layout + per-image Im2col + Gemm_Call
 * (core/inc/SOFIE/operators/ROperator_Conv.hxx:406-642; Im2col core/src/utils/SOFIE_common_helpers.cxx:47-83)
 * and the alpaka Im2ColKernel/BiasBroadcastKernel/blas.matmul triple (ROperator_Conv.hxx:732-1103)
 * with ONE implicit-GEMM launch over the whole batch (no materialised column matrix).
 * X is NCHW [N,C,H,W], W is [Cout, C/group, kh, kw], Y is NCHW [N,Cout,OH,OW]; 1-D convs pass H=1,kh=1.
 * pads follow the reference's order {h_begin, w_begin, h_end, w_end} (ROperator_Conv.hxx:517-530). */
typedef struct sofie_conv_desc {
   int32_t N, C, H, W;
   int32_t Cout, kh, kw;
   int32_t pad_h0, pad_w0, pad_h1, pad_w1;
   int32_t stride_h, stride_w;
   int32_t dil_h, dil_w;
   int32_t group;
   int32_t OH, OW; /* as computed by the caller's shape inference; checked */
} sofie_conv_desc;
int sofie_hip_conv_f32(sofie_hip_ctx *ctx, const sofie_conv_desc *d, const float *X, const float *W,
                       const float *bias /* [Cout] or NULL */, int32_t act, float act_alpha, float *Y,
                       const sofie_post_ops *post /* applied after `act`; NULL = none */,
                       const float *residual /* [N,Cout,OH,OW] added before `act`, or NULL */);
/* 3-D convolution (ROperator_Conv with three spatial dimensions, core/inc/SOFIE/operators/ROperator_Conv.hxx:533-552, and
 * UTILITY::Im2col_3d, core/src/utils/SOFIE_common_helpers.cxx:85-139): the same implicit GEMM with the reduction over
 * (channel, kd, kh, kw).  X is [N,C,D,H,W], W is [Cout, C/group, kd, kh, kw], Y is [N,Cout,OD,OH,OW]; the pads are ordered as the
 * ONNX attribute: {d_begin, h_begin, w_begin, d_end, h_end, w_end}. */
typedef struct sofie_conv3d_desc {
   int32_t N, C, D, H, W;
   int32_t Cout, kd, kh, kw;
   int32_t pad[6];
   int32_t stride[3];
   int32_t dil[3];
   int32_t group;
   int32_t OD, OH, OW; /* as computed by the caller's shape inference; checked */
} sofie_conv3d_desc;
int sofie_hip_conv3d_f32(sofie_hip_ctx *ctx, const sofie_conv3d_desc *d, const float *X, const float *W,
                         const float *bias /* [Cout] or NULL */, int32_t act, float act_alpha, float *Y,
                         const sofie_post_ops *post /* applied after `act`; NULL = none */,
                         const float *residual /* of Y's shape, added before `act`, or NULL */);
/* int8 form (no counterpart in the reference): acc = conv_i32(X_i8, W_i8) + bias_i32[co], then by `out`
 *   SOFIE_I8OUT_I8   Y_i8  = sat8(rne(float(acc)*scale[co])), then max(.,0) if relu
 *   SOFIE_I8OUT_F32  Y_f32 = float(acc)*scale[co], then max(.,0) if relu
 *   SOFIE_I8OUT_I32  Y_i32 = relu ? max(acc,0) : acc
 *   SOFIE_I8OUT_I8_PLANE_SUMS  the int8 feature map of SOFIE_I8OUT_I8 is not stored; Y is int32 [N, Cout] and receives
 *                    Y[n,co] += sum over the OH*OW output pixels of that int8 value (integer additions from the kernel's store,
 *                    exact in any order).  The caller clears Y first (sofie_hip_fill_zero).  For a GlobalAveragePool that is
 *                    the only reader of a convolution: the largest activation of the network is neither written nor read
 *                    back.  Needs OH*OW to be a multiple of 256 and a shape that takes no column matrix (workspace 0), else
 *                    the call is refused; y_layout is ignored.
 * Activations are NCHW (the ONNX layout) or NHWC (channels fastest), chosen per tensor: a chain of
 * convolutions keeps NHWC between its layers.  W is the ONNX weight [Cout, C/group, kh, kw], or, with
 * w_is_packed, the re-laid-out form sofie_hip_pack_conv_weight_i8 writes once at Session construction
 * (the role of tensor_<Y>_f in the reference, ROperator_Conv.hxx:456-476).  NHWC input whose channels
 * per group are a power of two >= 64 (and at most 32 filter taps) is read directly by the GEMM kernel
 * (implicit GEMM, no column matrix); any other case gathers a column matrix first.  The workspace holds
 * the packed weights (unless w_is_packed) and, when a column matrix is needed, that of as many images as
 * fit (at least one); sofie_hip_conv_i8_workspace returns the minimum, which may be 0. */
enum { SOFIE_LAYOUT_NCHW = 0, SOFIE_LAYOUT_NHWC = 1 };
typedef struct sofie_conv_i8_args {
   const int8_t *X;
   const int8_t *W;
   const int32_t *bias; /* [Cout] or NULL */
   const float *scale;  /* [Cout]; may be NULL for SOFIE_I8OUT_I32 */
   int32_t relu;
   int32_t out;
   int32_t x_layout, y_layout;
   int32_t w_is_packed;
   void *Y;
   void *workspace;
   size_t workspace_bytes;
} sofie_conv_i8_args;
int sofie_hip_conv_i8(sofie_hip_ctx *ctx, const sofie_conv_desc *d, const sofie_conv_i8_args *a);
size_t sofie_hip_conv_i8_workspace(const sofie_conv_desc *d, const sofie_conv_i8_args *a); /* minimum bytes */
size_t sofie_hip_conv_i8_column_matrix_bytes(const sofie_conv_desc *d); /* column matrix of one image (what "conv_explicit" needs on top) */
size_t sofie_hip_conv_weight_i8_packed_bytes(const sofie_conv_desc *d);
int sofie_hip_pack_conv_weight_i8(sofie_hip_ctx *ctx, const sofie_conv_desc *d, int8_t *dst, const int8_t *src);

/* ---- pooling tail --------------------------------------------------------------------------- */
/* GlobalAveragePool (ROperator_Pool, core/inc/SOFIE/operators/ROperator_Pool.hxx:225-237):
 * Y[n,c] = (sum over the HW plane of X[n,c,:]) / float(HW); the fp32 sum is a tree reduction, so it
 * agrees with the reference's sequential loop to rounding only. */
int sofie_hip_global_avg_pool_f32(sofie_hip_ctx *ctx, float *Y, const float *X, int32_t NC, int32_t HW);
/* MaxPool / AveragePool over 1-D and 2-D windows of an NCHW tensor, the loops of ROperator_Pool<float>::Generate
 * (core/inc/SOFIE/operators/ROperator_Pool.hxx:286-412): the window of output (oh, ow) starts at
 * (oh*stride_h - pad_h0, ow*stride_w - pad_w0) and spans kh x kw positions (for a dilated MaxPool kh, kw are the DILATED
 * extents and every position inside is visited, as the reference does); positions outside the image are skipped.
 * MaxPool: the largest value met (-inf for an empty window; NaN never wins `x > value`).  AveragePool: the fp32 sum in
 * row-major window order, divided by float(nsum): nsum = kh*kw when `dynamic_divisor` is 0, else per dimension
 * min(start + k, hi) - lo with hi = size (+ end padding if count_include_pad), lo = start (clamped at 0 unless
 * count_include_pad) -- the reference's windowExtent (:328-333).  1-D pooling passes H = OH = kh = 1. */
enum { SOFIE_POOL_MAX = 0, SOFIE_POOL_AVERAGE = 1 };
typedef struct sofie_pool_desc {
   int32_t planes; /* N * C */
   int32_t H, W, OH, OW;
   int32_t kh, kw;
   int32_t pad_h0, pad_w0, pad_h1, pad_w1;
   int32_t stride_h, stride_w;
   int32_t mode; /* SOFIE_POOL_* */
   int32_t count_include_pad;
   int32_t dynamic_divisor; /* the reference sets it when any padding is non-zero or ceil_mode is on */
} sofie_pool_desc;
int sofie_hip_pool_f32(sofie_hip_ctx *ctx, const sofie_pool_desc *d, float *Y, const float *X);
/* The same over three spatial axes, slowest first (the third branch of ROperator_Pool::Generate,
 * core/inc/SOFIE/operators/ROperator_Pool.hxx:293-300, 421-475): the window is visited axis 0, then 1, then 2, the divisor of an
 * average is the product of the three window extents (:433-438).  k is the window per axis (the dilated extent). */
typedef struct sofie_pool3d_desc {
   int32_t planes; /* N * C */
   int32_t in[3], out[3];
   int32_t k[3];
   int32_t pad_begin[3], pad_end[3];
   int32_t stride[3];
   int32_t mode; /* SOFIE_POOL_* */
   int32_t count_include_pad;
   int32_t dynamic_divisor;
} sofie_pool3d_desc;
int sofie_hip_pool3d_f32(sofie_hip_ctx *ctx, const sofie_pool3d_desc *d, float *Y, const float *X);
/* int8 input, fp32 output: Y = (float(sum_i32) * scale) / float(HW), exact sum -- not in the reference. */
int sofie_hip_global_avg_pool_i8(sofie_hip_ctx *ctx, float *Y /* [N,C] */, const int8_t *X, int32_t N, int32_t C, int32_t HW,
                                 int32_t x_layout /* SOFIE_LAYOUT_* */, float scale);
/* The same average when a convolution has already added the planes up (sofie_hip_conv_i8 with
 * SOFIE_I8OUT_I8_PLANE_SUMS): Y[i] = (float(sums[i]) * scale) / float(HW) -- the bits sofie_hip_global_avg_pool_i8 gives
 * on the feature map that was never stored. */
int sofie_hip_plane_sums_to_average(sofie_hip_ctx *ctx, float *Y /* [NC] */, const int32_t *sums /* [NC] */, int32_t NC, int32_t HW,
                                    float scale);
/* The same average, and the sums are set back to zero behind the read.  For a caller that keeps one sums buffer per
 * convolution and clears it once (an emitted Session does, at construction): every inference leaves the buffer as the next
 * one needs it, and the clearing launch per inference goes away. */
int sofie_hip_plane_sums_take_average(sofie_hip_ctx *ctx, float *Y /* [NC] */, int32_t *sums /* [NC], zero afterwards */, int32_t NC,
                                      int32_t HW, float scale);

/* Softmax / LogSoftmax along one axis of a tensor seen as [outer, axis_len, inner] (ROperator_Softmax::Generate,
 * core/inc/SOFIE/operators/ROperator_Softmax.hxx:82-198): vmax = max over the axis, e = exp(x - vmax), sum = sum of e;
 * Softmax gives e * (1.0f / sum) when the axis is the last one (inner == 1, :114-117) and e / sum otherwise (:188); LogSoftmax
 * gives x - vmax - log(sum).  The sum is a tree over the axis here, a sequential loop in the reference: results agree to
 * the rounding of that sum, which for the loop grows with the axis length (1e-7 relative at 10 classes, 6e-5 at 70000). */
int sofie_hip_softmax_f32(sofie_hip_ctx *ctx, float *Y, const float *X, int64_t outer, int32_t axis_len, int64_t inner, int32_t log_softmax);

/* The Reduce family over the middle dimension of a tensor seen as [outer, A, inner] (ROperator_Reduce<Op>::Generate,
 * core/inc/SOFIE/operators/ROperator_Reduce.hxx:349-400: start value 0, 1 for Prod, lowest() for Max, max() for Min; y += x, y += x*x,
 * y *= x, y = std::max(y, x), y = std::min(y, x) over the reduced elements in increasing order; Mean then divides by float(A), L2 takes
 * std::sqrt).  Reduced axes that are adjacent fold into one A.  Few long lines (inner == 1, A >= 64, fewer than 16384 outputs) are
 * reduced by a wave each, as a tree: sums and products then agree with the loop to rounding only; every other case runs the loop's order. */
enum { SOFIE_REDUCE_SUM = 0, SOFIE_REDUCE_MEAN = 1, SOFIE_REDUCE_SUM_SQUARE = 2, SOFIE_REDUCE_PROD = 3, SOFIE_REDUCE_L2 = 4, SOFIE_REDUCE_MAX = 5,
       SOFIE_REDUCE_MIN = 6 };
int sofie_hip_reduce_f32(sofie_hip_ctx *ctx, float *Y, const float *X, int64_t outer, int32_t A, int64_t inner, int32_t op);

/* LayerNormalization over the trailing dimensions of a tensor seen as [rows, L] (ROperator_LayerNormalization::Generate,
 * core/inc/SOFIE/operators/ROperator_LayerNormalization.hxx:247-312): mean = sum(x) / L, invStdDev = 1 / sqrt(sum((x - mean)^2) / L + epsilon),
 * Y = scale[j] * invStdDev * (x - mean) + bias[j].  scale and bias hold L elements (bias may be NULL); mean_out / inv_std_out, when not
 * NULL, receive the per-row statistics (the operator's optional outputs).  The two sums are trees here, loops in the reference. */
int sofie_hip_layernorm_f32(sofie_hip_ctx *ctx, float *Y, const float *X, const float *scale, const float *bias, int64_t rows, int32_t L,
                            float epsilon, float *mean_out, float *inv_std_out);

/* BatchNormalization at inference, for models whose normalisation was not folded into the weights
 * (core/inc/SOFIE/operators/ROperator_BatchNormalization.hxx:139-158): X is [N, C, spatial...],
 *   Y = (X - mean[c]) * fused_scale[c] + bias[c],   fused_scale[c] = scale[c] / sqrt(var[c] + eps) formed by the generator,
 * then x > 0 ? x : 0 when `relu` is set (the reference's BN + Relu fusion).  Three separately rounded fp32 operations. */
int sofie_hip_batchnorm_f32(sofie_hip_ctx *ctx, float *Y, const float *X, const float *fused_scale, const float *mean,
                            const float *bias, int32_t N, int32_t C, int32_t spatial, int32_t relu);

/* ---- measurement helpers used by the benchmark ------------------------------------------------ */
/* hipEvent pair on the context's stream (torch's events only see torch's streams). */
int sofie_hip_timer_start(sofie_hip_ctx *ctx);
int sofie_hip_timer_stop(sofie_hip_ctx *ctx, float *elapsed_ms); /* records, synchronises, returns ms */

#ifdef __cplusplus
}
#endif
#endif /* SOFIE_HIP_H */
