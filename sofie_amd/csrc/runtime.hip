// Context, stream, arena and copy entry points of include/sofie_hip.h.
#include "common.hpp"
#include <cstdlib>
#include <new>

namespace sofie_hip {

static thread_local char g_last_error[512] = "";

int fail(int code, const char *fmt, ...)
{
   va_list ap;
   va_start(ap, fmt);
   vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
   va_end(ap);
   return code;
}

__global__ void fill_zero_kernel(uint32_t *dst, size_t nwords)
{
   size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
   size_t stride = (size_t)gridDim.x * blockDim.x;
   for (; i < nwords; i += stride)
      dst[i] = 0u;
}

__global__ void fill_zero_bytes_kernel(uint8_t *dst, size_t n)
{
   size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
   if (i < n)
      dst[i] = 0;
}

} // namespace sofie_hip

using namespace sofie_hip;

extern "C" {

const char *sofie_hip_last_error(void) { return g_last_error; }
int sofie_hip_abi_version(void) { return SOFIE_HIP_ABI_VERSION; }

namespace {
struct OptionName {
   const char *name, *env;
   int sofie_hip_options::*field;
};
const OptionName kOptionNames[] = {
   {"swizzle", "SOFIE_HIP_SWIZZLE", &sofie_hip_options::swizzle},
   {"i8_tile", "SOFIE_HIP_I8_TILE", &sofie_hip_options::i8_tile},
   {"f8_tile", "SOFIE_HIP_F8_TILE", &sofie_hip_options::f8_tile},
   {"gemm_variant", "SOFIE_HIP_GEMM_VARIANT", &sofie_hip_options::gemm_variant},
   {"conv_explicit", "SOFIE_HIP_CONV_EXPLICIT", &sofie_hip_options::conv_explicit},
   {"f32_skinny", "SOFIE_HIP_F32_SKINNY", &sofie_hip_options::f32_skinny},
   {"f32_chain", "SOFIE_HIP_F32_CHAIN", &sofie_hip_options::f32_chain},
};
} // namespace

int sofie_hip_ctx_create(sofie_hip_ctx **out, int device, void *external_stream)
{
   SOFIE_HIP_REQUIRE(out != nullptr, "sofie_hip_ctx_create: out is NULL");
   *out = nullptr;
   int ndev = 0;
   SOFIE_HIP_CHECK(hipGetDeviceCount(&ndev));
   SOFIE_HIP_REQUIRE(device >= 0 && device < ndev, "sofie_hip_ctx_create: device %d not in [0,%d)", device, ndev);
   SOFIE_HIP_CHECK(hipSetDevice(device));
   sofie_hip_ctx *ctx = new (std::nothrow) sofie_hip_ctx();
   if (!ctx)
      return fail(SOFIE_HIP_ERR_NOMEM, "sofie_hip_ctx_create: out of host memory");
   ctx->device = device;
   if (external_stream) {
      ctx->stream = (hipStream_t)external_stream;
      ctx->owns_stream = false;
   } else {
      hipError_t e = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking);
      if (e != hipSuccess) {
         delete ctx;
         return fail(SOFIE_HIP_ERR_RUNTIME, "hipStreamCreateWithFlags failed: %s", hipGetErrorString(e));
      }
      ctx->owns_stream = true;
   }
   hipError_t e0 = hipEventCreate(&ctx->ev0);
   hipError_t e1 = hipEventCreate(&ctx->ev1);
   if (e0 != hipSuccess || e1 != hipSuccess) {
      if (ctx->owns_stream)
         (void)hipStreamDestroy(ctx->stream);
      delete ctx;
      return fail(SOFIE_HIP_ERR_RUNTIME, "hipEventCreate failed");
   }
   for (const OptionName &o : kOptionNames)
      if (const char *v = getenv(o.env))
         ctx->opt.*(o.field) = (int)strtol(v, nullptr, 0);
   *out = ctx;
   return SOFIE_HIP_OK;
}

int sofie_hip_ctx_set_option(sofie_hip_ctx *ctx, const char *name, int32_t value)
{
   SOFIE_HIP_REQUIRE(ctx && name, "sofie_hip_ctx_set_option: NULL argument");
   for (const OptionName &o : kOptionNames)
      if (strcmp(name, o.name) == 0) {
         ctx->opt.*(o.field) = value;
         return SOFIE_HIP_OK;
      }
   return fail(SOFIE_HIP_ERR_INVALID, "sofie_hip_ctx_set_option: unknown option '%s'", name);
}

int sofie_hip_ctx_destroy(sofie_hip_ctx *ctx)
{
   if (!ctx)
      return SOFIE_HIP_OK;
   (void)hipSetDevice(ctx->device);
   (void)hipStreamSynchronize(ctx->stream);
   if (ctx->owns_arena && ctx->arena)
      (void)hipFree(ctx->arena);
   if (ctx->ev0)
      (void)hipEventDestroy(ctx->ev0);
   if (ctx->ev1)
      (void)hipEventDestroy(ctx->ev1);
   if (ctx->owns_stream)
      (void)hipStreamDestroy(ctx->stream);
   delete ctx;
   return SOFIE_HIP_OK;
}

int sofie_hip_arena_create(sofie_hip_ctx *ctx, size_t bytes, size_t align)
{
   SOFIE_HIP_REQUIRE(ctx != nullptr, "sofie_hip_arena_create: ctx is NULL");
   SOFIE_HIP_REQUIRE(ctx->arena == nullptr, "sofie_hip_arena_create: the context already has an arena");
   SOFIE_HIP_REQUIRE(align >= 256 && (align & (align - 1)) == 0,
                     "sofie_hip_arena_create: align %zu must be a power of two >= 256", align);
   SOFIE_HIP_CHECK(hipSetDevice(ctx->device));
   if (bytes == 0)
      bytes = align;
   void *p = nullptr;
   hipError_t e = hipMalloc(&p, bytes);
   if (e != hipSuccess)
      return fail(SOFIE_HIP_ERR_NOMEM, "hipMalloc(%zu) failed: %s", bytes, hipGetErrorString(e));
   if (((uintptr_t)p & (align - 1)) != 0) {
      (void)hipFree(p);
      return fail(SOFIE_HIP_ERR_NOMEM, "hipMalloc returned memory not aligned to %zu", align);
   }
   ctx->arena = (char *)p;
   ctx->arena_bytes = bytes;
   ctx->owns_arena = true;
   return SOFIE_HIP_OK;
}

int sofie_hip_arena_adopt(sofie_hip_ctx *ctx, void *device_ptr, size_t bytes)
{
   SOFIE_HIP_REQUIRE(ctx != nullptr, "sofie_hip_arena_adopt: ctx is NULL");
   SOFIE_HIP_REQUIRE(ctx->arena == nullptr, "sofie_hip_arena_adopt: the context already has an arena");
   SOFIE_HIP_REQUIRE(device_ptr != nullptr, "sofie_hip_arena_adopt: memory block is NULL");
   SOFIE_HIP_REQUIRE(((uintptr_t)device_ptr & 255) == 0, "sofie_hip_arena_adopt: memory block is not 256-byte aligned");
   ctx->arena = (char *)device_ptr;
   ctx->arena_bytes = bytes;
   ctx->owns_arena = false;
   return SOFIE_HIP_OK;
}

void *sofie_hip_arena_ptr(sofie_hip_ctx *ctx, size_t offset)
{
   if (!ctx || !ctx->arena || offset >= ctx->arena_bytes) {
      fail(SOFIE_HIP_ERR_NOMEM, "sofie_hip_arena_ptr: offset %zu outside the arena (%zu bytes)", offset,
           ctx ? ctx->arena_bytes : (size_t)0);
      return nullptr;
   }
   return ctx->arena + offset;
}

size_t sofie_hip_arena_bytes(sofie_hip_ctx *ctx) { return ctx ? ctx->arena_bytes : 0; }
void *sofie_hip_stream(sofie_hip_ctx *ctx) { return ctx ? (void *)ctx->stream : nullptr; }

int sofie_hip_upload(sofie_hip_ctx *ctx, void *dst_device, const void *src_host, size_t bytes)
{
   SOFIE_HIP_REQUIRE(ctx != nullptr, "sofie_hip_upload: ctx is NULL");
   if (bytes == 0)
      return SOFIE_HIP_OK;
   SOFIE_HIP_REQUIRE(dst_device && src_host, "sofie_hip_upload: NULL pointer");
   SOFIE_HIP_CHECK(hipMemcpyAsync(dst_device, src_host, bytes, hipMemcpyHostToDevice, ctx->stream));
   return SOFIE_HIP_OK;
}

int sofie_hip_download(sofie_hip_ctx *ctx, void *dst_host, const void *src_device, size_t bytes)
{
   SOFIE_HIP_REQUIRE(ctx != nullptr, "sofie_hip_download: ctx is NULL");
   if (bytes == 0)
      return SOFIE_HIP_OK;
   SOFIE_HIP_REQUIRE(dst_host && src_device, "sofie_hip_download: NULL pointer");
   SOFIE_HIP_CHECK(hipMemcpyAsync(dst_host, src_device, bytes, hipMemcpyDeviceToHost, ctx->stream));
   return SOFIE_HIP_OK;
}

int sofie_hip_copy(sofie_hip_ctx *ctx, void *dst_device, const void *src_device, size_t bytes)
{
   SOFIE_HIP_REQUIRE(ctx != nullptr, "sofie_hip_copy: ctx is NULL");
   if (bytes == 0)
      return SOFIE_HIP_OK;
   SOFIE_HIP_REQUIRE(dst_device && src_device, "sofie_hip_copy: NULL pointer");
   SOFIE_HIP_CHECK(hipMemcpyAsync(dst_device, src_device, bytes, hipMemcpyDeviceToDevice, ctx->stream));
   return SOFIE_HIP_OK;
}

int sofie_hip_fill_zero(sofie_hip_ctx *ctx, void *dst_device, size_t bytes)
{
   SOFIE_HIP_REQUIRE(ctx != nullptr, "sofie_hip_fill_zero: ctx is NULL");
   if (bytes == 0)
      return SOFIE_HIP_OK;
   SOFIE_HIP_REQUIRE(dst_device != nullptr, "sofie_hip_fill_zero: NULL pointer");
   // a fill kernel rather than hipMemsetAsync, so that a caller may capture it into a HIP graph
   if (((uintptr_t)dst_device & 3) == 0 && (bytes & 3) == 0) {
      size_t nwords = bytes / 4;
      size_t blocks = (nwords + 255) / 256;
      if (blocks > 65536)
         blocks = 65536;
      hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, (uint32_t *)dst_device, nwords);
   } else {
      size_t blocks = (bytes + 255) / 256;
      SOFIE_HIP_REQUIRE(blocks < (1ull << 31), "sofie_hip_fill_zero: unaligned region too large");
      hipLaunchKernelGGL(fill_zero_bytes_kernel, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, (uint8_t *)dst_device, bytes);
   }
   return launch_status("fill_zero");
}

int sofie_hip_sync(sofie_hip_ctx *ctx)
{
   SOFIE_HIP_REQUIRE(ctx != nullptr, "sofie_hip_sync: ctx is NULL");
   SOFIE_HIP_CHECK(hipStreamSynchronize(ctx->stream));
   return SOFIE_HIP_OK;
}

int sofie_hip_timer_start(sofie_hip_ctx *ctx)
{
   SOFIE_HIP_REQUIRE(ctx != nullptr, "sofie_hip_timer_start: ctx is NULL");
   SOFIE_HIP_CHECK(hipEventRecord(ctx->ev0, ctx->stream));
   return SOFIE_HIP_OK;
}

int sofie_hip_timer_stop(sofie_hip_ctx *ctx, float *elapsed_ms)
{
   SOFIE_HIP_REQUIRE(ctx != nullptr && elapsed_ms != nullptr, "sofie_hip_timer_stop: NULL argument");
   SOFIE_HIP_CHECK(hipEventRecord(ctx->ev1, ctx->stream));
   SOFIE_HIP_CHECK(hipEventSynchronize(ctx->ev1));
   SOFIE_HIP_CHECK(hipEventElapsedTime(elapsed_ms, ctx->ev0, ctx->ev1));
   return SOFIE_HIP_OK;
}

} // extern "C"
