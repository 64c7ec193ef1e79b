// Context, memory and error plumbing of the tpuhip C ABI.
#include "common.hpp"

#include <cstdlib>
#include <cstring>

namespace tpuhip {

static thread_local std::string g_last_error;

int set_error(int status, const char *fmt, ...) {
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_last_error = buf;
  return status;
}

}  // namespace tpuhip

using namespace tpuhip;

extern "C" {

const char *tpuhip_last_error(void) { return g_last_error.c_str(); }
const char *tpuhip_version(void) { return "tpuhip 0.1 (gfx950)"; }

static int ctx_create(int device, void *stream, bool own, tpuhip_ctx **out) {
  TPUHIP_REQUIRE(out != nullptr, "tpuhip_ctx_create: out is NULL");
  int count = 0;
  TPUHIP_CHECK_HIP(hipGetDeviceCount(&count));
  TPUHIP_REQUIRE(device >= 0 && device < count, "tpuhip_ctx_create: device %d of %d", device,
                 count);
  TPUHIP_CHECK_HIP(hipSetDevice(device));
  hipDeviceProp_t prop;
  TPUHIP_CHECK_HIP(hipGetDeviceProperties(&prop, device));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return set_error(TPUHIP_ERR_UNSUPPORTED, "tpuhip is built for gfx950 only, device %d is %s",
                     device, prop.gcnArchName);
  if (int rc = tpuhip_static_scratch_init(device)) return rc;
  tpuhip_ctx *c = new tpuhip_ctx();
  c->device = device;
  c->num_cu = prop.multiProcessorCount;
  if (const char *e = getenv("TPUHIP_AUTOTUNE")) c->autotune = atoi(e) != 0;
  if (own) {
    hipError_t e = hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking);
    if (e != hipSuccess) {
      delete c;
      return set_error(TPUHIP_ERR_HIP, "hipStreamCreate failed: %s", hipGetErrorString(e));
    }
    c->owns_stream = true;
  } else {
    c->stream = (hipStream_t)stream;
  }
  *out = c;
  return TPUHIP_OK;
}

int tpuhip_ctx_create(int device, tpuhip_ctx **out) { return ctx_create(device, nullptr, true, out); }

int tpuhip_ctx_create_on_stream(int device, void *hip_stream, tpuhip_ctx **out) {
  return ctx_create(device, hip_stream, false, out);
}

int tpuhip_ctx_destroy(tpuhip_ctx *ctx) {
  if (!ctx) return TPUHIP_OK;
  (void)hipSetDevice(ctx->device);
  if (ctx->owns_stream && ctx->stream) {
    (void)hipStreamSynchronize(ctx->stream);
    (void)hipStreamDestroy(ctx->stream);
  } else if (ctx->stream) {
    (void)hipStreamSynchronize(ctx->stream);
  }
  if (ctx->workspace) (void)hipFree(ctx->workspace);
  tpuhip_static_scratch_forget(ctx);
  delete ctx;
  return TPUHIP_OK;
}

int tpuhip_ctx_set_autotune(tpuhip_ctx *ctx, int enable) {
  TPUHIP_REQUIRE(ctx, "tpuhip_ctx_set_autotune: NULL context");
  ctx->autotune = enable != 0;
  return TPUHIP_OK;
}

void *tpuhip_ctx_stream(tpuhip_ctx *ctx) { return ctx ? (void *)ctx->stream : nullptr; }

int tpuhip_malloc(tpuhip_ctx *ctx, size_t bytes, void **dptr) {
  TPUHIP_REQUIRE(ctx && dptr, "tpuhip_malloc: NULL argument");
  TPUHIP_CHECK_HIP(hipSetDevice(ctx->device));
  // 256 spare bytes: vector loads of the last pixel may touch up to 15 bytes
  // past the logical end of a tensor.
  hipError_t e = hipMalloc(dptr, bytes + 256);
  if (e == hipErrorOutOfMemory)
    return set_error(TPUHIP_ERR_NOMEM, "tpuhip_malloc: out of device memory (%zu bytes)", bytes);
  TPUHIP_CHECK_HIP(e);
  return TPUHIP_OK;
}

int tpuhip_free(tpuhip_ctx *ctx, void *dptr) {
  TPUHIP_REQUIRE(ctx, "tpuhip_free: NULL context");
  if (!dptr) return TPUHIP_OK;
  TPUHIP_CHECK_HIP(hipSetDevice(ctx->device));
  TPUHIP_CHECK_HIP(hipStreamSynchronize(ctx->stream));
  TPUHIP_CHECK_HIP(hipFree(dptr));
  return TPUHIP_OK;
}

int tpuhip_host_malloc(tpuhip_ctx *ctx, size_t bytes, void **hptr) {
  TPUHIP_REQUIRE(ctx && hptr, "tpuhip_host_malloc: NULL argument");
  TPUHIP_CHECK_HIP(hipSetDevice(ctx->device));
  TPUHIP_CHECK_HIP(hipHostMalloc(hptr, bytes ? bytes : 1, hipHostMallocDefault));
  return TPUHIP_OK;
}

int tpuhip_host_free(tpuhip_ctx *ctx, void *hptr) {
  TPUHIP_REQUIRE(ctx, "tpuhip_host_free: NULL context");
  if (!hptr) return TPUHIP_OK;
  TPUHIP_CHECK_HIP(hipStreamSynchronize(ctx->stream));
  TPUHIP_CHECK_HIP(hipHostFree(hptr));
  return TPUHIP_OK;
}

__global__ void fill_bytes_kernel(uint8_t *p, uint8_t v, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) p[i] = v;
}

int tpuhip_memset(tpuhip_ctx *ctx, void *dptr, int value, size_t bytes) {
  TPUHIP_REQUIRE(ctx && (dptr || bytes == 0), "tpuhip_memset: NULL argument");
  if (bytes == 0) return TPUHIP_OK;
  // a fill kernel, not hipMemsetAsync: stays correct inside a captured graph
  const int threads = 256;
  size_t blocks = (bytes + threads - 1) / threads;
  if (blocks > 4096) blocks = 4096;
  launch(ctx, fill_bytes_kernel, dim3((unsigned)blocks), dim3(threads), (uint8_t *)dptr, (uint8_t)value, bytes);
  TPUHIP_CHECK_HIP(hipGetLastError());
  return TPUHIP_OK;
}

int tpuhip_mem_info(tpuhip_ctx *ctx, size_t *free_bytes, size_t *total_bytes) {
  TPUHIP_REQUIRE(ctx && free_bytes && total_bytes, "tpuhip_mem_info: NULL argument");
  TPUHIP_CHECK_HIP(hipSetDevice(ctx->device));
  TPUHIP_CHECK_HIP(hipMemGetInfo(free_bytes, total_bytes));
  return TPUHIP_OK;
}

int tpuhip_upload(tpuhip_ctx *ctx, void *dst_dev, const void *src_host, size_t bytes) {
  TPUHIP_REQUIRE(ctx && (bytes == 0 || (dst_dev && src_host)), "tpuhip_upload: NULL argument");
  if (bytes == 0) return TPUHIP_OK;
  TPUHIP_CHECK_HIP(hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, ctx->stream));
  TPUHIP_CHECK_HIP(hipStreamSynchronize(ctx->stream));
  return TPUHIP_OK;
}

int tpuhip_download(tpuhip_ctx *ctx, void *dst_host, const void *src_dev, size_t bytes) {
  TPUHIP_REQUIRE(ctx && (bytes == 0 || (dst_host && src_dev)), "tpuhip_download: NULL argument");
  if (bytes == 0) return TPUHIP_OK;
  TPUHIP_CHECK_HIP(hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, ctx->stream));
  TPUHIP_CHECK_HIP(hipStreamSynchronize(ctx->stream));
  return TPUHIP_OK;
}

int tpuhip_sync(tpuhip_ctx *ctx) {
  TPUHIP_REQUIRE(ctx, "tpuhip_sync: NULL context");
  TPUHIP_CHECK_HIP(hipStreamSynchronize(ctx->stream));
  return TPUHIP_OK;
}

int tpuhip_event_create(tpuhip_ctx *ctx, void **event) {
  TPUHIP_REQUIRE(ctx && event, "tpuhip_event_create: NULL argument");
  hipEvent_t e;
  TPUHIP_CHECK_HIP(hipEventCreate(&e));
  *event = (void *)e;
  return TPUHIP_OK;
}

int tpuhip_event_destroy(tpuhip_ctx *ctx, void *event) {
  TPUHIP_REQUIRE(ctx, "tpuhip_event_destroy: NULL context");
  if (event) TPUHIP_CHECK_HIP(hipEventDestroy((hipEvent_t)event));
  return TPUHIP_OK;
}

int tpuhip_event_record(tpuhip_ctx *ctx, void *event) {
  TPUHIP_REQUIRE(ctx && event, "tpuhip_event_record: NULL argument");
  TPUHIP_CHECK_HIP(hipEventRecord((hipEvent_t)event, ctx->stream));
  return TPUHIP_OK;
}

int tpuhip_event_elapsed_ms(tpuhip_ctx *ctx, void *start, void *stop, float *ms) {
  TPUHIP_REQUIRE(ctx && start && stop && ms, "tpuhip_event_elapsed_ms: NULL argument");
  TPUHIP_CHECK_HIP(hipEventSynchronize((hipEvent_t)stop));
  TPUHIP_CHECK_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
  return TPUHIP_OK;
}

int tpuhip_ctx_set_kernel_events(tpuhip_ctx *ctx, void *start, void *stop) {
  TPUHIP_REQUIRE(ctx, "tpuhip_ctx_set_kernel_events: NULL context");
  TPUHIP_REQUIRE((start == nullptr) == (stop == nullptr), "set_kernel_events: pass both events or none");
  ctx->prof_start = (hipEvent_t)start;
  ctx->prof_stop = (hipEvent_t)stop;
  return TPUHIP_OK;
}

int tpuhip_channel_stride(int c) {
  if (c <= 0) return 0;
  return round_up(c, 16);
}

}  // extern "C"
