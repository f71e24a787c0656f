// runtime.hip -- device selection, zero-initialised allocation, transfers,
// stream/event plumbing and the error channel of libwaffe2-hip.so.
//
// cl-waffe2's CPU path needs none of this (Lisp owns host vectors and pins
// them per call, source/backends/cpu/tensor.lisp:43-57); a device backend
// does: the AbstractTensor allocation hook (source/vm/generic-tensor/
// tensor.lisp:146-210), tensor-finalizer (:323-329), vref (:719-746) and
// convert-tensor-facet (source/array-converter.lisp:15-197) map onto
// malloc/free/memcpy below.
#include <mutex>
#include <string.h>

#include "wf2_common.h"

namespace wf2 {

static Runtime g_rt;
static std::mutex g_mu;
static thread_local char g_err[512] = "";

Runtime& rt() { return g_rt; }

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof g_err, fmt, ap);
  va_end(ap);
  return code;
}

int check_hip(hipError_t e, const char* what) {
  if (e == hipSuccess) return 0;
  return fail((int)e, "%s: %s", what, hipGetErrorString(e));
}

int require_init() {
  if (!g_rt.initialised) return fail(WF2HIP_ENOTINIT, "wf2hip_init has not been called");
  return 0;
}

__global__ void fill_kernel(float* __restrict__ x, size_t n, float v) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) x[i] = v;
}

}  // namespace wf2

using namespace wf2;

WF2_API int wf2hip_abi_version(void) { return WF2HIP_ABI_VERSION; }

WF2_API const char* wf2hip_last_error(void) { return g_err; }

WF2_API int wf2hip_init(int device) {
  std::lock_guard<std::mutex> lock(g_mu);
  if (g_rt.initialised && g_rt.device == device) return 0;
  int count = 0;
  WF2_TRY(check_hip(hipGetDeviceCount(&count), "hipGetDeviceCount"));
  if (device < 0 || device >= count)
    return fail(WF2HIP_EINVAL, "device %d out of range (%d visible)", device, count);
  WF2_TRY(check_hip(hipSetDevice(device), "hipSetDevice"));
  hipDeviceProp_t prop;
  WF2_TRY(check_hip(hipGetDeviceProperties(&prop, device), "hipGetDeviceProperties"));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return fail(WF2HIP_EUNSUPPORTED, "kernels are built for gfx950 only, device is %s",
                prop.gcnArchName);
  if (g_rt.partials) {
    (void)hipFree(g_rt.partials);
    g_rt.partials = nullptr;
  }
  WF2_TRY(check_hip(hipMalloc((void**)&g_rt.partials, kPartialCapacity * sizeof(float)),
                    "hipMalloc(partials)"));
  g_rt.device = device;
  g_rt.num_cus = prop.multiProcessorCount;
  g_rt.total_mem = prop.totalGlobalMem;
  snprintf(g_rt.name, sizeof g_rt.name, "%s", prop.name);
  snprintf(g_rt.arch, sizeof g_rt.arch, "%s", prop.gcnArchName);
  g_rt.stream = nullptr;
  g_rt.initialised = true;
  return 0;
}

WF2_API int wf2hip_shutdown(void) {
  std::lock_guard<std::mutex> lock(g_mu);
  if (!g_rt.initialised) return 0;
  (void)hipStreamSynchronize(g_rt.stream);
  if (g_rt.partials) (void)hipFree(g_rt.partials);
  g_rt = Runtime();
  return 0;
}

WF2_API int wf2hip_device_info(char* buf, size_t buflen) {
  WF2_TRY(require_init());
  if (!buf || buflen == 0) return fail(WF2HIP_EINVAL, "null buffer");
  snprintf(buf, buflen, "%s|%s|%d|%zu", g_rt.name, g_rt.arch, g_rt.num_cus, g_rt.total_mem);
  return 0;
}

WF2_API int wf2hip_malloc(void** ptr, size_t bytes) {
  WF2_TRY(require_init());
  if (!ptr) return fail(WF2HIP_EINVAL, "null result pointer");
  *ptr = nullptr;
  if (bytes == 0) return 0;
  hipError_t e = hipMalloc(ptr, bytes);
  if (e == hipErrorOutOfMemory) {
    (void)hipGetLastError();
    return fail(WF2HIP_ENOMEM, "out of device memory allocating %zu bytes", bytes);
  }
  WF2_TRY(check_hip(e, "hipMalloc"));
  // Zero fill on the library's stream so it is ordered with the kernels that
  // will use the buffer.
  size_t words = bytes / 4;
  if (words) {
    int blocks = (int)(ceil_div((int64_t)words, kBlock * 8) < 16384
                           ? ceil_div((int64_t)words, kBlock * 8)
                           : 16384);
    fill_kernel<<<blocks, kBlock, 0, g_rt.stream>>>((float*)*ptr, words, 0.0f);
    WF2_TRY(after_launch("zero fill"));
  }
  if (bytes % 4)
    WF2_TRY(check_hip(hipMemsetAsync((char*)*ptr + words * 4, 0, bytes % 4, g_rt.stream),
                      "hipMemsetAsync"));
  return 0;
}

WF2_API int wf2hip_free(void* ptr) {
  WF2_TRY(require_init());
  if (!ptr) return 0;
  // Kernels still reading the buffer must finish first.
  WF2_TRY(check_hip(hipStreamSynchronize(g_rt.stream), "hipStreamSynchronize"));
  return check_hip(hipFree(ptr), "hipFree");
}

WF2_API int wf2hip_memcpy_h2d(void* dst, const void* src, size_t bytes) {
  WF2_TRY(require_init());
  if (bytes == 0) return 0;
  if (!dst || !src) return fail(WF2HIP_EINVAL, "null pointer");
  WF2_TRY(check_hip(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, g_rt.stream),
                    "hipMemcpyAsync(h2d)"));
  // The host buffer may be unpinned or moved by the caller's GC right after.
  return check_hip(hipStreamSynchronize(g_rt.stream), "hipStreamSynchronize");
}

WF2_API int wf2hip_memcpy_d2h(void* dst, const void* src, size_t bytes) {
  WF2_TRY(require_init());
  if (bytes == 0) return 0;
  if (!dst || !src) return fail(WF2HIP_EINVAL, "null pointer");
  WF2_TRY(check_hip(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, g_rt.stream),
                    "hipMemcpyAsync(d2h)"));
  return check_hip(hipStreamSynchronize(g_rt.stream), "hipStreamSynchronize");
}

WF2_API int wf2hip_memcpy_d2d(void* dst, const void* src, size_t bytes) {
  WF2_TRY(require_init());
  if (bytes == 0) return 0;
  if (!dst || !src) return fail(WF2HIP_EINVAL, "null pointer");
  return check_hip(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, g_rt.stream),
                   "hipMemcpyAsync(d2d)");
}

WF2_API int wf2hip_fill_f32(float* x, size_t n, float value) {
  WF2_TRY(require_init());
  if (n == 0) return 0;
  if (!x) return fail(WF2HIP_EINVAL, "null pointer");
  int64_t want = ceil_div((int64_t)n, kBlock * 8);
  int blocks = (int)(want < 16384 ? want : 16384);
  fill_kernel<<<blocks, kBlock, 0, g_rt.stream>>>(x, n, value);
  return after_launch("fill_f32");
}

WF2_API int wf2hip_sync(void) {
  WF2_TRY(require_init());
  return check_hip(hipStreamSynchronize(g_rt.stream), "hipStreamSynchronize");
}

WF2_API int wf2hip_set_stream(void* hip_stream) {
  WF2_TRY(require_init());
  g_rt.stream = (hipStream_t)hip_stream;
  return 0;
}

WF2_API void* wf2hip_get_stream(void) { return (void*)g_rt.stream; }

WF2_API int wf2hip_event_create(void** event) {
  WF2_TRY(require_init());
  if (!event) return fail(WF2HIP_EINVAL, "null result pointer");
  hipEvent_t ev;
  WF2_TRY(check_hip(hipEventCreate(&ev), "hipEventCreate"));
  *event = (void*)ev;
  return 0;
}

WF2_API int wf2hip_event_record(void* event) {
  WF2_TRY(require_init());
  return check_hip(hipEventRecord((hipEvent_t)event, g_rt.stream), "hipEventRecord");
}

WF2_API int wf2hip_event_elapsed_ms(void* start, void* stop, float* ms) {
  WF2_TRY(require_init());
  if (!ms) return fail(WF2HIP_EINVAL, "null result pointer");
  WF2_TRY(check_hip(hipEventSynchronize((hipEvent_t)stop), "hipEventSynchronize"));
  return check_hip(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop),
                   "hipEventElapsedTime");
}

WF2_API int wf2hip_event_destroy(void* event) {
  WF2_TRY(require_init());
  return check_hip(hipEventDestroy((hipEvent_t)event), "hipEventDestroy");
}

WF2_API int wf2hip_set_reduce_mode(int mode) {
  if (mode != 0 && mode != 1) return fail(WF2HIP_EINVAL, "reduce mode must be 0 or 1");
  g_rt.reduce_mode = mode;
  return 0;
}

WF2_API int wf2hip_get_reduce_mode(void) { return g_rt.reduce_mode; }
