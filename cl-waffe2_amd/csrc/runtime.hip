// runtime.hip -- device selection, zero-initialised allocation, transfers,
// stream/event plumbing and the error channel of libwaffe2-hip.so.
//
// cl-waffe2's CPU path needs none of this (Lisp owns host vectors and pins
// them per call, source/backends/cpu/tensor.lisp:43-57); a device backend
// does: the AbstractTensor allocation hook (source/vm/generic-tensor/
// tensor.lisp:146-210), tensor-finalizer (:323-329), vref (:719-746) and
// convert-tensor-facet (source/array-converter.lisp:15-197) map onto
// malloc/free/memcpy below.
#include <map>
#include <mutex>
#include <stdlib.h>
#include <string.h>
#include <iterator>
#include <unordered_map>
#include <vector>

#include "wf2_common.h"
#include "wf2_pool.h"

namespace wf2 {

static Runtime g_rt;
static std::mutex g_mu;
static thread_local char g_err[512] = "";

Runtime& rt() { return g_rt; }

int reduce_setup_device(int device);  // reduce.hip: address of its static scratch on this device

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

// ---- caching allocator -------------------------------------------------------
// The bookkeeping (idle blocks, blocks that captured graphs still write into) is
// BlockPool, wf2_pool.h.  Blocks are recycled without synchronising: every kernel and
// copy of the library runs on one stream, so a recycled block's new user is ordered
// after its old one.  hipFree (which does synchronise) only happens on trim/shutdown
// or when the device is out of memory.
struct Graph : GraphBlocks {
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
};
static Graph* g_capture = nullptr;  // non-null between graph_begin and graph_end
static std::vector<Graph*> g_destroy_after_capture;  // graphs released while another was being recorded (guarded by g_pool_mu)

static std::mutex g_pool_mu;
static BlockPool g_pool;  // guarded by g_pool_mu
static size_t g_pool_requests = 0;  // guarded by g_pool_mu

static void pool_release_idle_locked() {
  std::vector<void*> release;
  g_pool.drain_idle(&release);
  for (void* ptr : release) (void)hipFree(ptr);
}

static int pool_alloc(void** ptr, size_t bytes) {
  const size_t cls = BlockPool::size_class(bytes);
  std::lock_guard<std::mutex> lock(g_pool_mu);
  g_pool_requests++;
  *ptr = g_pool.take(cls, g_capture);
  if (*ptr) return 0;
  if (g_capture)
    return fail(WF2HIP_ECAPTURE,
                "a %zu-byte block is not in the pool and hipMalloc cannot run during graph "
                "capture: run the sequence once before capturing it", bytes);
  hipError_t e = hipMalloc(ptr, cls);
  if (e == hipErrorOutOfMemory && g_pool.has_idle()) {
    (void)hipGetLastError();
    (void)hipStreamSynchronize(g_rt.stream);
    pool_release_idle_locked();
    e = hipMalloc(ptr, cls);
  }
  if (e == hipErrorOutOfMemory) {
    (void)hipGetLastError();
    *ptr = nullptr;
    return fail(WF2HIP_ENOMEM, "out of device memory allocating %zu bytes", bytes);
  }
  WF2_TRY(check_hip(e, "hipMalloc"));
  g_pool.adopt(*ptr, cls);
  return 0;
}

static int pool_free(void* ptr) {
  BlockPool::Outcome what;
  {
    std::lock_guard<std::mutex> lock(g_pool_mu);
    what = g_pool.give_back(ptr, g_capture);
  }
  if (what == BlockPool::kUnknown)
    return fail(WF2HIP_EINVAL, "wf2hip_free: %p was not allocated by wf2hip_malloc", ptr);
  if (what == BlockPool::kKept) return 0;
  WF2_TRY(check_hip(hipStreamSynchronize(g_rt.stream), "hipStreamSynchronize"));
  return check_hip(hipFree(ptr), "hipFree");
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
  WF2_TRY(reduce_setup_device(device));
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
  // The library's own stream (default priority).  A real stream rather than
  // the null stream so that it can be captured into a graph.
  if (!g_rt.own_stream)
    WF2_TRY(check_hip(hipStreamCreateWithFlags(&g_rt.own_stream, hipStreamNonBlocking),
                      "hipStreamCreateWithFlags"));
  g_rt.stream = g_rt.own_stream;
  g_rt.initialised = true;
  const char* pool_env = getenv("WF2HIP_POOL");
  g_pool.enabled = !(pool_env && pool_env[0] == '0');
  return 0;
}

WF2_API int wf2hip_shutdown(void) {
  std::lock_guard<std::mutex> lock(g_mu);
  if (!g_rt.initialised) return 0;
  (void)hipStreamSynchronize(g_rt.stream);
  {
    std::lock_guard<std::mutex> pool_lock(g_pool_mu);
    pool_release_idle_locked();
  }
  if (g_rt.partials) (void)hipFree(g_rt.partials);
  if (g_rt.own_stream) (void)hipStreamDestroy(g_rt.own_stream);
  g_rt = Runtime();
  return 0;
}

WF2_API int wf2hip_pool_trim(void) {
  WF2_TRY(require_init());
  WF2_TRY(check_hip(hipStreamSynchronize(g_rt.stream), "hipStreamSynchronize"));
  std::lock_guard<std::mutex> lock(g_pool_mu);
  pool_release_idle_locked();
  return 0;
}

WF2_API size_t wf2hip_pool_idle_bytes(void) {
  std::lock_guard<std::mutex> lock(g_pool_mu);
  return g_pool.idle_bytes();
}

WF2_API size_t wf2hip_pool_requests(void) {
  std::lock_guard<std::mutex> lock(g_pool_mu);
  return g_pool_requests;
}

WF2_API int wf2hip_device_info(char* buf, size_t buflen) {
  WF2_TRY(require_init());
  if (!buf || buflen == 0) return fail(WF2HIP_EINVAL, "null buffer");
  snprintf(buf, buflen, "%s|%s|%d|%zu", g_rt.name, g_rt.arch, g_rt.num_cus, g_rt.total_mem);
  return 0;
}

WF2_API int wf2hip_malloc_uninitialized(void** ptr, size_t bytes) {
  WF2_TRY(require_init());
  if (!ptr) return fail(WF2HIP_EINVAL, "null result pointer");
  *ptr = nullptr;
  if (bytes == 0) return 0;
  return pool_alloc(ptr, bytes);
}

WF2_API int wf2hip_malloc(void** ptr, size_t bytes) {
  WF2_TRY(wf2hip_malloc_uninitialized(ptr, bytes));
  if (bytes == 0) return 0;
  // Zero fill on the library's stream so it is ordered with the kernels that
  // will use the buffer (a fill kernel rather than a memset node, so callers
  // may capture it).  Blocks are multiples of 512 bytes: whole words.
  const size_t words = (bytes + 3) / 4;
  int64_t want = ceil_div((int64_t)words, kBlock * 8);
  int blocks = (int)(want < 16384 ? want : 16384);
  fill_kernel<<<blocks, kBlock, 0, g_rt.stream>>>((float*)*ptr, words, 0.0f);
  return after_launch("zero fill");
}

WF2_API int wf2hip_free(void* ptr) {
  WF2_TRY(require_init());
  if (!ptr) return 0;
  return pool_free(ptr);
}

WF2_API int wf2hip_memcpy_h2d(void* dst, const void* src, size_t bytes) {
  WF2_TRY(require_init());
  if (g_capture) return fail(WF2HIP_ECAPTURE, "host transfers block and cannot be captured");
  if (bytes == 0) return 0;
  if (!dst || !src) return fail(WF2HIP_EINVAL, "null pointer");
  WF2_TRY(check_hip(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, g_rt.stream),
                    "hipMemcpyAsync(h2d)"));
  // The host buffer may be unpinned or moved by the caller's GC right after.
  return check_hip(hipStreamSynchronize(g_rt.stream), "hipStreamSynchronize");
}

WF2_API int wf2hip_memcpy_d2h(void* dst, const void* src, size_t bytes) {
  WF2_TRY(require_init());
  if (g_capture) return fail(WF2HIP_ECAPTURE, "host transfers block and cannot be captured");
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
  if (g_capture) return fail(WF2HIP_ECAPTURE, "cannot synchronise during graph capture");
  return check_hip(hipStreamSynchronize(g_rt.stream), "hipStreamSynchronize");
}

WF2_API int wf2hip_set_stream(void* hip_stream) {
  WF2_TRY(require_init());
  // recycled blocks rely on single-stream ordering: drain the old stream first
  if (g_capture) return fail(WF2HIP_ECAPTURE, "cannot change the stream during graph capture");
  WF2_TRY(check_hip(hipStreamSynchronize(g_rt.stream), "hipStreamSynchronize"));
  g_rt.stream = hip_stream ? (hipStream_t)hip_stream : g_rt.own_stream;
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

// ---- graph capture ------------------------------------------------------------
// cl-waffe2 compiles a model into an instruction sequence once and replays it on
// every forward (source/vm/generic-tensor/acceptor.lisp:409-508, vm.lisp:260).
// The device-side analogue: record the kernel sequence of one forward on the
// library's stream into a HIP graph and replay it with a single launch, which
// removes the per-node host cost.  Zero fills are fill kernels, never memset
// nodes, so everything the library enqueues is a kernel or a copy node.

WF2_API int wf2hip_graph_begin(void) {
  WF2_TRY(require_init());
  std::lock_guard<std::mutex> lock(g_pool_mu);
  if (g_capture) return fail(WF2HIP_ECAPTURE, "a capture is already in progress");
  if (g_rt.stream == nullptr)
    return fail(WF2HIP_ECAPTURE, "the null stream cannot be captured; use the library's own stream");
  Graph* g = new Graph();
  int rc = check_hip(hipStreamBeginCapture(g_rt.stream, hipStreamCaptureModeThreadLocal),
                     "hipStreamBeginCapture");
  if (rc != 0) {
    delete g;
    return rc;
  }
  g_capture = g;
  return 0;
}

WF2_API int wf2hip_graph_end(void** graph) {
  WF2_TRY(require_init());
  if (!graph) return fail(WF2HIP_EINVAL, "null result pointer");
  *graph = nullptr;
  Graph* g;
  {
    std::lock_guard<std::mutex> lock(g_pool_mu);
    g = g_capture;
    g_capture = nullptr;
  }
  if (!g) return fail(WF2HIP_ECAPTURE, "no capture in progress");
  int rc = check_hip(hipStreamEndCapture(g_rt.stream, &g->graph), "hipStreamEndCapture");
  {
    std::vector<Graph*> waiting;
    {
      std::lock_guard<std::mutex> lock(g_pool_mu);
      waiting.swap(g_destroy_after_capture);
    }
    for (Graph* old : waiting) (void)wf2hip_graph_destroy(old);
  }
  if (rc == 0) rc = check_hip(hipGraphInstantiate(&g->exec, g->graph, nullptr, nullptr, 0),
                              "hipGraphInstantiate");
  if (rc != 0) {
    wf2hip_graph_destroy(g);
    return rc;
  }
  *graph = g;
  return 0;
}

WF2_API int wf2hip_graph_launch(void* graph) {
  WF2_TRY(require_init());
  Graph* g = (Graph*)graph;
  if (!g || !g->exec) return fail(WF2HIP_EINVAL, "not an instantiated graph");
  if (g_capture) return fail(WF2HIP_ECAPTURE, "cannot launch a graph while capturing");
  return check_hip(hipGraphLaunch(g->exec, g_rt.stream), "hipGraphLaunch");
}

WF2_API int wf2hip_graph_destroy(void* graph) {
  Graph* g = (Graph*)graph;
  if (!g) return 0;
  {
    // Destroying a graph synchronises the stream, which a capture in progress does not survive (a handle
    // rebound inside a recording, `with Graph() as g:` over an older g): it waits for wf2hip_graph_end.
    std::lock_guard<std::mutex> lock(g_pool_mu);
    if (g_capture && g != g_capture) {
      g_destroy_after_capture.push_back(g);
      return 0;
    }
  }
  // replays still in flight read and write the held blocks
  if (g_rt.initialised) (void)hipStreamSynchronize(g_rt.stream);
  if (g->exec) (void)hipGraphExecDestroy(g->exec);
  if (g->graph) (void)hipGraphDestroy(g->graph);
  {
    std::lock_guard<std::mutex> lock(g_pool_mu);
    std::vector<void*> release;
    g_pool.forget_graph(g, &release);
    for (void* ptr : release) (void)hipFree(ptr);
  }
  delete g;
  return 0;
}
