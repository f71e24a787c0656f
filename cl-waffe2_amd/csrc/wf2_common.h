// wf2_common.h -- shared state, error channel and launch helpers of
// libwaffe2-hip.so (internal; the public ABI is include/waffe2_hip.h).
#pragma once

#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/waffe2_hip.h"

#define WF2_API extern "C" __attribute__((visibility("default")))

namespace wf2 {

constexpr int kWave = 64;            // CDNA wavefront width
constexpr int kBlock = 256;          // 4 wavefronts, one per SIMD of a CU
constexpr int kPartialCapacity = 1 << 16;  // floats of reduction scratch

struct Runtime {
  bool initialised = false;
  int device = -1;
  int num_cus = 0;
  hipStream_t stream = nullptr;      // where every kernel and copy is enqueued
  hipStream_t own_stream = nullptr;  // created by wf2hip_init, the default
  int reduce_mode = 0;
  float* partials = nullptr;  // kPartialCapacity floats, owned by the library
  char name[128] = {0};
  char arch[64] = {0};
  size_t total_mem = 0;
};

Runtime& rt();

// Records a message in the thread-local error slot and returns `code`.
int fail(int code, const char* fmt, ...);
int check_hip(hipError_t e, const char* what);
int require_init();

// Every launch goes through this: catches launch-configuration errors at the
// call that caused them.
inline int after_launch(const char* what) { return check_hip(hipGetLastError(), what); }

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Scratch for a faster route of a kernel that also has a route without scratch.  true: *ptr is the block
// (release it with wf2hip_free once the launches that use it are enqueued).  false with *rc == 0: the device is
// out of memory and the caller takes its other route.  false with *rc != 0: a graph capture is in progress and
// the pool holds no such block -- the caller gives up with that code, because a route chosen by what the pool
// happens to hold would let an eager run and a replay of the same node round differently.
inline bool scratch_block(void** ptr, size_t bytes, int* rc) {
  *rc = wf2hip_malloc_uninitialized(ptr, bytes);
  if (*rc == 0) return true;
  if (*rc != WF2HIP_ECAPTURE) *rc = 0;
  *ptr = nullptr;
  return false;
}

}  // namespace wf2

#define WF2_TRY(expr)            \
  do {                           \
    int _rc = (expr);            \
    if (_rc != 0) return _rc;    \
  } while (0)
