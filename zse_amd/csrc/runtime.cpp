// Host-side HIP runtime calls behind a flat C interface for ctypes.
//
// The reference binds libamdhip64 symbol by symbol from Python
// (zse-compiler/zse_compiler/runtime/memory.py:71-447) and drives graphs through
// hipStreamBeginCapture / hipGraphInstantiate / hipGraphLaunch
// (zse-engine/zse_engine/orchestrator/hip_graph.py:76-130).  The same calls
// live here so that every failure carries HIP's own error text.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstring>
#include <string>

static thread_local std::string g_err;

static int fail(hipError_t e, const char* what) {
  g_err = std::string(what) + ": " + hipGetErrorString(e);
  return (int)e == 0 ? -1 : (int)e;
}

#define CHECK(call)                          \
  do {                                       \
    hipError_t e_ = (call);                  \
    if (e_ != hipSuccess) return fail(e_, #call); \
  } while (0)

extern "C" {

const char* zrt_last_error() { return g_err.c_str(); }

int zrt_device_count(int* n) {
  CHECK(hipGetDeviceCount(n));
  return 0;
}

int zrt_init(int device) {
  CHECK(hipSetDevice(device));
  CHECK(hipFree(nullptr));
  return 0;
}

int zrt_device_info(int device, char* name, int name_len, size_t* total_mem, size_t* free_mem,
                    int* compute_units, char* arch, int arch_len) {
  hipDeviceProp_t p;
  CHECK(hipGetDeviceProperties(&p, device));
  std::snprintf(name, name_len, "%s", p.name);
  std::snprintf(arch, arch_len, "%s", p.gcnArchName);
  *compute_units = p.multiProcessorCount;
  CHECK(hipMemGetInfo(free_mem, total_mem));
  return 0;
}

int zrt_malloc(void** p, size_t n) {
  CHECK(hipMalloc(p, n));
  return 0;
}

int zrt_free(void* p) {
  CHECK(hipFree(p));
  return 0;
}

int zrt_host_alloc(void** p, size_t n) {
  CHECK(hipHostMalloc(p, n, hipHostMallocDefault));
  return 0;
}

int zrt_host_free(void* p) {
  CHECK(hipHostFree(p));
  return 0;
}

int zrt_h2d(void* dst, const void* src, size_t n, void* stream, int async) {
  if (async) {
    CHECK(hipMemcpyAsync(dst, src, n, hipMemcpyHostToDevice, (hipStream_t)stream));
  } else {
    CHECK(hipMemcpyAsync(dst, src, n, hipMemcpyHostToDevice, (hipStream_t)stream));
    CHECK(hipStreamSynchronize((hipStream_t)stream));
  }
  return 0;
}

int zrt_d2h(void* dst, const void* src, size_t n, void* stream, int async) {
  CHECK(hipMemcpyAsync(dst, src, n, hipMemcpyDeviceToHost, (hipStream_t)stream));
  if (!async) CHECK(hipStreamSynchronize((hipStream_t)stream));
  return 0;
}

int zrt_d2d(void* dst, const void* src, size_t n, void* stream) {
  CHECK(hipMemcpyAsync(dst, src, n, hipMemcpyDeviceToDevice, (hipStream_t)stream));
  return 0;
}

int zrt_stream_create(void** s) {
  hipStream_t st;
  CHECK(hipStreamCreate(&st));
  *s = (void*)st;
  return 0;
}

int zrt_stream_destroy(void* s) {
  CHECK(hipStreamDestroy((hipStream_t)s));
  return 0;
}

int zrt_stream_sync(void* s) {
  CHECK(hipStreamSynchronize((hipStream_t)s));
  return 0;
}

int zrt_device_sync() {
  CHECK(hipDeviceSynchronize());
  return 0;
}

int zrt_event_create(void** e) {
  hipEvent_t ev;
  CHECK(hipEventCreate(&ev));
  *e = (void*)ev;
  return 0;
}

int zrt_event_record(void* e, void* s) {
  CHECK(hipEventRecord((hipEvent_t)e, (hipStream_t)s));
  return 0;
}

int zrt_event_sync(void* e) {
  CHECK(hipEventSynchronize((hipEvent_t)e));
  return 0;
}

int zrt_event_elapsed_ms(void* a, void* b, float* ms) {
  CHECK(hipEventElapsedTime(ms, (hipEvent_t)a, (hipEvent_t)b));
  return 0;
}

int zrt_event_destroy(void* e) {
  CHECK(hipEventDestroy((hipEvent_t)e));
  return 0;
}

// ---- graphs: capture what a stream is given, replay it later ----

int zrt_capture_begin(void* s) {
  CHECK(hipStreamBeginCapture((hipStream_t)s, hipStreamCaptureModeThreadLocal));
  return 0;
}

int zrt_capture_end(void* s, void** exec) {
  hipGraph_t g = nullptr;
  CHECK(hipStreamEndCapture((hipStream_t)s, &g));
  hipGraphExec_t ex = nullptr;
  hipError_t e = hipGraphInstantiate(&ex, g, nullptr, nullptr, 0);
  hipGraphDestroy(g);
  if (e != hipSuccess) return fail(e, "hipGraphInstantiate");
  *exec = (void*)ex;
  return 0;
}

int zrt_graph_launch(void* exec, void* s) {
  CHECK(hipGraphLaunch((hipGraphExec_t)exec, (hipStream_t)s));
  return 0;
}

int zrt_graph_destroy(void* exec) {
  CHECK(hipGraphExecDestroy((hipGraphExec_t)exec));
  return 0;
}

}  // extern "C"
