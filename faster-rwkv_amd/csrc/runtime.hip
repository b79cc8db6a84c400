// Runtime entry points of the C ABI: device selection, memory, streams, events and
// graph capture.  These stand where the reference calls cudart directly
// (tensor.cpp:58-96, kernels/cuda/allocator.cpp:412-460).
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>

#include "frhip_internal.h"

namespace frhip {

static thread_local std::string g_err = "no error";
static int g_cus = 0;
static int g_wgs_per_cu = 1;

int set_error(int code, const char* msg) {
  g_err = msg ? msg : "error";
  return code;
}

int hip_result(hipError_t e, const char* what) {
  if (e == hipSuccess) return 0;
  g_err = std::string(what) + ": " + hipGetErrorString(e);
  return (int)e;
}

int check_launch(const char* kernel) { return hip_result(hipGetLastError(), kernel); }

int compute_units() {
  if (g_cus == 0) {
    int dev = 0;
    hipDeviceProp_t p;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&p, dev) == hipSuccess)
      g_cus = p.multiProcessorCount;
    else
      g_cus = 256;
    const char* e = getenv("FRHIP_WGS_PER_CU");
    if (e && atoi(e) > 0 && atoi(e) <= 8) g_wgs_per_cu = atoi(e);
  }
  return g_cus;
}

int decode_grid() { return compute_units() * g_wgs_per_cu; }

}  // namespace frhip

using namespace frhip;

#define HIP_TRY(call) \
  do {                \
    int _r = hip_result((call), #call); \
    if (_r) return _r; \
  } while (0)

extern "C" {

int frhip_abi_version(void) { return FRHIP_ABI_VERSION; }

const char* frhip_error_string(void) { return g_err.c_str(); }

int frhip_device_count(int* count) {
  if (!count) return set_error(FRHIP_EINVAL, "count is null");
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess) {
    *count = 0;
    return hip_result(e, "hipGetDeviceCount");
  }
  *count = n;
  return 0;
}

int frhip_init(int device) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) return set_error(FRHIP_ENODEV, "no HIP device visible");
  if (device < 0 || device >= n) return set_error(FRHIP_EINVAL, "device index out of range");
  HIP_TRY(hipSetDevice(device));
  hipDeviceProp_t p;
  HIP_TRY(hipGetDeviceProperties(&p, device));
  if (strncmp(p.gcnArchName, "gfx950", 6) != 0) {
    g_err = std::string("device is ") + p.gcnArchName + ", this library holds gfx950 code only";
    return FRHIP_ENODEV;
  }
  g_cus = 0;
  compute_units();
  if (int e = allow_large_lds()) return e;
  return static_scratch(nullptr);  // this device's copy of the built-in scratch
}

int frhip_device_info(char* name, size_t name_len, int* cus, size_t* total_mem) {
  int dev = 0;
  HIP_TRY(hipGetDevice(&dev));
  hipDeviceProp_t p;
  HIP_TRY(hipGetDeviceProperties(&p, dev));
  if (name && name_len) {
    snprintf(name, name_len, "%s (%s)", p.name, p.gcnArchName);
  }
  if (cus) *cus = p.multiProcessorCount;
  if (total_mem) *total_mem = p.totalGlobalMem;
  return 0;
}

int frhip_malloc(void** ptr, size_t bytes) {
  if (!ptr) return set_error(FRHIP_EINVAL, "ptr is null");
  *ptr = nullptr;
  if (bytes == 0) return 0;
  const hipError_t e = hipMalloc(ptr, bytes);
  if (e != hipSuccess) {
    (void)hipGetLastError();  // a refused allocation must not surface again as the next launch's error
    *ptr = nullptr;
    return hip_result(e, "hipMalloc");
  }
  return 0;
}

int frhip_free(void* ptr) {
  if (!ptr) return 0;
  HIP_TRY(hipFree(ptr));
  return 0;
}

int frhip_host_malloc(void** ptr, size_t bytes) {
  if (!ptr) return set_error(FRHIP_EINVAL, "ptr is null");
  *ptr = nullptr;
  if (bytes == 0) return 0;
  HIP_TRY(hipHostMalloc(ptr, bytes, hipHostMallocDefault));
  return 0;
}

int frhip_host_free(void* ptr) {
  if (!ptr) return 0;
  HIP_TRY(hipHostFree(ptr));
  return 0;
}

static int to_kind(int kind, hipMemcpyKind* k) {
  switch (kind) {
    case FRHIP_H2D: *k = hipMemcpyHostToDevice; return 0;
    case FRHIP_D2H: *k = hipMemcpyDeviceToHost; return 0;
    case FRHIP_D2D: *k = hipMemcpyDeviceToDevice; return 0;
    default: return set_error(FRHIP_EINVAL, "unknown memcpy kind");
  }
}

int frhip_memcpy(void* dst, const void* src, size_t bytes, int kind) {
  if (bytes == 0) return 0;
  if (!dst || !src) return set_error(FRHIP_EINVAL, "memcpy: null pointer");
  hipMemcpyKind k;
  int r = to_kind(kind, &k);
  if (r) return r;
  HIP_TRY(hipMemcpy(dst, src, bytes, k));
  return 0;
}

int frhip_memcpy_async(void* dst, const void* src, size_t bytes, int kind, frhip_stream s) {
  if (bytes == 0) return 0;
  if (!dst || !src) return set_error(FRHIP_EINVAL, "memcpy: null pointer");
  hipMemcpyKind k;
  int r = to_kind(kind, &k);
  if (r) return r;
  HIP_TRY(hipMemcpyAsync(dst, src, bytes, k, static_cast<hipStream_t>(s)));
  return 0;
}

int frhip_memset_async(void* dst, int byte, size_t bytes, frhip_stream s) {
  if (bytes == 0) return 0;
  if (!dst) return set_error(FRHIP_EINVAL, "memset: null pointer");
  HIP_TRY(hipMemsetAsync(dst, byte, bytes, static_cast<hipStream_t>(s)));
  return 0;
}

int frhip_stream_create(frhip_stream* s) {
  if (!s) return set_error(FRHIP_EINVAL, "stream out-pointer is null");
  hipStream_t st;
  HIP_TRY(hipStreamCreate(&st));  // default priority; ordered against the null stream's blocking copies
  *s = st;
  return 0;
}

int frhip_stream_destroy(frhip_stream s) {
  if (!s) return 0;
  HIP_TRY(hipStreamDestroy(static_cast<hipStream_t>(s)));
  return 0;
}

int frhip_stream_sync(frhip_stream s) {
  HIP_TRY(hipStreamSynchronize(static_cast<hipStream_t>(s)));
  return 0;
}

int frhip_device_sync(void) {
  HIP_TRY(hipDeviceSynchronize());
  return 0;
}

int frhip_event_create(frhip_event* e) {
  if (!e) return set_error(FRHIP_EINVAL, "event out-pointer is null");
  hipEvent_t ev;
  HIP_TRY(hipEventCreate(&ev));
  *e = ev;
  return 0;
}

int frhip_event_destroy(frhip_event e) {
  if (!e) return 0;
  HIP_TRY(hipEventDestroy(static_cast<hipEvent_t>(e)));
  return 0;
}

int frhip_event_record(frhip_event e, frhip_stream s) {
  if (!e) return set_error(FRHIP_EINVAL, "event is null");
  HIP_TRY(hipEventRecord(static_cast<hipEvent_t>(e), static_cast<hipStream_t>(s)));
  return 0;
}

int frhip_event_sync(frhip_event e) {
  if (!e) return set_error(FRHIP_EINVAL, "event is null");
  HIP_TRY(hipEventSynchronize(static_cast<hipEvent_t>(e)));
  return 0;
}

int frhip_event_elapsed_ms(frhip_event start, frhip_event stop, float* ms) {
  if (!start || !stop || !ms) return set_error(FRHIP_EINVAL, "event_elapsed: null argument");
  HIP_TRY(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
  return 0;
}

int frhip_graph_begin(frhip_stream s) {
  if (!s) return set_error(FRHIP_EINVAL, "graph capture needs an explicit stream");
  HIP_TRY(hipStreamBeginCapture(static_cast<hipStream_t>(s), hipStreamCaptureModeThreadLocal));
  return 0;
}

int frhip_graph_end(frhip_stream s, frhip_graph* g) {
  if (!s || !g) return set_error(FRHIP_EINVAL, "graph_end: null argument");
  hipGraph_t graph = nullptr;
  HIP_TRY(hipStreamEndCapture(static_cast<hipStream_t>(s), &graph));
  hipGraphExec_t exec = nullptr;
  hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  (void)hipGraphDestroy(graph);
  if (e != hipSuccess) return hip_result(e, "hipGraphInstantiate");
  *g = exec;
  return 0;
}

int frhip_graph_launch(frhip_graph g, frhip_stream s) {
  if (!g) return set_error(FRHIP_EINVAL, "graph is null");
  HIP_TRY(hipGraphLaunch(static_cast<hipGraphExec_t>(g), static_cast<hipStream_t>(s)));
  return 0;
}

int frhip_graph_destroy(frhip_graph g) {
  if (!g) return 0;
  HIP_TRY(hipGraphExecDestroy(static_cast<hipGraphExec_t>(g)));
  return 0;
}

}  // extern "C"
