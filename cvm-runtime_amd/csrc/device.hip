// Device memory, streams and events behind plain C entry points, so the host
// runtime (plain C++) never sees a HIP type.
#include "hip_common.h"

using namespace cvmhip;

#define HIP_TRY(expr, what)                                         \
  do {                                                              \
    hipError_t e_ = (expr);                                         \
    if (e_ != hipSuccess) {                                         \
      set_error("%s: %s", what, hipGetErrorString(e_));             \
      return CVMHIP_ERR_RUNTIME;                                    \
    }                                                               \
  } while (0)

#include <string.h>
#include <map>
#include <string>
#include <vector>

namespace cvmhip {

namespace {
struct TimedLaunch { std::string name, desc; double work, bytes; hipEvent_t e0, e1; };
bool g_timing = false;
std::vector<TimedLaunch> g_launches;
}  // namespace

bool kernel_timing_enabled() { return g_timing; }

void kernel_timing_mark(const char* name, double work, double bytes, const char* desc, hipStream_t s, bool start) {
  if (start) {
    TimedLaunch t;
    t.name = name;
    t.desc = desc ? desc : "";
    t.work = work;
    t.bytes = bytes;
    if (hipEventCreate(&t.e0) != hipSuccess || hipEventCreate(&t.e1) != hipSuccess) return;
    hipEventRecord(t.e0, s);
    g_launches.push_back(t);
  } else if (!g_launches.empty()) {
    hipEventRecord(g_launches.back().e1, s);
  }
}

__global__ void __launch_bounds__(256) k_fill32(int32_t* p, int32_t v, size_t n) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) p[i] = v;
}
}  // namespace cvmhip

extern "C" {

int cvmhip_device_count(int* count) {
  if (!count) return arg_error("device_count");
  HIP_TRY(hipGetDeviceCount(count), "hipGetDeviceCount");
  return CVMHIP_OK;
}

int cvmhip_set_device(int device_id) {
  HIP_TRY(hipSetDevice(device_id), "hipSetDevice");
  return CVMHIP_OK;
}

int cvmhip_alloc(void** ptr, size_t bytes) {
  if (!ptr) return arg_error("alloc");
  HIP_TRY(hipMalloc(ptr, bytes ? bytes : 256), "hipMalloc");
  return CVMHIP_OK;
}

int cvmhip_free(void* ptr) {
  if (ptr) HIP_TRY(hipFree(ptr), "hipFree");
  return CVMHIP_OK;
}

// A fill kernel rather than hipMemsetAsync so the call stays valid inside a captured graph.
int cvmhip_memset32(void* ptr, int32_t value, size_t count, void* stream) {
  if (count == 0) return CVMHIP_OK;
  if (!ptr) return arg_error("memset32");
  k_fill32<<<grid_for((int64_t)count, 256), 256, 0, as_stream(stream)>>>((int32_t*)ptr, value, count);
  return check_launch("memset32");
}

int cvmhip_host_alloc(void** ptr, size_t bytes) {
  if (!ptr) return arg_error("host_alloc");
  HIP_TRY(hipHostMalloc(ptr, bytes ? bytes : 256, hipHostMallocDefault), "hipHostMalloc");
  return CVMHIP_OK;
}

int cvmhip_host_free(void* ptr) {
  if (ptr) HIP_TRY(hipHostFree(ptr), "hipHostFree");
  return CVMHIP_OK;
}

// int8 -> int32 with the input clamp of the graph runtime (graph_runtime.cc:345-352)
__global__ void __launch_bounds__(256) k_widen_clamp(const int8_t* __restrict__ src, int32_t* __restrict__ dst, int64_t count,
                                                     int32_t range) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += stride) {
    const int32_t v = src[i];
    dst[i] = v > range ? range : (v < -range ? -range : v);
  }
}

int cvmhip_widen_clamp_i8(const void* src, int32_t* dst, int64_t count, int32_t range, void* stream) {
  if (!src || !dst || count < 0 || range < 0) return arg_error("widen_clamp_i8");
  if (count == 0) return CVMHIP_OK;
  k_widen_clamp<<<grid_for(count, 256), 256, 0, as_stream(stream)>>>(reinterpret_cast<const int8_t*>(src), dst, count, range);
  return check_launch("widen_clamp_i8");
}

// plain 16-bytes-per-lane copy
__global__ void __launch_bounds__(256) k_copy16(const int4* __restrict__ src, int4* __restrict__ dst, int64_t count) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += stride) dst[i] = src[i];
}

int cvmhip_copy_kernel(void* dst, const void* src, size_t bytes, void* stream) {
  if (!dst || !src || (bytes & 15) || ((uintptr_t)dst & 15) || ((uintptr_t)src & 15)) return arg_error("copy_kernel: 16-byte granules");
  if (bytes == 0 || dst == src) return CVMHIP_OK;
  const int64_t count = (int64_t)(bytes / 16);
  int64_t blocks = (count + 255) / 256;
  if (blocks > 256 * 32) blocks = 256 * 32;
  k_copy16<<<(unsigned)blocks, 256, 0, as_stream(stream)>>>(reinterpret_cast<const int4*>(src), reinterpret_cast<int4*>(dst), count);
  return check_launch("copy_kernel");
}

int cvmhip_copy_h2d(void* dst, const void* src, size_t bytes, void* stream) {
  if (bytes == 0) return CVMHIP_OK;
  HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, as_stream(stream)), "copy_h2d");
  return CVMHIP_OK;
}

int cvmhip_copy_d2h(void* dst, const void* src, size_t bytes, void* stream) {
  if (bytes == 0) return CVMHIP_OK;
  HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, as_stream(stream)), "copy_d2h");
  return CVMHIP_OK;
}

int cvmhip_copy_d2d(void* dst, const void* src, size_t bytes, void* stream) {
  if (bytes == 0 || dst == src) return CVMHIP_OK;
  HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, as_stream(stream)), "copy_d2d");
  return CVMHIP_OK;
}

int cvmhip_stream_create(void** stream) {
  if (!stream) return arg_error("stream_create");
  hipStream_t s;
  HIP_TRY(hipStreamCreate(&s), "hipStreamCreate");  // default priority
  *stream = s;
  return CVMHIP_OK;
}

int cvmhip_stream_destroy(void* stream) {
  if (stream) HIP_TRY(hipStreamDestroy(as_stream(stream)), "hipStreamDestroy");
  return CVMHIP_OK;
}

int cvmhip_stream_sync(void* stream) {
  HIP_TRY(hipStreamSynchronize(as_stream(stream)), "hipStreamSynchronize");
  return CVMHIP_OK;
}

// Timing is process-wide and meant for a single-threaded measurement harness.
int cvmhip_kernel_timing_begin(void) {
  g_launches.clear();
  g_timing = true;
  return CVMHIP_OK;
}

// Writes {"kernel": {"launches": n, "ms": total, "work": total}, ...}; with per_launch a list, in launch
// order, of {"kernel", "desc", "work", "bytes", "ms"}
static int timing_end(char* json_out, int capacity, bool per_launch) {
  g_timing = false;
  HIP_TRY(hipDeviceSynchronize(), "kernel_timing_end");
  struct Acc { long n = 0; double ms = 0, work = 0; };
  std::map<std::string, Acc> acc;
  std::string list = "[";
  for (TimedLaunch& t : g_launches) {
    float ms = 0;
    if (hipEventElapsedTime(&ms, t.e0, t.e1) == hipSuccess) {
      Acc& a = acc[t.name];
      a.n += 1;
      a.ms += ms;
      a.work += t.work;
      if (per_launch) {
        char buf[512];
        snprintf(buf, sizeof(buf), "%s{\"kernel\": \"%s\", \"desc\": \"%s\", \"work\": %.6e, \"bytes\": %.6e, \"ms\": %.6f}",
                 list.size() > 1 ? ", " : "", t.name.c_str(), t.desc.c_str(), t.work, t.bytes, ms);
        list += buf;
      }
    }
    hipEventDestroy(t.e0);
    hipEventDestroy(t.e1);
  }
  list += "]";
  g_launches.clear();
  std::string out = "{";
  bool first = true;
  for (const auto& kv : acc) {
    char buf[256];
    snprintf(buf, sizeof(buf), "%s\"%s\": {\"launches\": %ld, \"ms\": %.6f, \"work\": %.6e}", first ? "" : ", ",
             kv.first.c_str(), kv.second.n, kv.second.ms, kv.second.work);
    out += buf;
    first = false;
  }
  out += "}";
  const std::string& res = per_launch ? list : out;
  if (!json_out || (int)res.size() >= capacity) return arg_error("kernel_timing_end buffer");
  memcpy(json_out, res.c_str(), res.size() + 1);
  return CVMHIP_OK;
}

int cvmhip_kernel_timing_end(char* json_out, int capacity) { return timing_end(json_out, capacity, false); }

int cvmhip_kernel_timing_end_launches(char* json_out, int capacity) { return timing_end(json_out, capacity, true); }

int cvmhip_event_create(void** event) {
  if (!event) return arg_error("event_create");
  hipEvent_t e;
  HIP_TRY(hipEventCreate(&e), "hipEventCreate");
  *event = e;
  return CVMHIP_OK;
}

int cvmhip_event_destroy(void* event) {
  if (event) HIP_TRY(hipEventDestroy((hipEvent_t)event), "hipEventDestroy");
  return CVMHIP_OK;
}

int cvmhip_event_record(void* event, void* stream) {
  HIP_TRY(hipEventRecord((hipEvent_t)event, as_stream(stream)), "hipEventRecord");
  return CVMHIP_OK;
}

int cvmhip_device_sync(void) {
  HIP_TRY(hipDeviceSynchronize(), "hipDeviceSynchronize");
  return CVMHIP_OK;
}

int cvmhip_stream_wait_event(void* stream, void* event) {
  HIP_TRY(hipStreamWaitEvent(as_stream(stream), (hipEvent_t)event, 0), "hipStreamWaitEvent");
  return CVMHIP_OK;
}

int cvmhip_event_elapsed_ms(void* start, void* stop, float* ms) {
  HIP_TRY(hipEventSynchronize((hipEvent_t)stop), "hipEventSynchronize");
  HIP_TRY(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop), "hipEventElapsedTime");
  return CVMHIP_OK;
}

int cvmhip_kernel_timing_active(void) { return g_timing ? 1 : 0; }

int cvmhip_capture_begin(void* stream) {
  HIP_TRY(hipStreamBeginCapture(as_stream(stream), hipStreamCaptureModeThreadLocal), "hipStreamBeginCapture");
  return CVMHIP_OK;
}

int cvmhip_capture_end(void* stream, void** graph_exec) {
  if (!graph_exec) return arg_error("capture_end");
  hipGraph_t graph = nullptr;
  HIP_TRY(hipStreamEndCapture(as_stream(stream), &graph), "hipStreamEndCapture");
  hipGraphExec_t exec = nullptr;
  hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  hipGraphDestroy(graph);
  if (e != hipSuccess) {
    set_error("hipGraphInstantiate: %s", hipGetErrorString(e));
    return CVMHIP_ERR_RUNTIME;
  }
  *graph_exec = exec;
  return CVMHIP_OK;
}

int cvmhip_graph_launch(void* graph_exec, void* stream) {
  HIP_TRY(hipGraphLaunch((hipGraphExec_t)graph_exec, as_stream(stream)), "hipGraphLaunch");
  return CVMHIP_OK;
}

int cvmhip_graph_destroy(void* graph_exec) {
  if (graph_exec) HIP_TRY(hipGraphExecDestroy((hipGraphExec_t)graph_exec), "hipGraphExecDestroy");
  return CVMHIP_OK;
}

}  // extern "C"
