// Device, stream, memory and event entry points of the C ABI: the HIP runtime
// calls a Minerva device needs (reference minerva/device/device.cpp:146-222).
#include <stdio.h>
#include <string.h>

#include <atomic>

#include "mnv_common.h"

int mnv_cu_count() {
  static std::atomic<int> cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
    (void)hipGetLastError();
    return 256;
  }
  int n = cached[dev].load(std::memory_order_relaxed);
  if (n > 0) return n;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 1) {
    (void)hipGetLastError();
    return 256;
  }
  cached[dev].store(n, std::memory_order_relaxed);
  return n;
}

extern "C" {

int mnv_device_count(int* count) {
  if (!count) return MNV_ERR_INVALID;
  MNV_HIP_TRY(hipGetDeviceCount(count));
  return MNV_OK;
}

int mnv_device_set(int device) {
  MNV_HIP_TRY(hipSetDevice(device));
  return MNV_OK;
}

int mnv_device_info(int device, char* name_out, int* cu_count, int* clock_khz, size_t* hbm_bytes) {
  hipDeviceProp_t prop;
  MNV_HIP_TRY(hipGetDeviceProperties(&prop, device));
  if (name_out) {
    snprintf(name_out, 256, "%s (%s)", prop.name, prop.gcnArchName);
  }
  if (cu_count) *cu_count = prop.multiProcessorCount;
  if (clock_khz) *clock_khz = prop.clockRate;
  if (hbm_bytes) *hbm_bytes = prop.totalGlobalMem;
  return MNV_OK;
}

int mnv_stream_create(mnv_stream_t* stream) {
  if (!stream) return MNV_ERR_INVALID;
  hipStream_t s;
  MNV_HIP_TRY(hipStreamCreate(&s));  // default priority only
  *stream = reinterpret_cast<mnv_stream_t>(s);
  return MNV_OK;
}

int mnv_stream_destroy(mnv_stream_t stream) {
  if (!stream) return MNV_ERR_INVALID;
  MNV_HIP_TRY(hipStreamDestroy(mnv_stream(stream)));
  return MNV_OK;
}

int mnv_stream_sync(mnv_stream_t stream) {
  MNV_HIP_TRY(hipStreamSynchronize(mnv_stream(stream)));
  return MNV_OK;
}

int mnv_device_sync(void) {
  MNV_HIP_TRY(hipDeviceSynchronize());
  return MNV_OK;
}

int mnv_malloc(void** ptr, size_t bytes) {
  if (!ptr) return MNV_ERR_INVALID;
  *ptr = nullptr;
  if (bytes == 0) return MNV_OK;
  MNV_HIP_TRY(hipMalloc(ptr, bytes));
  return MNV_OK;
}

int mnv_free(void* ptr) {
  if (!ptr) return MNV_OK;
  MNV_HIP_TRY(hipFree(ptr));
  return MNV_OK;
}

int mnv_host_malloc(void** ptr, size_t bytes) {
  if (!ptr) return MNV_ERR_INVALID;
  *ptr = nullptr;
  if (bytes == 0) return MNV_OK;
  MNV_HIP_TRY(hipHostMalloc(ptr, bytes, hipHostMallocDefault));
  return MNV_OK;
}

int mnv_host_free(void* ptr) {
  if (!ptr) return MNV_OK;
  MNV_HIP_TRY(hipHostFree(ptr));
  return MNV_OK;
}

int mnv_memcpy_h2d(void* dst, const void* src_host, size_t bytes, mnv_stream_t stream) {
  if (bytes == 0) return MNV_OK;
  if (!dst || !src_host) return MNV_ERR_INVALID;
  MNV_HIP_TRY(hipMemcpyAsync(dst, src_host, bytes, hipMemcpyHostToDevice, mnv_stream(stream)));
  return MNV_OK;
}

int mnv_memcpy_d2h(void* dst_host, const void* src, size_t bytes, mnv_stream_t stream) {
  if (bytes == 0) return MNV_OK;
  if (!dst_host || !src) return MNV_ERR_INVALID;
  MNV_HIP_TRY(hipMemcpyAsync(dst_host, src, bytes, hipMemcpyDeviceToHost, mnv_stream(stream)));
  return MNV_OK;
}

int mnv_memcpy_d2d(void* dst, const void* src, size_t bytes, mnv_stream_t stream) {
  if (bytes == 0) return MNV_OK;
  if (!dst || !src) return MNV_ERR_INVALID;
  MNV_HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, mnv_stream(stream)));
  return MNV_OK;
}

int mnv_event_create(void** event) {
  if (!event) return MNV_ERR_INVALID;
  hipEvent_t e;
  MNV_HIP_TRY(hipEventCreate(&e));
  *event = reinterpret_cast<void*>(e);
  return MNV_OK;
}

int mnv_event_create_ordering(void** event) {
  if (!event) return MNV_ERR_INVALID;
  hipEvent_t e;
  MNV_HIP_TRY(hipEventCreateWithFlags(&e, hipEventDisableTiming));
  *event = reinterpret_cast<void*>(e);
  return MNV_OK;
}

int mnv_stream_wait_event(mnv_stream_t stream, void* event) {
  if (!event) return MNV_ERR_INVALID;
  MNV_HIP_TRY(hipStreamWaitEvent(mnv_stream(stream), reinterpret_cast<hipEvent_t>(event), 0));
  return MNV_OK;
}

int mnv_event_destroy(void* event) {
  if (!event) return MNV_ERR_INVALID;
  MNV_HIP_TRY(hipEventDestroy(reinterpret_cast<hipEvent_t>(event)));
  return MNV_OK;
}

int mnv_event_record(void* event, mnv_stream_t stream) {
  if (!event) return MNV_ERR_INVALID;
  MNV_HIP_TRY(hipEventRecord(reinterpret_cast<hipEvent_t>(event), mnv_stream(stream)));
  return MNV_OK;
}

int mnv_event_sync(void* event) {
  if (!event) return MNV_ERR_INVALID;
  MNV_HIP_TRY(hipEventSynchronize(reinterpret_cast<hipEvent_t>(event)));
  return MNV_OK;
}

int mnv_event_elapsed_ms(void* start, void* stop, float* ms) {
  if (!start || !stop || !ms) return MNV_ERR_INVALID;
  MNV_HIP_TRY(hipEventElapsedTime(ms, reinterpret_cast<hipEvent_t>(start),
                                  reinterpret_cast<hipEvent_t>(stop)));
  return MNV_OK;
}

// ---- stream capture.  A launch-bound sequence of operators (a whole training step of a
// small network is a few dozen short kernels) is recorded once into a HIP graph and then
// replayed with one launch.  Only kernel launches may be recorded: the operator entry
// points of this library issue nothing else once their one-time set-up has run, so a
// sequence is executed once eagerly before it is captured.

int mnv_graph_begin_capture(mnv_stream_t stream) {
  if (!stream) return MNV_ERR_INVALID;  // the default stream cannot be captured
  MNV_HIP_TRY(hipStreamBeginCapture(mnv_stream(stream), hipStreamCaptureModeGlobal));
  return MNV_OK;
}

int mnv_graph_end_capture(mnv_stream_t stream, void** graph_exec, size_t* num_nodes) {
  if (!stream || !graph_exec) return MNV_ERR_INVALID;
  *graph_exec = nullptr;
  hipGraph_t graph = nullptr;
  MNV_HIP_TRY(hipStreamEndCapture(mnv_stream(stream), &graph));
  if (!graph) return MNV_ERR_INVALID;
  if (num_nodes) {
    hipError_t e = hipGraphGetNodes(graph, nullptr, num_nodes);
    if (e != hipSuccess) {
      hipGraphDestroy(graph);
      return (int)e;
    }
  }
  hipGraphExec_t exec = nullptr;
  hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  hipGraphDestroy(graph);
  if (e != hipSuccess) return (int)e;
  *graph_exec = reinterpret_cast<void*>(exec);
  return MNV_OK;
}

int mnv_graph_abort_capture(mnv_stream_t stream) {
  if (!stream) return MNV_ERR_INVALID;
  hipGraph_t graph = nullptr;
  hipError_t e = hipStreamEndCapture(mnv_stream(stream), &graph);
  if (graph) hipGraphDestroy(graph);
  (void)hipGetLastError();  // an invalidated capture reports its error here; it is dropped
  return e == hipSuccess || e == hipErrorStreamCaptureInvalidated ? MNV_OK : (int)e;
}

int mnv_graph_launch(void* graph_exec, mnv_stream_t stream) {
  if (!graph_exec) return MNV_ERR_INVALID;
  MNV_HIP_TRY(hipGraphLaunch(reinterpret_cast<hipGraphExec_t>(graph_exec), mnv_stream(stream)));
  return MNV_OK;
}

int mnv_graph_destroy(void* graph_exec) {
  if (!graph_exec) return MNV_OK;
  MNV_HIP_TRY(hipGraphExecDestroy(reinterpret_cast<hipGraphExec_t>(graph_exec)));
  return MNV_OK;
}

const char* mnv_error_string(int status) {
  if (status == MNV_OK) return "ok";
  if (status == MNV_ERR_INVALID) return "invalid argument (null pointer or non-positive extent)";
  if (status == MNV_ERR_WORKSPACE) return "workspace too small";
  if (status == MNV_ERR_TOO_LARGE) return "problem exceeds the maximum of this entry point's fixed scratch area";
  return hipGetErrorString(static_cast<hipError_t>(status));
}

}  // extern "C"
