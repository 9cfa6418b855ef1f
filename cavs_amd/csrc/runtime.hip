// Runtime services of the C ABI: device memory, copies, streams, events, fills.
#include "common.h"

#include <cstring>

namespace cavs {

static thread_local char g_err[512] = "";
static int g_cus = 0;

int set_error(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof g_err, fmt, ap);
  va_end(ap);
  return code;
}

LaunchProbe &launch_probe() {
  static thread_local LaunchProbe probe;
  return probe;
}

int num_cus() {
  if (g_cus == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess)
      g_cus = prop.multiProcessorCount;
    if (g_cus <= 0) g_cus = 256;
  }
  return g_cus;
}

__global__ void fill_kernel(float *p, float v, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) p[i] = v;
}

__global__ void fill4_kernel(float4 *p, float v, size_t n4) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  size_t stride = (size_t)gridDim.x * blockDim.x;
  float4 x = make_float4(v, v, v, v);
  for (; i < n4; i += stride) p[i] = x;
}

static int fill_impl(float *ptr, float value, size_t n, hipStream_t st) {
  if (n == 0) return CAVS_OK;
  size_t head = 0;
  // align to 16 bytes, then vector stores, then the tail
  while (head < n && !aligned16(ptr + head)) head++;
  if (head) {
    launch(fill_kernel, 1, 64, 0, st, ptr, value, head);
  }
  size_t n4 = (n - head) / 4;
  if (n4) {
    size_t blocks = (n4 + 255) / 256;
    size_t cap = (size_t)num_cus() * 8;
    launch(fill4_kernel, (unsigned)(blocks < cap ? blocks : cap), 256, 0, st, 
        reinterpret_cast<float4 *>(ptr + head), value, n4);
  }
  size_t done = head + n4 * 4;
  if (done < n) launch(fill_kernel, 1, 64, 0, st, ptr + done, value, n - done);
  CAVS_LAUNCH_CHECK();
  return CAVS_OK;
}

}  // namespace cavs

using namespace cavs;

extern "C" {

const char *cavs_last_error(void) { return g_err; }
int cavs_abi_version(void) { return 2; }

int cavs_init(int device) {
  CAVS_HIP_TRY(hipSetDevice(device));
  g_cus = 0;
  num_cus();
  // The entry point that allocates nothing finds its scratch here, with this device current.  A
  // device on which the lookup fails keeps everything else: that entry point reports it.
  (void)static_scratch_setup(nullptr);
  return CAVS_OK;
}

int cavs_device_name(char *buf, size_t len) {
  CAVS_REQUIRE(buf && len > 0, "cavs_device_name: null buffer");
  int dev = 0;
  hipDeviceProp_t prop;
  CAVS_HIP_TRY(hipGetDevice(&dev));
  CAVS_HIP_TRY(hipGetDeviceProperties(&prop, dev));
  snprintf(buf, len, "%s (%s, %d CUs)", prop.name, prop.gcnArchName, prop.multiProcessorCount);
  return CAVS_OK;
}

int cavs_malloc(void **ptr, size_t bytes) {
  CAVS_REQUIRE(ptr, "cavs_malloc: null out pointer");
  *ptr = nullptr;
  if (bytes == 0) return CAVS_OK;
  hipError_t e = hipMalloc(ptr, bytes);
  if (e == hipErrorOutOfMemory) return set_error(CAVS_ENOMEM, "hipMalloc(%zu) out of memory", bytes);
  CAVS_HIP_TRY(e);
  return CAVS_OK;
}

int cavs_free(void *ptr) {
  if (ptr) CAVS_HIP_TRY(hipFree(ptr));
  return CAVS_OK;
}

int cavs_host_alloc(void **ptr, size_t bytes) {
  CAVS_REQUIRE(ptr, "cavs_host_alloc: null out pointer");
  *ptr = nullptr;
  if (bytes == 0) return CAVS_OK;
  CAVS_HIP_TRY(hipHostMalloc(ptr, bytes, hipHostMallocDefault));
  return CAVS_OK;
}

int cavs_host_free(void *ptr) {
  if (ptr) CAVS_HIP_TRY(hipHostFree(ptr));
  return CAVS_OK;
}

int cavs_memcpy_h2d(void *dst, const void *src, size_t bytes, void *stream) {
  if (bytes == 0) return CAVS_OK;
  CAVS_REQUIRE(dst && src, "cavs_memcpy_h2d: null pointer");
  CAVS_HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, as_stream(stream)));
  return CAVS_OK;
}

int cavs_memcpy_d2h(void *dst, const void *src, size_t bytes, void *stream) {
  if (bytes == 0) return CAVS_OK;
  CAVS_REQUIRE(dst && src, "cavs_memcpy_d2h: null pointer");
  CAVS_HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, as_stream(stream)));
  return CAVS_OK;
}

int cavs_memcpy_d2d(void *dst, const void *src, size_t bytes, void *stream) {
  if (bytes == 0) return CAVS_OK;
  CAVS_REQUIRE(dst && src, "cavs_memcpy_d2d: null pointer");
  CAVS_HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, as_stream(stream)));
  return CAVS_OK;
}

int cavs_zero(void *ptr, size_t bytes, void *stream) {
  if (bytes == 0) return CAVS_OK;
  CAVS_REQUIRE(ptr && bytes % 4 == 0 && (reinterpret_cast<uintptr_t>(ptr) & 3u) == 0,
               "cavs_zero: pointer and size must be multiples of 4 bytes");
  return fill_impl(static_cast<float *>(ptr), 0.f, bytes / 4, as_stream(stream));
}

int cavs_fill(float *ptr, float value, size_t n, void *stream) {
  if (n == 0) return CAVS_OK;
  CAVS_REQUIRE(ptr, "cavs_fill: null pointer");
  return fill_impl(ptr, value, n, as_stream(stream));
}

int cavs_stream_create(void **stream) {
  CAVS_REQUIRE(stream, "cavs_stream_create: null out pointer");
  hipStream_t s;
  CAVS_HIP_TRY(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  *stream = s;
  return CAVS_OK;
}

int cavs_stream_destroy(void *stream) {
  if (stream) CAVS_HIP_TRY(hipStreamDestroy(as_stream(stream)));
  return CAVS_OK;
}

int cavs_stream_sync(void *stream) {
  CAVS_HIP_TRY(hipStreamSynchronize(as_stream(stream)));
  return CAVS_OK;
}

int cavs_event_create(void **event) {
  CAVS_REQUIRE(event, "cavs_event_create: null out pointer");
  hipEvent_t e;
  CAVS_HIP_TRY(hipEventCreate(&e));
  *event = e;
  return CAVS_OK;
}

int cavs_event_destroy(void *event) {
  if (event) CAVS_HIP_TRY(hipEventDestroy(static_cast<hipEvent_t>(event)));
  return CAVS_OK;
}

int cavs_event_record(void *event, void *stream) {
  CAVS_REQUIRE(event, "cavs_event_record: null event");
  CAVS_HIP_TRY(hipEventRecord(static_cast<hipEvent_t>(event), as_stream(stream)));
  return CAVS_OK;
}

int cavs_stream_wait_event(void *stream, void *event) {
  CAVS_REQUIRE(event, "cavs_stream_wait_event: null event");
  CAVS_HIP_TRY(hipStreamWaitEvent(as_stream(stream), static_cast<hipEvent_t>(event), 0));
  return CAVS_OK;
}

int cavs_event_sync(void *event) {
  CAVS_REQUIRE(event, "cavs_event_sync: null event");
  CAVS_HIP_TRY(hipEventSynchronize(static_cast<hipEvent_t>(event)));
  return CAVS_OK;
}

int cavs_event_elapsed_ms(float *ms, void *start, void *stop) {
  CAVS_REQUIRE(ms && start && stop, "cavs_event_elapsed_ms: null argument");
  CAVS_HIP_TRY(hipEventSynchronize(static_cast<hipEvent_t>(stop)));
  CAVS_HIP_TRY(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
  return CAVS_OK;
}

int cavs_graph_capture_begin(void *stream) {
  CAVS_REQUIRE(stream, "cavs_graph_capture_begin: the default stream cannot be captured");
  // relaxed: other threads of the process (an allocator, another session) may go on calling the runtime
  CAVS_HIP_TRY(hipStreamBeginCapture(as_stream(stream), hipStreamCaptureModeRelaxed));
  return CAVS_OK;
}

int cavs_graph_capture_end(void *stream, void **graph_exec) {
  CAVS_REQUIRE(stream, "cavs_graph_capture_end: null stream");
  hipGraph_t graph = nullptr;
  const hipError_t rc = hipStreamEndCapture(as_stream(stream), &graph);
  if (!graph_exec) {  // the caller gives the capture up
    if (graph) (void)hipGraphDestroy(graph);
    (void)hipGetLastError();
    // (an invalidated capture is supposed to end here; if the stream is still in it, say so)
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(as_stream(stream), &status) != hipSuccess || status != hipStreamCaptureStatusNone) {
      (void)hipGetLastError();
      return cavs::set_error(CAVS_EHIP, "cavs_graph_capture_end: the stream is still in a capture (%s, status %d)", hipGetErrorString(rc),
                             (int)status);
    }
    return CAVS_OK;
  }
  *graph_exec = nullptr;
  if (rc != hipSuccess || !graph) {
    (void)hipGetLastError();
    if (graph) (void)hipGraphDestroy(graph);
    return cavs::set_error(CAVS_EHIP, "cavs_graph_capture_end: the capture was invalidated (%s)", hipGetErrorString(rc));
  }
  hipGraphExec_t exec = nullptr;
  const hipError_t ri = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  (void)hipGraphDestroy(graph);
  if (ri != hipSuccess) {
    (void)hipGetLastError();
    return cavs::set_error(CAVS_EHIP, "cavs_graph_capture_end: hipGraphInstantiate: %s", hipGetErrorString(ri));
  }
  *graph_exec = exec;
  return CAVS_OK;
}

int cavs_graph_launch(void *graph_exec, void *stream) {
  CAVS_REQUIRE(graph_exec, "cavs_graph_launch: null graph");
  CAVS_HIP_TRY(hipGraphLaunch(static_cast<hipGraphExec_t>(graph_exec), as_stream(stream)));
  return CAVS_OK;
}

int cavs_graph_destroy(void *graph_exec) {
  if (graph_exec) CAVS_HIP_TRY(hipGraphExecDestroy(static_cast<hipGraphExec_t>(graph_exec)));
  return CAVS_OK;
}

int cavs_profile_arm(void *start_event, void *stop_event) {
  CAVS_REQUIRE(start_event && stop_event, "cavs_profile_arm: null event");
  LaunchProbe &p = launch_probe();
  p.start = static_cast<hipEvent_t>(start_event);
  p.stop = static_cast<hipEvent_t>(stop_event);
  p.armed = true;
  p.started = false;
  return CAVS_OK;
}

int cavs_profile_disarm(int *launched) {
  LaunchProbe &p = launch_probe();
  if (launched) *launched = p.armed && p.started;
  p = LaunchProbe{};
  return CAVS_OK;
}

}  // extern "C"
