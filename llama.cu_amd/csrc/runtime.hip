// Runtime part of the C ABI: device set-up, buffers, copies, streams, events.
// Counterpart of llama_cu.cu:691-736 (scoped_gpu, gpu_buffer, gpu_buffer_view) and 1525-1542
// (initialize) in the reference.
#include <stdarg.h>
#include <string.h>

#include <mutex>
#include <unordered_map>

#include "common.hpp"

namespace lcu {

int attention_static_init(int device);  // attention.hip

static thread_local char g_error[512] = "";
static device_state g_devices[16];

int set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

constexpr size_t WORKSPACE_BYTES = 32u << 20;
static std::mutex g_stream_mutex;
static std::unordered_map<hipStream_t, workspace_t> g_stream_workspaces;

workspace_t workspace_for(hipStream_t stream) {
  if (stream != nullptr) {
    std::lock_guard<std::mutex> lock(g_stream_mutex);
    auto it = g_stream_workspaces.find(stream);
    if (it != g_stream_workspaces.end()) {
      return it->second;
    }
  }
  device_state* st = current_device_state();
  if (st == nullptr || !st->ready) {
    return workspace_t{};
  }
  return workspace_t{st->workspace, st->workspace_bytes, st->workspace_sync, false};
}

device_state* current_device_state() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) {
    return nullptr;
  }
  return &g_devices[dev];
}

}  // namespace lcu

using namespace lcu;

namespace {
__global__ void add_u32_kernel(uint32_t* word, uint32_t count) { atomicAdd(word, count); }
}  // namespace

extern "C" {

const char* lcu_last_error(void) { return g_error; }

int lcu_init(int device) {
  LCU_REQUIRE(device >= 0 && device < 16, "lcu_init: device %d out of range", device);
  LCU_HIP(hipSetDevice(device));
  device_state& st = g_devices[device];
  if (st.ready) {
    return LCU_OK;
  }
  hipDeviceProp_t prop;
  LCU_HIP(hipGetDeviceProperties(&prop, device));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
    return set_error(LCU_E_HIP, "lcu_init: device %d is %s, this library is built for gfx950 only",
                     device, prop.gcnArchName);
  }
  st.compute_units = prop.multiProcessorCount;
  // workspace of the default stream for operators that work in two launches (lcu_error_stats:
  // 256 x 3 partial sums; decode attention over long rows: its scores; GEMMs with few rows: the
  // fp32 partial sums of their K splits); streams from lcu_stream_create bring their own
  st.workspace_bytes = WORKSPACE_BYTES;
  LCU_HIP(hipMalloc(&st.workspace, st.workspace_bytes + SYNC_WORDS * sizeof(uint32_t)));
  LCU_HIP(hipMemset(st.workspace, 0, st.workspace_bytes + SYNC_WORDS * sizeof(uint32_t)));
  st.workspace_sync = reinterpret_cast<uint32_t*>((char*)st.workspace + st.workspace_bytes);
  LCU_HIP(hipDeviceSynchronize());
  const int rc = attention_static_init(device);
  if (rc != LCU_OK) {
    return rc;
  }
  st.ready = true;
  return LCU_OK;
}

int lcu_device_get_props(int device, lcu_device_props* out) {
  LCU_REQUIRE(out != nullptr, "lcu_device_get_props: null output");
  hipDeviceProp_t prop;
  LCU_HIP(hipGetDeviceProperties(&prop, device));
  memset(out, 0, sizeof(*out));
  snprintf(out->name, sizeof(out->name), "%s (%s)", prop.name, prop.gcnArchName);
  out->compute_units = prop.multiProcessorCount;
  out->lds_bytes_per_block = (int)prop.sharedMemPerBlock;
  out->l2_bytes = prop.l2CacheSize;
  out->clock_khz = prop.clockRate;
  out->memory_clock_khz = prop.memoryClockRate;
  out->memory_bus_bits = prop.memoryBusWidth;
  out->total_memory = prop.totalGlobalMem;
  size_t free_b = 0, total_b = 0;
  int prev = 0;
  LCU_HIP(hipGetDevice(&prev));
  LCU_HIP(hipSetDevice(device));
  LCU_HIP(hipMemGetInfo(&free_b, &total_b));
  LCU_HIP(hipSetDevice(prev));
  out->free_memory = free_b;
  return LCU_OK;
}

int lcu_get_device(int* out_device) {
  LCU_REQUIRE(out_device != nullptr, "lcu_get_device: null output");
  LCU_HIP(hipGetDevice(out_device));
  return LCU_OK;
}

int lcu_set_device(int device) {
  LCU_HIP(hipSetDevice(device));
  return LCU_OK;
}

int lcu_malloc(void** out_dev, size_t bytes) {
  LCU_REQUIRE(out_dev != nullptr, "lcu_malloc: null output");
  *out_dev = nullptr;
  if (bytes == 0) {
    return LCU_OK;
  }
  LCU_HIP(hipMalloc(out_dev, bytes));
  return LCU_OK;
}

int lcu_free(void* dev) {
  if (dev) {
    LCU_HIP(hipFree(dev));
  }
  return LCU_OK;
}

int lcu_h2d(void* dst_dev, const void* src_host, size_t bytes, void* stream) {
  if (bytes == 0) return LCU_OK;
  LCU_REQUIRE(dst_dev && src_host, "lcu_h2d: null pointer");
  LCU_HIP(hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, as_stream(stream)));
  return LCU_OK;
}

int lcu_d2h(void* dst_host, const void* src_dev, size_t bytes, void* stream) {
  if (bytes == 0) return LCU_OK;
  LCU_REQUIRE(dst_host && src_dev, "lcu_d2h: null pointer");
  LCU_HIP(hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, as_stream(stream)));
  LCU_HIP(hipStreamSynchronize(as_stream(stream)));
  return LCU_OK;
}

int lcu_d2d(void* dst_dev, const void* src_dev, size_t bytes, void* stream) {
  if (bytes == 0) return LCU_OK;
  LCU_REQUIRE(dst_dev && src_dev, "lcu_d2d: null pointer");
  LCU_HIP(hipMemcpyAsync(dst_dev, src_dev, bytes, hipMemcpyDeviceToDevice, as_stream(stream)));
  return LCU_OK;
}

int lcu_stream_create(void** out_stream) {
  LCU_REQUIRE(out_stream != nullptr, "lcu_stream_create: null output");
  hipStream_t s;
  LCU_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));  // default priority
  // the stream's own scratch, allocated here and not at first use: a first use may sit inside a
  // graph capture, where nothing may be allocated
  workspace_t ws;
  ws.bytes = WORKSPACE_BYTES;
  hipError_t e = hipMalloc(&ws.ptr, ws.bytes + SYNC_WORDS * sizeof(uint32_t));
  if (e == hipSuccess) {
    e = hipMemset(ws.ptr, 0, ws.bytes + SYNC_WORDS * sizeof(uint32_t));
  }
  if (e == hipSuccess) {
    e = hipDeviceSynchronize();  // the clearing is done before any stream can use the flags
  }
  ws.sync = reinterpret_cast<uint32_t*>((char*)ws.ptr + ws.bytes);
  ws.owned = true;
  if (e != hipSuccess) {
    (void)hipFree(ws.ptr);
    (void)hipStreamDestroy(s);
    return set_error(LCU_E_HIP, "lcu_stream_create: workspace allocation failed: %s", hipGetErrorString(e));
  }
  {
    std::lock_guard<std::mutex> lock(g_stream_mutex);
    g_stream_workspaces[s] = ws;
  }
  *out_stream = s;
  return LCU_OK;
}

int lcu_stream_destroy(void* stream) {
  if (stream) {
    workspace_t ws;
    {
      std::lock_guard<std::mutex> lock(g_stream_mutex);
      auto it = g_stream_workspaces.find(as_stream(stream));
      if (it != g_stream_workspaces.end()) {
        ws = it->second;
        g_stream_workspaces.erase(it);
      }
    }
    LCU_HIP(hipStreamSynchronize(as_stream(stream)));
    LCU_HIP(hipStreamDestroy(as_stream(stream)));
    if (ws.ptr) {
      LCU_HIP(hipFree(ws.ptr));
    }
  }
  return LCU_OK;
}

int lcu_sync_timeouts(void* stream, unsigned* out_count) {
  LCU_REQUIRE(out_count != nullptr, "lcu_sync_timeouts: null output");
  const workspace_t ws = workspace_for(as_stream(stream));
  if (ws.sync == nullptr) return set_error(LCU_E_NOINIT, "lcu_sync_timeouts: lcu_init has not run on this device");
  LCU_HIP(hipMemcpyAsync(out_count, ws.sync + SYNC_TIMEOUTS, sizeof(unsigned), hipMemcpyDeviceToHost, as_stream(stream)));
  LCU_HIP(hipStreamSynchronize(as_stream(stream)));
  return LCU_OK;
}

int lcu_sync_add_timeouts(void* stream, unsigned count) {
  const workspace_t ws = workspace_for(as_stream(stream));
  if (ws.sync == nullptr) return set_error(LCU_E_NOINIT, "lcu_sync_add_timeouts: lcu_init has not run on this device");
  add_u32_kernel<<<1, 1, 0, as_stream(stream)>>>(ws.sync + SYNC_TIMEOUTS, count);
  LCU_LAUNCH_CHECK();
  return LCU_OK;
}

int lcu_sync_reset(void* stream) {
  const workspace_t ws = workspace_for(as_stream(stream));
  if (ws.sync == nullptr) return set_error(LCU_E_NOINIT, "lcu_sync_reset: lcu_init has not run on this device");
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  if (stream) LCU_HIP(hipStreamIsCapturing(as_stream(stream), &capturing));
  LCU_REQUIRE(capturing == hipStreamCaptureStatusNone, "lcu_sync_reset: the stream is capturing");
  LCU_HIP(hipMemsetAsync(ws.sync + SYNC_EXCHANGE, 0, (size_t)(SYNC_WORDS - SYNC_EXCHANGE) * sizeof(uint32_t),
                         as_stream(stream)));
  return LCU_OK;
}

int lcu_sync(void* stream) {
  if (stream) {
    LCU_HIP(hipStreamSynchronize(as_stream(stream)));
  } else {
    LCU_HIP(hipDeviceSynchronize());
  }
  return LCU_OK;
}

int lcu_graph_begin_capture(void* stream) {
  LCU_REQUIRE(stream != nullptr, "lcu_graph_begin_capture: capture needs an explicit stream");
  LCU_HIP(hipStreamBeginCapture(as_stream(stream), hipStreamCaptureModeThreadLocal));
  return LCU_OK;
}

int lcu_graph_end_capture(void* stream, void** out_graph_exec) {
  LCU_REQUIRE(stream && out_graph_exec, "lcu_graph_end_capture: null argument");
  hipGraph_t graph = nullptr;
  LCU_HIP(hipStreamEndCapture(as_stream(stream), &graph));
  hipGraphExec_t exec = nullptr;
  hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  (void)hipGraphDestroy(graph);
  if (e != hipSuccess) {
    return set_error(LCU_E_HIP, "lcu_graph_end_capture: hipGraphInstantiate failed: %s", hipGetErrorString(e));
  }
  *out_graph_exec = exec;
  return LCU_OK;
}

int lcu_graph_launch(void* graph_exec, void* stream) {
  LCU_REQUIRE(graph_exec != nullptr, "lcu_graph_launch: null graph");
  LCU_HIP(hipGraphLaunch(reinterpret_cast<hipGraphExec_t>(graph_exec), as_stream(stream)));
  return LCU_OK;
}

int lcu_graph_destroy(void* graph_exec) {
  if (graph_exec) {
    LCU_HIP(hipGraphExecDestroy(reinterpret_cast<hipGraphExec_t>(graph_exec)));
  }
  return LCU_OK;
}

int lcu_event_create(void** out_event) {
  LCU_REQUIRE(out_event != nullptr, "lcu_event_create: null output");
  hipEvent_t e;
  LCU_HIP(hipEventCreate(&e));
  *out_event = e;
  return LCU_OK;
}

int lcu_event_destroy(void* event) {
  if (event) {
    LCU_HIP(hipEventDestroy(reinterpret_cast<hipEvent_t>(event)));
  }
  return LCU_OK;
}

int lcu_event_record(void* event, void* stream) {
  LCU_REQUIRE(event != nullptr, "lcu_event_record: null event");
  LCU_HIP(hipEventRecord(reinterpret_cast<hipEvent_t>(event), as_stream(stream)));
  return LCU_OK;
}

int lcu_event_elapsed_ms(float* out_ms, void* start_event, void* stop_event) {
  LCU_REQUIRE(out_ms && start_event && stop_event, "lcu_event_elapsed_ms: null argument");
  LCU_HIP(hipEventSynchronize(reinterpret_cast<hipEvent_t>(stop_event)));
  LCU_HIP(hipEventElapsedTime(out_ms, reinterpret_cast<hipEvent_t>(start_event),
                              reinterpret_cast<hipEvent_t>(stop_event)));
  return LCU_OK;
}

}  // extern "C"
