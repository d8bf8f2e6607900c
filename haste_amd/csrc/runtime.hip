// Library runtime: version, error text, and the per-(device, stream) workspace cache.
#include "recurrent.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <utility>
#include <vector>

namespace haste_hip {

namespace {

thread_local std::string g_last_error;

struct Key {
  int device;
  hipStream_t stream;
  bool operator<(const Key& o) const {
    return device != o.device ? device < o.device : stream < o.stream;
  }
};

std::mutex g_mutex;
std::map<Key, Workspace> g_workspaces;
std::map<int, int> g_cu_count;

// Clears a range of device words with a kernel rather than a memset node, so that
// callers may record the library's work into a HIP graph.
__global__ void fill_zero_kernel(unsigned int* p, size_t n) {
  size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0u;
}

struct TimedLaunch {
  const char* name;
  hipEvent_t start, stop;
  int products;
};
bool g_profile_on = false;
std::vector<TimedLaunch> g_timed;

}  // namespace

ScopedKernelTimer::ScopedKernelTimer(const char* name, hipStream_t stream, int products)
    : stream_(stream), slot_(-1) {
  if (!g_profile_on) return;
  TimedLaunch t;
  t.name = name;
  t.products = products;
  if (hipEventCreate(&t.start) != hipSuccess) return;
  if (hipEventCreate(&t.stop) != hipSuccess) { (void)hipEventDestroy(t.start); return; }
  (void)hipEventRecord(t.start, stream);
  std::lock_guard<std::mutex> lock(g_mutex);
  g_timed.push_back(t);
  slot_ = (int)g_timed.size() - 1;
}

ScopedKernelTimer::~ScopedKernelTimer() {
  if (slot_ < 0) return;
  std::lock_guard<std::mutex> lock(g_mutex);
  if (slot_ < (int)g_timed.size()) (void)hipEventRecord(g_timed[slot_].stop, stream_);
}

void set_runtime_error(hipError_t err, const char* what) {
  char buf[512];
  std::snprintf(buf, sizeof(buf), "%s: %s (%d)", what, hipGetErrorString(err), (int)err);
  g_last_error = buf;
  (void)hipGetLastError();  // do not leave the error for an unrelated later call
}

void set_error_text(const char* text) { g_last_error = text; }

namespace {
struct LastPersistent {
  hipEvent_t event = nullptr;
  hipStream_t stream = nullptr;
  bool valid = false;
};
std::map<int, LastPersistent> g_last_persistent;
}  // namespace

int order_persistent_launches(hipStream_t stream, bool before) {
  int dev = 0;
  HASTE_HIP_TRY(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(g_mutex);
  LastPersistent& lp = g_last_persistent[dev];
  if (before) {
    if (lp.valid && lp.stream != stream) HASTE_HIP_TRY(hipStreamWaitEvent(stream, lp.event, 0));
    return HASTE_HIP_OK;
  }
  if (lp.event == nullptr) HASTE_HIP_TRY(hipEventCreateWithFlags(&lp.event, hipEventDisableTiming));
  HASTE_HIP_TRY(hipEventRecord(lp.event, stream));
  lp.stream = stream;
  lp.valid = true;
  return HASTE_HIP_OK;
}

bool xcd_local_enabled() {
  static const bool enabled = [] {
    const char* v = std::getenv("HASTE_HIP_XCD_LOCAL");
    return v == nullptr || v[0] != '0';
  }();
  return enabled;
}

bool paired_sets_enabled() {
  static const bool enabled = [] {
    const char* v = std::getenv("HASTE_HIP_PAIRED_SETS");
    return v == nullptr || v[0] != '0';
  }();
  return enabled;
}

bool single_row_enabled() {
  static const bool enabled = [] {
    const char* v = std::getenv("HASTE_HIP_SINGLE_ROW");
    return v == nullptr || v[0] != '0';
  }();
  return enabled;
}

bool fused_input_enabled() {
  static const bool enabled = [] {
    const char* v = std::getenv("HASTE_HIP_FUSED_INPUT");
    return v == nullptr || v[0] != '0';
  }();
  return enabled;
}

int device_cu_count() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  std::lock_guard<std::mutex> lock(g_mutex);
  auto it = g_cu_count.find(dev);
  if (it != g_cu_count.end()) return it->second;
  int n = 0;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) n = 0;
  g_cu_count[dev] = n;
  return n;
}

int get_workspace(hipStream_t stream, size_t scratch_bytes, Workspace* out) {
  int dev = 0;
  HASTE_HIP_TRY(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(g_mutex);
  Workspace& ws = g_workspaces[Key{dev, stream}];
  if (ws.control == nullptr) {
    HASTE_HIP_TRY(hipMalloc(reinterpret_cast<void**>(&ws.control), sizeof(ControlBlock)));
    const size_t words = sizeof(ControlBlock) / sizeof(unsigned int);
    fill_zero_kernel<<<dim3((unsigned)((words + 255) / 256)), dim3(256), 0, stream>>>(
        reinterpret_cast<unsigned int*>(ws.control), words);
    HASTE_HIP_TRY(hipGetLastError());
    HASTE_HIP_TRY(hipHostMalloc(reinterpret_cast<void**>(&ws.host_status), 64,
                                hipHostMallocMapped));
    std::memset(ws.host_status, 0, 64);
    HASTE_HIP_TRY(hipHostGetDevicePointer(reinterpret_cast<void**>(&ws.host_status_dev),
                                          ws.host_status, 0));
  }
  if (ws.scratch_bytes < scratch_bytes) {
    // Growing replaces the buffer; work already enqueued on the stream may still be
    // using the old one, so the stream is drained first (rare: sizes stabilise
    // after the first call of each shape).
    if (ws.scratch != nullptr) {
      HASTE_HIP_TRY(hipStreamSynchronize(stream));
      HASTE_HIP_TRY(hipFree(ws.scratch));
      ws.scratch = nullptr;
      ws.scratch_bytes = 0;
    }
    size_t bytes = (scratch_bytes + (size_t(1) << 20) - 1) & ~((size_t(1) << 20) - 1);
    HASTE_HIP_TRY(hipMalloc(reinterpret_cast<void**>(&ws.scratch), bytes));
    ws.scratch_bytes = bytes;
  }
  *out = ws;
  return HASTE_HIP_OK;
}

int reserve_epochs(hipStream_t stream, unsigned int count, unsigned int* base) {
  int dev = 0;
  HASTE_HIP_TRY(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(g_mutex);
  auto it = g_workspaces.find(Key{dev, stream});
  if (it == g_workspaces.end()) return HASTE_HIP_ERROR_INVALID_ARGUMENT;
  *base = it->second.epoch;
  it->second.epoch += count;
  return HASTE_HIP_OK;
}

int reserve_tickets(hipStream_t stream, unsigned int count, unsigned int* base) {
  int dev = 0;
  HASTE_HIP_TRY(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(g_mutex);
  auto it = g_workspaces.find(Key{dev, stream});
  if (it == g_workspaces.end()) return HASTE_HIP_ERROR_INVALID_ARGUMENT;
  *base = it->second.ticket_base;
  it->second.ticket_base += count;
  return HASTE_HIP_OK;
}

int check_and_clear_abort(hipStream_t stream, Workspace* ws) {
  volatile unsigned int* status = ws->host_status;
  if (status == nullptr || *status == 0u) return HASTE_HIP_OK;
  *status = 0u;
  {
    // the control block is wiped below, so flag and ticket numbering restart from zero
    int dev = 0;
    HASTE_HIP_TRY(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lock(g_mutex);
    auto it = g_workspaces.find(Key{dev, stream});
    if (it != g_workspaces.end()) {
      it->second.epoch = 0;
      it->second.ticket_base = 0;
    }
  }
  const size_t words = sizeof(ControlBlock) / sizeof(unsigned int);
  fill_zero_kernel<<<dim3((unsigned)((words + 255) / 256)), dim3(256), 0, stream>>>(
      reinterpret_cast<unsigned int*>(ws->control), words);
  HASTE_HIP_TRY(hipGetLastError());
  return HASTE_HIP_ERROR_STEP_BARRIER;
}

}  // namespace haste_hip

extern "C" {

int haste_hip_version(void) { return 100; }  // 0.1.0

const char* haste_hip_error_string(int code) {
  switch (code) {
    case HASTE_HIP_OK: return "ok";
    case HASTE_HIP_ERROR_INVALID_ARGUMENT: return "invalid argument (null pointer or non-positive dimension)";
    case HASTE_HIP_ERROR_UNSUPPORTED_SIZE: return "unsupported size (recurrent weight slice does not fit on chip or batch too large for one cooperative grid)";
    case HASTE_HIP_ERROR_RUNTIME: return "HIP runtime error";
    case HASTE_HIP_ERROR_STEP_BARRIER: return "a persistent kernel launched earlier timed out at its step barrier";
    default: return "unknown error code";
  }
}

const char* haste_hip_last_runtime_error(void) { return haste_hip::g_last_error.c_str(); }

int haste_hip_stream_order(void* first, void* then) {
  if (first == then) return HASTE_HIP_OK;
  hipEvent_t ev;
  HASTE_HIP_TRY(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
  hipError_t err = hipEventRecord(ev, haste_hip::as_stream(first));
  if (err == hipSuccess) err = hipStreamWaitEvent(haste_hip::as_stream(then), ev, 0);
  // Destroying a recorded event is legal: its resources are released once it has completed.
  const hipError_t err2 = hipEventDestroy(ev);
  HASTE_HIP_TRY(err);
  HASTE_HIP_TRY(err2);
  return HASTE_HIP_OK;
}

int haste_hip_max_hidden_size(int gates, int batch_size) {
  if (gates < 1 || gates > 4 || batch_size < 1) return 0;
  if (haste_hip::device_cu_count() <= 0) return 0;
  // The geometry search of the LSTM (4 gates) / GRU (3 gates) entry points themselves: the
  // largest hidden size for which both the forward and the backward recurrence find a tile.
  auto fits = [&](int H) {
    const int k_back = gates == 3 ? 48 * ((H + 15) / 16) : gates * H;
    const size_t reduce_floats = gates == 3 ? 6 * 16 : (size_t)gates * 16;
    return haste_hip::pick_forward_tile(gates, batch_size, H, 0, haste_hip::kWorkgroupLdsBytes).ok &&
           haste_hip::pick_backward_tile(k_back, batch_size, H, reduce_floats, 0).ok;
  };
  int best = 0;
  for (int H = 16; H <= 8192; H += 16)
    if (fits(H)) best = H;
  return best;
}

int haste_hip_profile_enable(int on) {
  std::lock_guard<std::mutex> lock(haste_hip::g_mutex);
  haste_hip::g_profile_on = on != 0;
  return HASTE_HIP_OK;
}

int haste_hip_profile_reset(void) {
  std::lock_guard<std::mutex> lock(haste_hip::g_mutex);
  for (auto& t : haste_hip::g_timed) {
    (void)hipEventSynchronize(t.stop);
    (void)hipEventDestroy(t.start);
    (void)hipEventDestroy(t.stop);
  }
  haste_hip::g_timed.clear();
  return HASTE_HIP_OK;
}

int haste_hip_profile_read(const char* name, double* total_ms, int* launches) {
  if (name == nullptr || total_ms == nullptr || launches == nullptr)
    return HASTE_HIP_ERROR_INVALID_ARGUMENT;
  std::lock_guard<std::mutex> lock(haste_hip::g_mutex);
  double total = 0.0;
  int count = 0;
  for (auto& t : haste_hip::g_timed) {
    if (std::strcmp(t.name, name) != 0) continue;
    if (hipEventSynchronize(t.stop) != hipSuccess) return HASTE_HIP_ERROR_RUNTIME;
    float ms = 0.f;
    if (hipEventElapsedTime(&ms, t.start, t.stop) != hipSuccess) return HASTE_HIP_ERROR_RUNTIME;
    total += ms;
    count += t.products;
  }
  *total_ms = total;
  *launches = count;
  return HASTE_HIP_OK;
}

int haste_hip_release_workspaces(void) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return HASTE_HIP_ERROR_RUNTIME;
  std::lock_guard<std::mutex> lock(haste_hip::g_mutex);
  for (auto it = haste_hip::g_workspaces.begin(); it != haste_hip::g_workspaces.end();) {
    if (it->first.device == dev) {
      if (it->second.scratch) (void)hipFree(it->second.scratch);
      if (it->second.control) (void)hipFree(it->second.control);
      if (it->second.host_status) (void)hipHostFree(it->second.host_status);
      it = haste_hip::g_workspaces.erase(it);
    } else {
      ++it;
    }
  }
  return HASTE_HIP_OK;
}

}  // extern "C"
