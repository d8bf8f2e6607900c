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

namespace {
std::mutex g_persistent_order_mutex;
}  // namespace

PersistentLaunchOrder::PersistentLaunchOrder() { g_persistent_order_mutex.lock(); }
PersistentLaunchOrder::~PersistentLaunchOrder() { g_persistent_order_mutex.unlock(); }

int order_persistent_launches(hipStream_t stream, bool before) {
  int dev = 0;
  HASTE_HIP_TRY(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(g_mutex);
  LastPersistent& lp = g_last_persistent[dev];
  // A stream that is being captured into a graph is ordered by the graph: an event recorded
  // into a capture could not be waited for by eager work afterwards.  (While a graph with
  // persistent kernels replays, the caller keeps other persistent launches off the device.)
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &capture) != hipSuccess) (void)hipGetLastError();
  if (capture != hipStreamCaptureStatusNone) return HASTE_HIP_OK;
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

namespace {

// Where the workgroups of a launch of one workgroup per CU run: the placement the XCD-local
// launches of the persistent kernels rely on, looked at once per device.
__global__ void xcc_probe_kernel(unsigned int* out) {
  if (threadIdx.x == 0) out[blockIdx.x] = xcc_id();
}

struct XcdLayout {
  bool probed = false;
  int count = 0;                 // 0: no XCD-local launches on this device
  unsigned long long map = 0;    // 4 bits per hardware XCC id: its index among those in use
};
std::map<int, XcdLayout> g_xcd_layout;

bool xcd_local_requested() {
  static const bool enabled = [] {
    const char* v = std::getenv("HASTE_HIP_XCD_LOCAL");
    return v == nullptr || v[0] != '0';
  }();
  return enabled;
}

// One attempt: true when `cus` workgroups that cannot share a CU spread evenly over the XCDs.
bool probe_xcd_layout(int cus, XcdLayout* out) {
  const size_t lds = 84 * 1024;  // more than half of a CU's LDS, as in plan_launch
  unsigned int* dev_ids = nullptr;
  if (hipMalloc(reinterpret_cast<void**>(&dev_ids), (size_t)cus * sizeof(unsigned int)) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  std::vector<unsigned int> ids((size_t)cus, 0u);
  bool ok = hipFuncSetAttribute(reinterpret_cast<const void*>(xcc_probe_kernel),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) == hipSuccess;
  // Nothing else of this process may hold CUs while the probe runs.
  ok = ok && hipDeviceSynchronize() == hipSuccess;
  if (ok) {
    xcc_probe_kernel<<<dim3((unsigned)cus), dim3(64), lds, nullptr>>>(dev_ids);
    ok = hipGetLastError() == hipSuccess &&
         hipMemcpy(ids.data(), dev_ids, (size_t)cus * sizeof(unsigned int), hipMemcpyDeviceToHost) == hipSuccess;
  }
  (void)hipFree(dev_ids);
  if (!ok) {
    (void)hipGetLastError();
    return false;
  }
  int per_id[16] = {0};
  for (unsigned int id : ids) per_id[id & 15u] += 1;
  int count = 0;
  unsigned long long map = 0;
  for (int id = 0; id < 16; ++id) {
    if (per_id[id] == 0) continue;
    map |= (unsigned long long)count << (4 * id);
    count += 1;
  }
  if (count == 0 || cus % count != 0) return false;
  for (int id = 0; id < 16; ++id)
    if (per_id[id] != 0 && per_id[id] != cus / count) return false;
  out->count = count;
  out->map = map;
  return true;
}

// g_mutex held.
XcdLayout& xcd_layout_locked(int dev) {
  XcdLayout& x = g_xcd_layout[dev];
  if (!x.probed) {
    x.probed = true;
    int cus = 0;
    if (xcd_local_requested() &&
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && cus > 0) {
      // A kernel of another process may hold CUs for a moment: up to three looks.
      for (int attempt = 0; attempt < 3 && x.count == 0; ++attempt) (void)probe_xcd_layout(cus, &x);
      if (x.count == 0)
        set_error_text("the look at the device's XCD placement failed (CUs held by other work, a partition "
                       "mode or a CU mask): the persistent kernels use the placement-independent path");
    }
  }
  return x;
}

}  // namespace

int xcd_layout_ready(hipStream_t stream) {
  int dev = 0;
  HASTE_HIP_TRY(hipGetDevice(&dev));
  {
    std::lock_guard<std::mutex> lock(g_mutex);
    auto it = g_xcd_layout.find(dev);
    if (it != g_xcd_layout.end() && it->second.probed) return HASTE_HIP_OK;
  }
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &capture) != hipSuccess) (void)hipGetLastError();
  if (capture != hipStreamCaptureStatusNone) {
    set_error_text("the first persistent launch on a device looks at its XCD placement (allocation, device "
                   "synchronization): call haste_hip_set_workspace or any entry point once before capturing");
    return HASTE_HIP_ERROR_RUNTIME;
  }
  (void)device_xcd_count();
  return HASTE_HIP_OK;
}

namespace {
// A device shape assumed by this thread instead of the current device's (haste_hip_plan_tiles).
thread_local int t_assumed_cus = 0, t_assumed_xcds = 0;
}  // namespace

int device_xcd_count() {
  if (t_assumed_cus > 0) return t_assumed_xcds;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  std::lock_guard<std::mutex> lock(g_mutex);
  return xcd_layout_locked(dev).count;
}

unsigned long long device_xcc_logical_map() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  std::lock_guard<std::mutex> lock(g_mutex);
  return xcd_layout_locked(dev).map;
}

namespace {
bool test_hooks_requested() {
  static const bool on = [] {
    const char* v = std::getenv("HASTE_HIP_TEST_HOOKS");
    return v != nullptr && v[0] == '1';
  }();
  return on;
}
}  // namespace

unsigned int spin_limit() {
  static const unsigned int limit = [] {
    const char* v = std::getenv("HASTE_HIP_SPIN_LIMIT");
    const unsigned long n = v != nullptr ? std::strtoul(v, nullptr, 10) : 0ul;
    if (n == 0 || n >= (1ul << 31)) return 1u << 24;
    // an inherited variable must not make healthy launches give up: a floor of milliseconds
    const unsigned long floor = test_hooks_requested() ? 1ul : 1ul << 16;
    return (unsigned int)(n < floor ? floor : n);
  }();
  return limit;
}

int test_absent_workgroups() {
  static const int absent = [] {
    if (!test_hooks_requested()) return 0;
    const char* v = std::getenv("HASTE_HIP_TEST_ABSENT_WORKGROUP");
    const long n = v != nullptr ? std::strtol(v, nullptr, 10) : 0l;
    return n > 0 && n <= 4 ? (int)n : 0;
  }();
  return absent;
}

bool fused_input_enabled() {
  static const bool enabled = [] {
    const char* v = std::getenv("HASTE_HIP_FUSED_INPUT");
    return v == nullptr || v[0] != '0';
  }();
  return enabled;
}

int device_cu_count() {
  if (t_assumed_cus > 0) return t_assumed_cus;
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

namespace {

constexpr size_t kControlBytes = (sizeof(ControlBlock) + 255) / 256 * 256;

int zero_control(hipStream_t stream, ControlBlock* control) {
  const size_t words = sizeof(ControlBlock) / sizeof(unsigned int);
  fill_zero_kernel<<<dim3((unsigned)((words + 255) / 256)), dim3(256), 0, stream>>>(
      reinterpret_cast<unsigned int*>(control), words);
  HASTE_HIP_TRY(hipGetLastError());
  return HASTE_HIP_OK;
}

// The pinned word the kernels report to.  Kept for the life of the workspace.
int ensure_host_status(Workspace& ws) {
  if (ws.host_status != nullptr) return HASTE_HIP_OK;
  unsigned int* host = nullptr;
  unsigned int* dev = nullptr;
  HASTE_HIP_TRY(hipHostMalloc(reinterpret_cast<void**>(&host), 64, hipHostMallocMapped));
  std::memset(host, 0, 64);
  const hipError_t err = hipHostGetDevicePointer(reinterpret_cast<void**>(&dev), host, 0);
  if (err != hipSuccess) {
    (void)hipHostFree(host);
    HASTE_HIP_TRY(err);
  }
  ws.host_status = host;
  ws.host_status_dev = dev;
  return HASTE_HIP_OK;
}

// Creates the library-owned control block of `ws`; leaves `ws` without one (so that the next
// call starts over) when any step fails.
int create_control(hipStream_t stream, Workspace& ws) {
  HASTE_HIP_PROPAGATE(ensure_host_status(ws));
  ControlBlock* control = nullptr;
  HASTE_HIP_TRY(hipMalloc(reinterpret_cast<void**>(&control), sizeof(ControlBlock)));
  const int rc = zero_control(stream, control);
  if (rc != HASTE_HIP_OK) {
    (void)hipFree(control);
    return rc;
  }
  ws.control = control;
  ws.epoch = 0;
  ws.ticket_base = 0;
  return HASTE_HIP_OK;
}

// What a reported abort means for later launches: the control block is wiped (on `stream`), so
// flag and ticket numbering restart from zero; a launch that found an XCD with more workgroups
// than it had been promised (status 2) ends the XCD-local launches on this device.  g_mutex held.
int recover_from_abort_locked(int dev, hipStream_t stream, Workspace& ws, unsigned int status) {
  if (status == 2u) {
    XcdLayout& x = xcd_layout_locked(dev);
    x.count = 0;
    x.map = 0;
    set_error_text("a persistent kernel found more workgroups on an XCD than its launch assumed "
                   "(partitioned or masked device, or CUs held by other work): its results are "
                   "invalid; later launches use the placement-independent path");
  } else {
    set_error_text("a persistent kernel gave up waiting for another workgroup (step barrier / "
                   "exchange time-out): the results of that launch and of launches queued behind "
                   "it on the device are invalid");
  }
  ws.epoch = 0;
  ws.ticket_base = 0;
  HASTE_HIP_PROPAGATE(zero_control(stream, ws.control));
  return HASTE_HIP_ERROR_STEP_BARRIER;
}

}  // namespace

namespace {
thread_local size_t t_scratch_prefix = 0;
}  // namespace

ScratchPrefix::ScratchPrefix(size_t bytes) : saved_(t_scratch_prefix) { t_scratch_prefix = saved_ + bytes; }
ScratchPrefix::~ScratchPrefix() { t_scratch_prefix = saved_; }

int get_workspace(hipStream_t stream, size_t scratch_bytes, Workspace* out) {
  int dev = 0;
  HASTE_HIP_TRY(hipGetDevice(&dev));
  const size_t prefix = t_scratch_prefix;
  scratch_bytes += prefix;
  std::lock_guard<std::mutex> lock(g_mutex);
  Workspace& ws = g_workspaces[Key{dev, stream}];
  if (ws.control == nullptr) HASTE_HIP_PROPAGATE(create_control(stream, ws));
  // A persistent kernel launched earlier on this stream gave up: whichever entry point comes
  // next says so, once, instead of working on what that launch left behind.
  if (ws.host_status != nullptr) {
    volatile unsigned int* status = ws.host_status;
    const unsigned int seen = *status;
    if (seen != 0u) {
      *status = 0u;
      return recover_from_abort_locked(dev, stream, ws, seen);
    }
  }
  if (ws.scratch_bytes < scratch_bytes) {
    if (ws.caller_owned) {
      char buf[200];
      std::snprintf(buf, sizeof(buf),
                    "the workspace set with haste_hip_set_workspace is too small: this call needs %zu bytes",
                    scratch_bytes + kControlBytes);
      set_error_text(buf);
      return HASTE_HIP_ERROR_UNSUPPORTED_SIZE;
    }
    if (prefix != 0) {
      set_error_text("internal: the scratch buffer would have to grow while an entry point keeps staged "
                     "tensors in it");
      return HASTE_HIP_ERROR_UNSUPPORTED_SIZE;
    }
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
  if (ws.scratch_high_water < scratch_bytes) ws.scratch_high_water = scratch_bytes;
  *out = ws;
  out->scratch = reinterpret_cast<float*>(reinterpret_cast<char*>(ws.scratch) + prefix);
  out->scratch_bytes = ws.scratch_bytes - prefix;
  return HASTE_HIP_OK;
}

// The step flags count up from `epoch` and are never cleared, and the tagged row exchange of
// the layer-norm cells uses epoch + 2 + step as its tags, 0 meaning "nothing expected yet":
// before the numbering could wrap (or a tag become 0) the control block is wiped, in stream
// order, and the numbering starts over.
constexpr unsigned int kEpochLimit = 0xe0000000u;

int reserve_epochs(hipStream_t stream, unsigned int count, unsigned int* base) {
  int dev = 0;
  HASTE_HIP_TRY(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(g_mutex);
  auto it = g_workspaces.find(Key{dev, stream});
  if (it == g_workspaces.end()) return HASTE_HIP_ERROR_INVALID_ARGUMENT;
  Workspace& ws = it->second;
  if (count >= kEpochLimit) return HASTE_HIP_ERROR_UNSUPPORTED_SIZE;
  // A launch recorded into a graph runs again with the numbers it was recorded with, whatever
  // has run in between: from the first captured launch on, every persistent launch on this
  // stream wipes the control block itself (a small kernel in front of it, recorded with it) and
  // counts from zero.
  if (!ws.self_resetting) {
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &capture) != hipSuccess) (void)hipGetLastError();
    if (capture != hipStreamCaptureStatusNone) ws.self_resetting = true;
  }
  if (ws.self_resetting || ws.epoch > kEpochLimit - count) {
    HASTE_HIP_PROPAGATE(zero_control(stream, ws.control));
    ws.epoch = 0;
    ws.ticket_base = 0;
  }
  *base = ws.epoch;
  ws.epoch += count;
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
  const unsigned int seen = *status;
  *status = 0u;
  int dev = 0;
  HASTE_HIP_TRY(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(g_mutex);
  auto it = g_workspaces.find(Key{dev, stream});
  if (it == g_workspaces.end()) return HASTE_HIP_ERROR_STEP_BARRIER;
  return recover_from_abort_locked(dev, stream, it->second, seen);
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
    const int max_ct = gates == 3 ? 3 : (gates == 4 ? 2 : 0);
    return haste_hip::pick_forward_tile(gates, batch_size, H, 0, haste_hip::kWorkgroupLdsBytes, false, max_ct).ok &&
           haste_hip::pick_backward_tile(k_back, batch_size, H, reduce_floats, 0, true).ok;
  };
  int best = 0;
  for (int H = 16; H <= 8192; H += 16)
    if (fits(H)) best = H;
  return best;
}

int haste_hip_plan_tiles(int cus, int xcds, int gates, int batch_size, int hidden_size, int* plan) {
  HASTE_HIP_REQUIRE(plan != nullptr && (gates == 3 || gates == 4) && batch_size > 0 && hidden_size > 0);
  HASTE_HIP_REQUIRE(cus >= 0 && xcds >= 0 && (cus > 0 || xcds == 0));
  using namespace haste_hip;
  const int H = hidden_size;
  t_assumed_cus = cus;
  t_assumed_xcds = xcds;
  const int k_back = gates == 3 ? 48 * ((H + 15) / 16) : gates * H;
  const ForwardTile f = pick_forward_tile(gates, batch_size, H, 0, kWorkgroupLdsBytes, false, gates == 3 ? 3 : 2);
  const BackwardTile b = pick_backward_tile(k_back, batch_size, H, gates == 3 ? 6 * 16 : (size_t)gates * 16, 0, true);
  t_assumed_cus = 0;
  t_assumed_xcds = 0;
  const int out[16] = {f.ok, f.nb, f.hs, f.ct, f.gx, f.gy, f.reg_groups, (H + 63) / 64,
                       b.ok, b.nb, 16, 1, b.gx, b.gy, b.reg_groups, (k_back + 63) / 64};
  for (int i = 0; i < 16; ++i) plan[i] = (i % 8 == 0 || out[i - i % 8]) ? out[i] : 0;
  return HASTE_HIP_OK;
}

int haste_hip_stream_status(void* stream_) {
  hipStream_t stream = haste_hip::as_stream(stream_);
  int dev = 0;
  HASTE_HIP_TRY(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(haste_hip::g_mutex);
  auto it = haste_hip::g_workspaces.find(haste_hip::Key{dev, stream});
  if (it == haste_hip::g_workspaces.end() || it->second.host_status == nullptr) return HASTE_HIP_OK;
  volatile unsigned int* status = it->second.host_status;
  const unsigned int seen = *status;
  if (seen == 0u) return HASTE_HIP_OK;
  *status = 0u;
  return haste_hip::recover_from_abort_locked(dev, stream, it->second, seen);
}

int haste_hip_set_workspace(void* stream_, void* memory, size_t bytes) {
  using namespace haste_hip;
  hipStream_t stream = as_stream(stream_);
  int dev = 0;
  HASTE_HIP_TRY(hipGetDevice(&dev));
  if (memory != nullptr) {
    HASTE_HIP_REQUIRE((reinterpret_cast<uintptr_t>(memory) & 255u) == 0);
    HASTE_HIP_REQUIRE(bytes >= kControlBytes + 4096);
  }
  // The look at the XCD placement (once per device) happens here rather than inside the first
  // persistent launch, which may be recorded into a graph.
  (void)device_xcd_count();
  std::lock_guard<std::mutex> lock(g_mutex);
  Workspace& ws = g_workspaces[Key{dev, stream}];
  // Work enqueued earlier may still use what is replaced.
  if (ws.control != nullptr) HASTE_HIP_TRY(hipStreamSynchronize(stream));
  if (!ws.caller_owned) {
    if (ws.scratch) HASTE_HIP_TRY(hipFree(ws.scratch));
    ws.scratch = nullptr;
    if (ws.control) HASTE_HIP_TRY(hipFree(ws.control));
  }
  ws.control = nullptr;
  ws.scratch = nullptr;
  ws.scratch_bytes = 0;
  ws.caller_owned = false;
  ws.epoch = 0;
  ws.ticket_base = 0;
  if (memory == nullptr) return HASTE_HIP_OK;  // back to a workspace of the library's own
  HASTE_HIP_PROPAGATE(ensure_host_status(ws));
  HASTE_HIP_PROPAGATE(zero_control(stream, static_cast<ControlBlock*>(memory)));
  ws.control = static_cast<ControlBlock*>(memory);
  ws.scratch = reinterpret_cast<float*>(static_cast<char*>(memory) + kControlBytes);
  ws.scratch_bytes = bytes - kControlBytes;
  ws.caller_owned = true;
  return HASTE_HIP_OK;
}

int haste_hip_workspace_high_water(void* stream_, size_t* bytes) {
  using namespace haste_hip;
  HASTE_HIP_REQUIRE(bytes != nullptr);
  int dev = 0;
  HASTE_HIP_TRY(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(g_mutex);
  auto it = g_workspaces.find(Key{dev, as_stream(stream_)});
  *bytes = kControlBytes + 4096 + (it == g_workspaces.end() ? 0 : it->second.scratch_high_water);
  return HASTE_HIP_OK;
}

size_t haste_hip_workspace_bytes(int time_steps, int batch_size, int input_size, int hidden_size) {
  using namespace haste_hip;
  if (time_steps < 1 || batch_size < 1 || input_size < 1 || hidden_size < 1) return 0;
  const size_t T = (size_t)time_steps, N = (size_t)batch_size, C = (size_t)input_size, H = (size_t)hidden_size;
  const size_t cus = device_cu_count() > 0 ? (size_t)device_cu_count() : 256;
  const size_t widest = 4 * H > C ? 4 * H : C;  // longest row any kernel sums columns of
  size_t b = 0;
  // GEMM: K pieces of the tile kernel (at most 4 per CU, 64 KiB each), chunks of the
  // small-batch kernel (about three workgroups per CU with at most 32 x 128 outputs each,
  // plus one output's worth).
  b += 4 * cus * 128 * 128 * sizeof(float);
  b += (3 * cus + 8) * 64 * 128 * sizeof(float) + 128 * widest * sizeof(float);
  // Persistent recurrences: four exchange tiles (contraction at most 4H + 64, padded to 64;
  // batch tiles cover at most N + 63 rows), per-tile column sums (at most 64 tiles, two sets,
  // ten rows of H), the tagged row exchange of the layer-norm cells (two exchanges, two
  // buffers, 16 bytes per column workgroup and row).
  const size_t rows = N + 63, kpad = 4 * H + 128;
  b += 4 * kpad * rows * sizeof(float);
  b += 64 * 2 * 10 * (H + 4) * sizeof(float);
  b += 2 * 2 * 16 * (H / 4 + 2) * rows * 2 * sizeof(float);
  // Backward recurrences of 4-row tiles in scattered form (H <= 512): two tiles of pieces per
  // tile of 4 rows, [owners][up to 32 producers][64].
  if (H <= 512) b += (N / 4 + 2) * 2 * (H / 16 + 1) * 32 * 64 * sizeof(float);
  // Step-wise regime (any scalar type up to 8 bytes): the step's product [N, 4H], a scaled
  // copy of R, column sums in at most 128 chunks, row statistics of all steps, two [N, H]
  // buffers; the stand-alone layer norm's column sums (two workgroups per CU, two rows each).
  b += (N * 4 * H + H * 4 * H + 128 * widest + T * N * 2 + 2 * N * H) * 8 + 16 * 256;
  // ... and the K pieces of a double product of few tiles (at most one 64 x 64 piece per CU)
  b += cus * 64 * 64 * 8;
  b += 2 * cus * 2 * widest * sizeof(float);
  // Single forward steps: partial sums of at most 64 runs of the contraction, both sides, for 8
  // rows and every gate column, and the staged state.
  b += 64 * 2 * 8 * (H / 16 + 1) * 64 * sizeof(float) + 8 * H * sizeof(float) + 256;
  return kControlBytes + 4096 + (b + 255) / 256 * 256;
}

}  // extern "C"

namespace haste_hip {
size_t workspace_scratch_bound(int T, int N, int C, int H) {
  const size_t all = haste_hip_workspace_bytes(T, N, C, H);
  return all > kControlBytes ? all - kControlBytes : 0;
}
}  // namespace haste_hip

extern "C" {

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
      if (!it->second.caller_owned) {
        if (it->second.scratch) (void)hipFree(it->second.scratch);
        if (it->second.control) (void)hipFree(it->second.control);
      }
      if (it->second.host_status) (void)hipHostFree(it->second.host_status);
      it = haste_hip::g_workspaces.erase(it);
    } else {
      ++it;
    }
  }
  return HASTE_HIP_OK;
}

}  // extern "C"
