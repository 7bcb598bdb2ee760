// Host-side runtime shared by all entry points: thread-local error text, the
// per-device soft-error word, and per-(device, stream) scratch memory.
#include <stdarg.h>
#include <stdio.h>

#include <map>
#include <mutex>
#include <string>
#include <utility>
#include <vector>

#include "common.cuh"

namespace recis_hip {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int current_device() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return -1;
  return dev;
}

static std::mutex g_mu;

// The soft-error word lives in the code object of this library (one copy per device that loads
// it), so reaching it never allocates: entry points that must not allocate can use it too.
static __device__ int g_error_word[4];
constexpr int kMaxDevices = 64;
static int* g_err_words[kMaxDevices];

int* device_error_word(int device) {
  if (device < 0 || device >= kMaxDevices) return nullptr;
  std::lock_guard<std::mutex> l(g_mu);
  if (g_err_words[device]) return g_err_words[device];
  int cur = -1;
  if (hipGetDevice(&cur) != hipSuccess) return nullptr;
  if (cur != device && hipSetDevice(device) != hipSuccess) return nullptr;
  void* p = nullptr;
  const hipError_t rc = hipGetSymbolAddress(&p, HIP_SYMBOL(g_error_word));
  if (cur != device) (void)hipSetDevice(cur);
  if (rc != hipSuccess) return nullptr;
  g_err_words[device] = static_cast<int*>(p);
  return g_err_words[device];
}

struct Workspace {
  void* ptr = nullptr;
  size_t bytes = 0;
};
static std::map<std::pair<int, hipStream_t>, Workspace> g_ws;

int get_workspace(hipStream_t stream, size_t bytes, void** out) {
  int dev = current_device();
  std::lock_guard<std::mutex> l(g_mu);
  Workspace& w = g_ws[std::make_pair(dev, stream)];
  if (w.bytes < bytes) {
    // Work already queued on this stream may still read the old buffer:
    // drain the stream before the buffer is replaced.
    if (w.ptr) {
      RECIS_CHECK_HIP(hipStreamSynchronize(stream));
      RECIS_CHECK_HIP(hipFree(w.ptr));
      w.ptr = nullptr;
      w.bytes = 0;
    }
    size_t want = bytes < (size_t(1) << 20) ? (size_t(1) << 20) : bytes + bytes / 4;
    want = (want + 255) & ~size_t(255);
    RECIS_CHECK_HIP(hipMalloc(&w.ptr, want));
    w.bytes = want;
  }
  *out = w.ptr;
  return RECIS_OK;
}

struct CountStaging {
  int64_t* host = nullptr;  // pinned
  hipEvent_t event = nullptr;
};
static std::map<std::pair<int, hipStream_t>, CountStaging> g_staging;

int get_count_staging(hipStream_t stream, int64_t** host, hipEvent_t* event) {
  int dev = current_device();
  std::lock_guard<std::mutex> l(g_mu);
  CountStaging& c = g_staging[std::make_pair(dev, stream)];
  if (c.host == nullptr) {
    RECIS_CHECK_HIP(hipHostMalloc(reinterpret_cast<void**>(&c.host), 64, hipHostMallocDefault));
    for (int w = 0; w < 8; ++w) c.host[w] = 0;
    RECIS_CHECK_HIP(hipEventCreateWithFlags(&c.event, hipEventDisableTiming));
  }
  *host = c.host;
  *event = c.event;
  return RECIS_OK;
}

bool g_profile_on = false;

struct TimedLaunch {
  const char* name;
  hipEvent_t start, stop;
};
static std::vector<TimedLaunch> g_timed;

void KernelTimer::begin(const char* name, hipStream_t stream) {
  std::lock_guard<std::mutex> l(g_mu);
  TimedLaunch t;
  t.name = name;
  if (hipEventCreate(&t.start) != hipSuccess || hipEventCreate(&t.stop) != hipSuccess) {
    active_ = false;
    return;
  }
  (void)hipEventRecord(t.start, stream);
  g_timed.push_back(t);
  slot_ = static_cast<int>(g_timed.size()) - 1;
  stream_ = stream;
}

void KernelTimer::end() {
  std::lock_guard<std::mutex> l(g_mu);
  if (slot_ >= 0 && slot_ < static_cast<int>(g_timed.size())) (void)hipEventRecord(g_timed[slot_].stop, stream_);
}

}  // namespace recis_hip

extern "C" {

int recis_hip_profile_enable(int on) {
  std::lock_guard<std::mutex> l(recis_hip::g_mu);
  recis_hip::g_profile_on = on != 0;
  return RECIS_OK;
}

int recis_hip_profile_report(char* buf, int64_t cap) {
  using namespace recis_hip;
  RECIS_REQUIRE(buf != nullptr && cap > 0, "buf must hold the report");
  RECIS_CHECK_HIP(hipDeviceSynchronize());
  std::lock_guard<std::mutex> l(g_mu);
  std::map<std::string, std::pair<int64_t, double>> agg;
  for (auto& t : g_timed) {
    float ms = 0.f;
    if (hipEventElapsedTime(&ms, t.start, t.stop) == hipSuccess) {
      auto& a = agg[t.name];
      a.first += 1;
      a.second += ms;
    }
    (void)hipEventDestroy(t.start);
    (void)hipEventDestroy(t.stop);
  }
  g_timed.clear();
  std::string out;
  char line[256];
  for (auto& kv : agg) {
    snprintf(line, sizeof(line), "%s %lld %.6f\n", kv.first.c_str(), (long long)kv.second.first, kv.second.second);
    out += line;
  }
  snprintf(buf, static_cast<size_t>(cap), "%s", out.c_str());
  return RECIS_OK;
}

const char* recis_hip_last_error(void) { return recis_hip::g_err; }

int recis_hip_abi_version(void) { return RECIS_HIP_ABI_VERSION; }

int recis_hip_poll_device_errors(int* bits) {
  using namespace recis_hip;
  RECIS_REQUIRE(bits != nullptr, "bits must not be NULL");
  int dev = current_device();
  int* w = device_error_word(dev);
  RECIS_REQUIRE(w != nullptr, "could not reach the device error word");
  RECIS_CHECK_HIP(hipDeviceSynchronize());
  RECIS_CHECK_HIP(hipMemcpy(bits, w, sizeof(int), hipMemcpyDeviceToHost));
  if (*bits) RECIS_CHECK_HIP(hipMemset(w, 0, sizeof(int)));
  return RECIS_OK;
}

}  // extern "C"
