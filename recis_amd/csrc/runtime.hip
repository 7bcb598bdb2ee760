// Host-side runtime shared by all entry points: thread-local error text, the
// per-device soft-error word, and per-(device, stream) scratch memory.
#include <stdarg.h>
#include <stdio.h>

#include <map>
#include <mutex>
#include <utility>

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
static std::map<int, int*> g_err_words;

int* device_error_word(int device) {
  std::lock_guard<std::mutex> l(g_mu);
  auto it = g_err_words.find(device);
  if (it != g_err_words.end()) return it->second;
  int* p = nullptr;
  if (hipMalloc(reinterpret_cast<void**>(&p), sizeof(int)) != hipSuccess) return nullptr;
  if (hipMemset(p, 0, sizeof(int)) != hipSuccess) return nullptr;
  g_err_words[device] = p;
  return p;
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

}  // namespace recis_hip

extern "C" {

const char* recis_hip_last_error(void) { return recis_hip::g_err; }

int recis_hip_abi_version(void) { return RECIS_HIP_ABI_VERSION; }

int recis_hip_poll_device_errors(int* bits) {
  using namespace recis_hip;
  RECIS_REQUIRE(bits != nullptr, "bits must not be NULL");
  int dev = current_device();
  int* w = device_error_word(dev);
  RECIS_REQUIRE(w != nullptr, "could not allocate the device error word");
  RECIS_CHECK_HIP(hipDeviceSynchronize());
  RECIS_CHECK_HIP(hipMemcpy(bits, w, sizeof(int), hipMemcpyDeviceToHost));
  if (*bits) RECIS_CHECK_HIP(hipMemset(w, 0, sizeof(int)));
  return RECIS_OK;
}

}  // extern "C"
