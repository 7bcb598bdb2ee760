// Shared device/host helpers for the gfx950 sparse-embedding kernels.
//
// Conventions used by every kernel in this directory:
//   * wavefront = 64 lanes; a workgroup is 256 threads (4 waves) unless noted
//   * a "team" is a power-of-two group of lanes (<= 64, so never spans waves)
//     that cooperates on one segment / one row; geometry is passed at run time
//     as log2 values so one instantiation serves every embedding width
//   * rows are moved with the widest vector the row width allows (16 B when
//     D * sizeof(T) is a multiple of 16 and the base pointer is 16-B aligned)
//   * all arithmetic on row elements is done in fp32 whatever the storage type
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/recis_hip.h"

namespace recis_hip {

constexpr int kWave = 64;
constexpr int kBlock = 256;

// ---------------------------------------------------------------- error state
void set_error(const char* fmt, ...);
int fail(int code, const char* fmt, ...);

#define RECIS_CHECK_HIP(expr)                                                  \
  do {                                                                         \
    hipError_t _e = (expr);                                                    \
    if (_e != hipSuccess)                                                      \
      return ::recis_hip::fail(RECIS_ERR_HIP, "%s failed: %s (%s:%d)", #expr,  \
                               hipGetErrorString(_e), __FILE__, __LINE__);     \
  } while (0)

#define RECIS_REQUIRE(cond, ...)                                               \
  do {                                                                         \
    if (!(cond)) return ::recis_hip::fail(RECIS_ERR_ARG, __VA_ARGS__);         \
  } while (0)

#define RECIS_LAUNCH_CHECK()                                                   \
  do {                                                                         \
    hipError_t _e = hipGetLastError();                                         \
    if (_e != hipSuccess)                                                      \
      return ::recis_hip::fail(RECIS_ERR_HIP, "kernel launch failed: %s (%s:%d)", \
                               hipGetErrorString(_e), __FILE__, __LINE__);     \
  } while (0)

// Device-side soft error word (one per device): kernels that meet an index
// outside the range the host promised skip the access and set a bit here
// instead of faulting the GPU. Read with recis_hip_poll_device_errors().
int* device_error_word(int device);
int current_device();

// --------------------------------------------------------------- storage types
struct bf16_t {
  uint16_t bits;
};
struct f16_t {
  _Float16 v;
};

__device__ __forceinline__ float to_float(float x) { return x; }
__device__ __forceinline__ float to_float(bf16_t x) {
  return __uint_as_float(static_cast<uint32_t>(x.bits) << 16);
}
__device__ __forceinline__ float to_float(f16_t x) { return static_cast<float>(x.v); }

template <typename T>
__device__ __forceinline__ T from_float(float x);
template <>
__device__ __forceinline__ float from_float<float>(float x) {
  return x;
}
template <>
__device__ __forceinline__ bf16_t from_float<bf16_t>(float x) {
  // round-to-nearest-even, NaN kept quiet (same rule as torch's c10::BFloat16)
  uint32_t u = __float_as_uint(x);
  bf16_t r;
  if ((u & 0x7fffffffu) > 0x7f800000u) {
    r.bits = 0x7fc0;
  } else {
    u += 0x7fffu + ((u >> 16) & 1u);
    r.bits = static_cast<uint16_t>(u >> 16);
  }
  return r;
}
template <>
__device__ __forceinline__ f16_t from_float<f16_t>(float x) {
  f16_t r;
  r.v = static_cast<_Float16>(x);
  return r;
}

// A pack of VEC elements moved with one memory instruction.
template <typename T, int VEC>
struct alignas(sizeof(T) * VEC) Pack {
  T v[VEC];
};

template <typename T, int VEC>
__device__ __forceinline__ void load_pack(const T* p, float (&out)[VEC]) {
  Pack<T, VEC> pk = *reinterpret_cast<const Pack<T, VEC>*>(p);
#pragma unroll
  for (int i = 0; i < VEC; ++i) out[i] = to_float(pk.v[i]);
}

template <typename T, int VEC>
__device__ __forceinline__ void store_pack(T* p, const float (&in)[VEC]) {
  Pack<T, VEC> pk;
#pragma unroll
  for (int i = 0; i < VEC; ++i) pk.v[i] = from_float<T>(in[i]);
  *reinterpret_cast<Pack<T, VEC>*>(p) = pk;
}

// streaming variants: data touched once, keep it from displacing reusable lines
template <typename T, int VEC>
__device__ __forceinline__ void load_pack_stream(const T* p, float (&out)[VEC]) {
  if constexpr (sizeof(T) * VEC == 16) {
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    u4 raw = __builtin_nontemporal_load(reinterpret_cast<const u4*>(p));
    Pack<T, VEC> pk;
    __builtin_memcpy(&pk, &raw, 16);
#pragma unroll
    for (int i = 0; i < VEC; ++i) out[i] = to_float(pk.v[i]);
  } else {
    load_pack<T, VEC>(p, out);
  }
}

template <typename T, int VEC>
__device__ __forceinline__ void store_pack_stream(T* p, const float (&in)[VEC]) {
  if constexpr (sizeof(T) * VEC == 16) {
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    Pack<T, VEC> pk;
#pragma unroll
    for (int i = 0; i < VEC; ++i) pk.v[i] = from_float<T>(in[i]);
    u4 raw;
    __builtin_memcpy(&raw, &pk, 16);
    __builtin_nontemporal_store(raw, reinterpret_cast<u4*>(p));
  } else {
    store_pack<T, VEC>(p, in);
  }
}

// int32 / int64 index arrays behind one pointer
__device__ __forceinline__ int64_t load_index(const void* p, int is64, int64_t i) {
  return is64 ? static_cast<const int64_t*>(p)[i]
              : static_cast<int64_t>(static_cast<const int32_t*>(p)[i]);
}

__device__ __forceinline__ void store_index(void* p, int is64, int64_t i, int64_t v) {
  if (is64)
    static_cast<int64_t*>(p)[i] = v;
  else
    static_cast<int32_t*>(p)[i] = static_cast<int32_t>(v);
}

__device__ __forceinline__ void raise_device_error(int* err_word, int bit) {
  atomicOr(err_word, bit);
}

// ---------------------------------------------------------------- row geometry
// How a row of D elements of `esize` bytes is split over lanes.
struct RowGeom {
  int vec;       // elements per lane access
  int lpr_log2;  // lanes per row (power of two, <= 64)
};

inline int ilog2_ceil(int64_t x) {
  int l = 0;
  while ((int64_t(1) << l) < x) ++l;
  return l;
}

// Largest power-of-two vector (in bytes, <= 16) dividing the row bytes and the
// alignment of every base pointer involved.
inline int pick_vec_bytes(int64_t row_bytes, uintptr_t align_or) {
  int vb = 16;
  while (vb > 1 && ((row_bytes % vb) != 0 || (align_or % vb) != 0)) vb >>= 1;
  return vb;
}

// The same with a caller-chosen upper limit (fp32 rows written by kernels whose inputs are
// 2-byte types go out as 32-byte packs, two 16-byte stores per lane).
inline int pick_vec_bytes_max(int64_t row_bytes, uintptr_t align_or, int max_bytes) {
  int vb = max_bytes;
  while (vb > 1 && ((row_bytes % vb) != 0 || (align_or % vb) != 0)) vb >>= 1;
  return vb;
}

inline RowGeom make_row_geom(int64_t D, int esize, int vec_bytes) {
  RowGeom g;
  g.vec = vec_bytes / esize;
  if (g.vec < 1) g.vec = 1;
  int64_t lanes = (D + g.vec - 1) / g.vec;
  g.lpr_log2 = ilog2_ceil(lanes);
  if (g.lpr_log2 > 6) g.lpr_log2 = 6;
  return g;
}

inline int dtype_size(int dtype) {
  switch (dtype) {
    case RECIS_F32: return 4;
    case RECIS_BF16: return 2;
    case RECIS_F16: return 2;
    default: return 0;
  }
}

// Optional per-kernel timing (off by default): when enabled through
// recis_hip_profile_enable(1), a KernelTimer brackets a launch with two HIP
// events on the launch stream; recis_hip_profile_report() sums them per kernel name.
extern bool g_profile_on;
struct KernelTimer {
  KernelTimer(const char* name, hipStream_t stream) : active_(g_profile_on) {
    if (active_) begin(name, stream);
  }
  ~KernelTimer() {
    if (active_) end();
  }
  // makes `for (KernelTimer t(...); t.once();) launch;` run the launch exactly once
  bool once() {
    const bool first = !done_;
    done_ = true;
    return first;
  }

 private:
  void begin(const char* name, hipStream_t stream);
  void end();
  bool active_;
  bool done_ = false;
  int slot_ = -1;
  hipStream_t stream_ = nullptr;
};
// usage: RECIS_TIME_KERNEL("name", stream) kernel<<<grid, block, 0, stream>>>(...);
#define RECIS_TIME_KERNEL(name, stream) for (::recis_hip::KernelTimer _recis_kt(name, stream); _recis_kt.once();)

// Per-(device, stream) scratch that grows on demand and is reused by later
// calls on that stream. Never shrinks; released at process exit.
int get_workspace(hipStream_t stream, size_t bytes, void** out);

// Per-(device, stream) pinned host words and an event, for handing a device-side count to the
// host while later kernels of the same call are still running.
int get_count_staging(hipStream_t stream, int64_t** host, hipEvent_t* event);

}  // namespace recis_hip
