// Feature-engine scalar ops for gfx950: string hashes, unsigned mod, bucketize,
// multi-hash. Each call handles a whole list of tensors in one launch
// (grid.y = tensor), the per-tensor pointers and parameters riding in the kernel
// arguments.
//
// Stand in for: fused_hash (csrc/ops/fused_hash_kernel.cu:386-458),
// fused_uint64_mod / uint64_mod (csrc/ops/fused_uint64_mod_kernel.cu:12-39,
// uint64_mod_kernel.cu:5-24), fused_bucketized / bucketize_op
// (csrc/ops/fused_bucketized_kernel.cu:19-60, bucketize_op_kernel.cu:6-43),
// fused_multi_hash (csrc/ops/multi_hash_kernel.cu:11-74).
#include <hip/hip_runtime.h>

#include <algorithm>

#include "common.cuh"

namespace recis_hip {
namespace {

constexpr int kMaxJobs = 40;

struct Jobs {
  const void* in[kMaxJobs];
  const void* aux[kMaxJobs];  // offsets (hash) / boundaries (bucketize)
  void* out[kMaxJobs];
  int64_t size[kMaxJobs];
  int64_t p0[kMaxJobs];  // mod / boundary count / mul
  int64_t p1[kMaxJobs];  // prime
  int64_t p2[kMaxJobs];  // bucket
};

inline int64_t grid_x_for(int64_t max_size) {
  return std::max<int64_t>(1, std::min<int64_t>((max_size + kBlock - 1) / kBlock, 256 * 8));
}

// ------------------------------------------------------------------ hashes
__device__ __forceinline__ uint64_t rd64(const uint8_t* p) {
  uint64_t v;
  __builtin_memcpy(&v, p, 8);
  return v;
}
__device__ __forceinline__ uint32_t rd32(const uint8_t* p) {
  uint32_t v;
  __builtin_memcpy(&v, p, 4);
  return v;
}

// MurmurHash64A (Austin Appleby), seed given by the caller
__device__ uint64_t murmur64(const uint8_t* data, uint64_t n, uint64_t seed) {
  const uint64_t m = 0xc6a4a7935bd1e995ULL;
  uint64_t h = seed ^ (n * m);
  const uint64_t full = n >> 3;
  for (uint64_t i = 0; i < full; ++i) {
    uint64_t k = rd64(data + 8 * i) * m;
    k ^= k >> 47;
    h = (h ^ (k * m)) * m;
  }
  const uint8_t* tail = data + 8 * full;
  const uint32_t rem = static_cast<uint32_t>(n & 7);
  if (rem) {
    uint64_t t = 0;
    for (uint32_t i = 0; i < rem; ++i) t |= static_cast<uint64_t>(tail[i]) << (8 * i);
    h = (h ^ t) * m;
  }
  h ^= h >> 47;
  h *= m;
  h ^= h >> 47;
  return h;
}

// FarmHash (farmhashna) Hash64, Geoff Pike / Google
constexpr uint64_t FK0 = 0xc3a5c85c97cb3127ULL;
constexpr uint64_t FK1 = 0xb492b66fbe98f273ULL;
constexpr uint64_t FK2 = 0x9ae16a3b2f90404fULL;

__device__ __forceinline__ uint64_t rotr(uint64_t v, int s) { return (v >> s) | (v << ((64 - s) & 63)); }
__device__ __forceinline__ uint64_t smix(uint64_t v) { return v ^ (v >> 47); }
__device__ __forceinline__ uint64_t hlen16(uint64_t u, uint64_t v, uint64_t mul) {
  uint64_t a = (u ^ v) * mul;
  a ^= a >> 47;
  uint64_t b = (v ^ a) * mul;
  b ^= b >> 47;
  return b * mul;
}
struct U128 {
  uint64_t lo, hi;
};
__device__ __forceinline__ U128 weak32(const uint8_t* s, uint64_t a, uint64_t b) {
  const uint64_t w = rd64(s), x = rd64(s + 8), y = rd64(s + 16), z = rd64(s + 24);
  a += w;
  b = rotr(b + a + z, 21);
  const uint64_t c = a;
  a += x + y;
  b += rotr(a, 44);
  return U128{a + z, b + c};
}

__device__ uint64_t farmhash64(const uint8_t* s, uint64_t len) {
  if (len <= 16) {
    if (len >= 8) {
      const uint64_t mul = FK2 + len * 2, a = rd64(s) + FK2, b = rd64(s + len - 8);
      return hlen16(rotr(b, 37) * mul + a, (rotr(a, 25) + b) * mul, mul);
    }
    if (len >= 4) {
      const uint64_t mul = FK2 + len * 2, a = rd32(s);
      return hlen16(len + (a << 3), rd32(s + len - 4), mul);
    }
    if (len > 0) {
      const uint32_t y = static_cast<uint32_t>(s[0]) + (static_cast<uint32_t>(s[len >> 1]) << 8);
      const uint32_t z = static_cast<uint32_t>(len) + (static_cast<uint32_t>(s[len - 1]) << 2);
      return smix(y * FK2 ^ z * FK0) * FK2;
    }
    return FK2;
  }
  if (len <= 32) {
    const uint64_t mul = FK2 + len * 2;
    const uint64_t a = rd64(s) * FK1, b = rd64(s + 8);
    const uint64_t c = rd64(s + len - 8) * mul, d = rd64(s + len - 16) * FK2;
    return hlen16(rotr(a + b, 43) + rotr(c, 30) + d, a + rotr(b + FK2, 18) + c, mul);
  }
  if (len <= 64) {
    const uint64_t mul = FK2 + len * 2;
    const uint64_t a = rd64(s) * FK2, b = rd64(s + 8);
    const uint64_t c = rd64(s + len - 8) * mul, d = rd64(s + len - 16) * FK2;
    const uint64_t y = rotr(a + b, 43) + rotr(c, 30) + d;
    const uint64_t z = hlen16(y, a + rotr(b + FK2, 18) + c, mul);
    const uint64_t e = rd64(s + 16) * mul, f = rd64(s + 24);
    const uint64_t g = (y + rd64(s + len - 32)) * mul, h = (z + rd64(s + len - 24)) * mul;
    return hlen16(rotr(e + f, 43) + rotr(g, 30) + h, e + rotr(f + a, 18) + g, mul);
  }
  const uint64_t seed = 81;
  uint64_t x = seed, y = seed * FK1 + 113, z = smix(y * FK2 + 113) * FK2;
  U128 v{0, 0}, w{0, 0};
  x = x * FK2 + rd64(s);
  const uint8_t* end = s + ((len - 1) / 64) * 64;
  const uint8_t* last64 = end + ((len - 1) & 63) - 63;
  do {
    x = rotr(x + y + v.lo + rd64(s + 8), 37) * FK1;
    y = rotr(y + v.hi + rd64(s + 48), 42) * FK1;
    x ^= w.hi;
    y += v.lo + rd64(s + 40);
    z = rotr(z + w.lo, 33) * FK1;
    v = weak32(s, v.hi * FK1, x + w.lo);
    w = weak32(s + 32, z + w.hi, y + rd64(s + 16));
    const uint64_t t = z;
    z = x;
    x = t;
    s += 64;
  } while (s != end);
  const uint64_t mul = FK1 + ((z & 0xff) << 1);
  s = last64;
  w.lo += (len - 1) & 63;
  v.lo += w.lo;
  w.lo += v.lo;
  x = rotr(x + y + v.lo + rd64(s + 8), 37) * mul;
  y = rotr(y + v.hi + rd64(s + 48), 42) * mul;
  x ^= w.hi * 9;
  y += v.lo * 9 + rd64(s + 40);
  z = rotr(z + w.lo, 33) * mul;
  v = weak32(s, v.hi * mul, x + w.lo);
  w = weak32(s + 32, z + w.hi, y + rd64(s + 16));
  const uint64_t t = z;
  z = x;
  x = t;
  return hlen16(hlen16(v.lo, w.lo, mul) + smix(y) * FK0 + z, hlen16(v.hi, w.hi, mul) + x, mul);
}

__global__ void __launch_bounds__(kBlock) hash_kernel(Jobs j, int off64, int kind, int* err) {
  const int t = blockIdx.y;
  const int64_t n = j.size[t];
  const uint8_t* bytes = static_cast<const uint8_t*>(j.in[t]);
  const int64_t total_bytes = j.p0[t];
  int64_t* out = static_cast<int64_t*>(j.out[t]);
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; i < n; i += stride) {
    const int64_t lo = load_index(j.aux[t], off64, i), hi = load_index(j.aux[t], off64, i + 1);
    if (lo < 0 || hi < lo || hi > total_bytes) {
      raise_device_error(err, RECIS_DEVERR_OFFSETS);
      out[i] = 0;
      continue;
    }
    const uint64_t len = static_cast<uint64_t>(hi - lo);
    out[i] = static_cast<int64_t>(kind == 0 ? farmhash64(bytes + lo, len) : murmur64(bytes + lo, len, 0));
  }
}

// ---------------------------------------------------------------- scalar ops
__global__ void __launch_bounds__(kBlock) uint64_mod_kernel(Jobs j) {
  const int t = blockIdx.y;
  const int64_t n = j.size[t];
  const int64_t* in = static_cast<const int64_t*>(j.in[t]);
  int64_t* out = static_cast<int64_t*>(j.out[t]);
  const uint64_t m = static_cast<uint64_t>(j.p0[t]);
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
  if (m >> 32) {
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; i < n; i += stride)
      out[i] = static_cast<int64_t>(static_cast<uint64_t>(in[i]) % m);
  } else {
    // 64-by-32 remainder in two 32-bit steps: (hi mod m) * 2^32 + lo fits 64 bits
    const uint32_t m32 = static_cast<uint32_t>(m);
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; i < n; i += stride) {
      const uint64_t x = static_cast<uint64_t>(in[i]);
      const uint32_t hi = static_cast<uint32_t>(x >> 32) % m32;
      const uint64_t rest = (static_cast<uint64_t>(hi) << 32) | (x & 0xffffffffu);
      out[i] = static_cast<int64_t>(rest % m32);
    }
  }
}

constexpr int kLdsBoundaries = 8192;

// upper bound: number of boundaries <= v, NaN -> len (fused_bucketized.cc:5-20); with a modulus
// (p1 != 0) the bucket is reduced at once, as a following fused_uint64_mod would
__global__ void __launch_bounds__(kBlock) bucketize_kernel(Jobs j) {
  __shared__ float s_b[kLdsBoundaries];
  const int t = blockIdx.y;
  const int64_t n = j.size[t];
  const float* in = static_cast<const float*>(j.in[t]);
  const float* bnd = static_cast<const float*>(j.aux[t]);
  int64_t* out = static_cast<int64_t*>(j.out[t]);
  const int32_t blen = static_cast<int32_t>(j.p0[t]);
  const uint32_t mod = static_cast<uint32_t>(j.p1[t]);  // buckets are below 2^31: a 32-bit remainder will do
  const bool in_lds = blen <= kLdsBoundaries;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
  const int64_t i_first = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  const float v_first = i_first < n ? in[i_first] : 0.f;  // on its way while the boundaries are staged
  if (in_lds) {
    for (int k = threadIdx.x; k < blen; k += kBlock) s_b[k] = bnd[k];
    __syncthreads();
  }
  const float* b = in_lds ? s_b : bnd;
  for (int64_t i = i_first; i < n; i += stride) {
    const float v = i == i_first ? v_first : in[i];
    int32_t bucket = 0, count = blen;
    while (count > 0) {
      const int32_t step = count >> 1;
      const int32_t mid = bucket + step;
      if (!(v < b[mid])) {
        bucket = mid + 1;
        count -= step + 1;
      } else {
        count = step;
      }
    }
    out[i] = mod ? static_cast<int64_t>(static_cast<uint32_t>(bucket) % mod) : bucket;
  }
}

// (((x * mul) % p + p) % p) % bucket in wrapping signed 64-bit (multi_hash.cc:18-26)
__global__ void __launch_bounds__(kBlock) multi_hash_kernel(Jobs j) {
  const int t = blockIdx.y;
  const int64_t n = j.size[t];
  const int64_t* in = static_cast<const int64_t*>(j.in[t]);
  int64_t* out = static_cast<int64_t*>(j.out[t]);
  const int64_t mul = j.p0[t], prime = j.p1[t], bucket = j.p2[t];
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; i < n; i += stride) {
    const int64_t x = static_cast<int64_t>(static_cast<uint64_t>(in[i]) * static_cast<uint64_t>(mul));
    out[i] = (((x % prime) + prime) % prime) % bucket;
  }
}

}  // namespace
}  // namespace recis_hip

using namespace recis_hip;

extern "C" {

int recis_fused_hash(const int8_t* const* values_ptrs, const int64_t* values_sizes,
                     const void* const* offsets_ptrs, int off_is64, const int64_t* n_strings,
                     int64_t* const* out_ptrs, int64_t n_tensors, int kind, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(n_tensors >= 0, "n_tensors must be >= 0");
  RECIS_REQUIRE(kind == 0 || kind == 1, "Unsupported hash type: %d (0 = farm, 1 = murmur)", kind);
  if (n_tensors == 0) return RECIS_OK;
  RECIS_REQUIRE(values_ptrs && values_sizes && offsets_ptrs && n_strings && out_ptrs, "NULL argument");
  int* err = device_error_word(current_device());
  RECIS_REQUIRE(err != nullptr, "could not reach the device error word");
  for (int64_t base = 0; base < n_tensors; base += kMaxJobs) {
    Jobs j;
    const int cnt = static_cast<int>(std::min<int64_t>(kMaxJobs, n_tensors - base));
    int64_t max_size = 0;
    for (int k = 0; k < cnt; ++k) {
      const int64_t t = base + k;
      RECIS_REQUIRE(n_strings[t] >= 0 && values_sizes[t] >= 0, "negative size");
      RECIS_REQUIRE(n_strings[t] == 0 || (offsets_ptrs[t] && out_ptrs[t]), "NULL tensor pointer");
      RECIS_REQUIRE(values_sizes[t] == 0 || values_ptrs[t], "NULL values pointer");
      j.in[k] = values_ptrs[t];
      j.aux[k] = offsets_ptrs[t];
      j.out[k] = out_ptrs[t];
      j.size[k] = n_strings[t];
      j.p0[k] = values_sizes[t];
      j.p1[k] = j.p2[k] = 0;
      max_size = std::max(max_size, n_strings[t]);
    }
    if (max_size == 0) continue;
    hash_kernel<<<dim3(grid_x_for(max_size), cnt), dim3(kBlock), 0, stream>>>(j, off_is64, kind, err);
    RECIS_LAUNCH_CHECK();
  }
  return RECIS_OK;
}

int recis_fused_uint64_mod(const int64_t* const* in_ptrs, const int64_t* sizes, const int64_t* mods,
                           int64_t* const* out_ptrs, int64_t n_tensors, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(n_tensors >= 0, "n_tensors must be >= 0");
  if (n_tensors == 0) return RECIS_OK;
  RECIS_REQUIRE(in_ptrs && sizes && mods && out_ptrs, "NULL argument");
  for (int64_t base = 0; base < n_tensors; base += kMaxJobs) {
    Jobs j;
    const int cnt = static_cast<int>(std::min<int64_t>(kMaxJobs, n_tensors - base));
    int64_t max_size = 0;
    for (int k = 0; k < cnt; ++k) {
      const int64_t t = base + k;
      RECIS_REQUIRE(sizes[t] >= 0, "negative size");
      RECIS_REQUIRE(mods[t] != 0, "mod by zero (tensor %lld)", (long long)t);
      RECIS_REQUIRE(sizes[t] == 0 || (in_ptrs[t] && out_ptrs[t]), "NULL tensor pointer");
      j.in[k] = in_ptrs[t];
      j.aux[k] = nullptr;
      j.out[k] = out_ptrs[t];
      j.size[k] = sizes[t];
      j.p0[k] = mods[t];
      j.p1[k] = j.p2[k] = 0;
      max_size = std::max(max_size, sizes[t]);
    }
    if (max_size == 0) continue;
    uint64_mod_kernel<<<dim3(grid_x_for(max_size), cnt), dim3(kBlock), 0, stream>>>(j);
    RECIS_LAUNCH_CHECK();
  }
  return RECIS_OK;
}

int recis_fused_bucketized(const float* const* in_ptrs, const int64_t* sizes,
                           const float* const* boundaries_ptrs, const int64_t* boundary_lens,
                           int64_t* const* out_ptrs, int64_t n_tensors, void* stream_) {
  return recis_fused_bucketized_mod(in_ptrs, sizes, boundaries_ptrs, boundary_lens, nullptr, out_ptrs, n_tensors,
                                    stream_);
}

int recis_fused_bucketized_mod(const float* const* in_ptrs, const int64_t* sizes,
                               const float* const* boundaries_ptrs, const int64_t* boundary_lens,
                               const int64_t* mods, int64_t* const* out_ptrs, int64_t n_tensors, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(n_tensors >= 0, "n_tensors must be >= 0");
  if (n_tensors == 0) return RECIS_OK;
  RECIS_REQUIRE(in_ptrs && sizes && boundaries_ptrs && boundary_lens && out_ptrs, "NULL argument");
  for (int64_t base = 0; base < n_tensors; base += kMaxJobs) {
    Jobs j;
    const int cnt = static_cast<int>(std::min<int64_t>(kMaxJobs, n_tensors - base));
    int64_t max_size = 0;
    for (int k = 0; k < cnt; ++k) {
      const int64_t t = base + k;
      RECIS_REQUIRE(sizes[t] >= 0 && boundary_lens[t] >= 0 && boundary_lens[t] < (int64_t(1) << 31),
                    "bad size");
      RECIS_REQUIRE(sizes[t] == 0 || (in_ptrs[t] && out_ptrs[t]), "NULL tensor pointer");
      RECIS_REQUIRE(boundary_lens[t] == 0 || boundaries_ptrs[t], "NULL boundaries pointer");
      j.in[k] = in_ptrs[t];
      j.aux[k] = boundaries_ptrs[t];
      j.out[k] = out_ptrs[t];
      j.size[k] = sizes[t];
      j.p0[k] = boundary_lens[t];
      j.p1[k] = j.p2[k] = 0;
      if (mods) {
        // a bucket is at most the number of boundaries: a modulus past 32 bits changes nothing
        RECIS_REQUIRE(mods[t] > 0, "mod must be positive (tensor %lld)", (long long)t);
        j.p1[k] = mods[t] > boundary_lens[t] ? 0 : mods[t];
      }
      max_size = std::max(max_size, sizes[t]);
    }
    if (max_size == 0) continue;
    bucketize_kernel<<<dim3(grid_x_for(max_size), cnt), dim3(kBlock), 0, stream>>>(j);
    RECIS_LAUNCH_CHECK();
  }
  return RECIS_OK;
}

int recis_fused_multi_hash(const int64_t* const* in_ptrs, const int64_t* sizes, const int64_t* muls,
                           const int64_t* primes, const int64_t* buckets, int64_t* const* out_ptrs,
                           int64_t n_jobs, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(n_jobs >= 0, "n_jobs must be >= 0");
  if (n_jobs == 0) return RECIS_OK;
  RECIS_REQUIRE(in_ptrs && sizes && muls && primes && buckets && out_ptrs, "NULL argument");
  for (int64_t base = 0; base < n_jobs; base += kMaxJobs) {
    Jobs j;
    const int cnt = static_cast<int>(std::min<int64_t>(kMaxJobs, n_jobs - base));
    int64_t max_size = 0;
    for (int k = 0; k < cnt; ++k) {
      const int64_t t = base + k;
      RECIS_REQUIRE(sizes[t] >= 0, "negative size");
      RECIS_REQUIRE(primes[t] != 0 && buckets[t] != 0, "zero prime or bucket (job %lld)", (long long)t);
      RECIS_REQUIRE(sizes[t] == 0 || (in_ptrs[t] && out_ptrs[t]), "NULL tensor pointer");
      j.in[k] = in_ptrs[t];
      j.aux[k] = nullptr;
      j.out[k] = out_ptrs[t];
      j.size[k] = sizes[t];
      j.p0[k] = muls[t];
      j.p1[k] = primes[t];
      j.p2[k] = buckets[t];
      max_size = std::max(max_size, sizes[t]);
    }
    if (max_size == 0) continue;
    multi_hash_kernel<<<dim3(grid_x_for(max_size), cnt), dim3(kBlock), 0, stream>>>(j);
    RECIS_LAUNCH_CHECK();
  }
  return RECIS_OK;
}

}  // extern "C"
