// ID tagging, offset merging and dedup (unique + inverse) for gfx950.
//
// ids_encode / merge_offsets stand in for csrc/ops/ids_encode_kernel.cu:16-59 and
// csrc/ops/embedding_segment_reduce_kernel.cu:357-391. The pointer/size tables
// of the fused multi-tensor launches travel as kernel arguments (no pinned
// staging buffer, no host-to-device copy, no stream synchronisation, unlike
// cuda/cuda_param.cuh:14-90 and cuda/element_wise_kernel.cuh:70-92).
//
// unique stands in for the dedup half of ids_partition
// (csrc/ops/ids_partition_kernel.cu:86-131: rotate, radix sort, flag, scan,
// scatter) and for the second torch.unique in HashTable.forward. It is hash
// based instead of sort based: one pass claims a slot per distinct id in a
// scratch open-addressing set and records the smallest occurrence position,
// a scan ranks the first occurrences, and a last pass writes the inverse. The
// unique ids come out in order of first occurrence (deterministic), not sorted.
#include <hip/hip_runtime.h>

#include <algorithm>

#include "common.cuh"

namespace recis_hip {
namespace {

constexpr int kMaxJobs = 48;

struct Jobs {
  const void* in[kMaxJobs];
  void* out[kMaxJobs];
  int64_t size[kMaxJobs];
  int64_t param[kMaxJobs];
};

__global__ void __launch_bounds__(kBlock) ids_encode_kernel(Jobs j) {
  const int t = blockIdx.y;
  const int64_t n = j.size[t];
  const int64_t* in = static_cast<const int64_t*>(j.in[t]);
  int64_t* out = static_cast<int64_t*>(j.out[t]);
  const int64_t tag = static_cast<int64_t>(static_cast<uint64_t>(j.param[t]) << 52);
  const int64_t mask = (int64_t(1) << 52) - 1;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; i < n; i += stride)
    out[i] = (in[i] & mask) | tag;
}

template <typename T>
__global__ void __launch_bounds__(kBlock) add_const_kernel(Jobs j) {
  const int t = blockIdx.y;
  const int64_t n = j.size[t];
  const T* in = static_cast<const T*>(j.in[t]);
  T* out = static_cast<T*>(j.out[t]);
  const T add = static_cast<T>(j.param[t]);
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; i < n; i += stride)
    out[i] = in[i] + add;
}

inline int64_t grid_x_for(int64_t max_size) {
  return std::max<int64_t>(1, std::min<int64_t>((max_size + kBlock - 1) / kBlock, 256 * 8));
}

// ------------------------------------------------------------------- unique
constexpr int64_t kSetEmpty = -1;
constexpr int32_t kNoPos = 0x7fffffff;

__device__ __forceinline__ uint64_t mix_id(int64_t key) {
  uint64_t x = static_cast<uint64_t>(key);
  x ^= x >> 33;
  x *= 0xff51afd7ed558ccdULL;
  x ^= x >> 33;
  x *= 0xc4ceb9fe1a85ec53ULL;
  x ^= x >> 33;
  return x;
}

__global__ void __launch_bounds__(kBlock)
set_init_kernel(int64_t* keys, int32_t* minpos, int64_t slots) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; i < slots; i += stride) {
    keys[i] = kSetEmpty;
    minpos[i] = kNoPos;
  }
}

// slot `cap` (one past the probed range) is reserved for the id that equals the
// empty marker, so every int64 value is a legal id
__global__ void __launch_bounds__(kBlock)
set_insert_kernel(int64_t* __restrict__ keys, int32_t* __restrict__ minpos, uint64_t mask,
                  const int64_t* __restrict__ ids, int64_t n, int32_t* __restrict__ slotpos) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (i >= n) return;
  const int64_t key = ids[i];
  uint64_t p;
  if (key == kSetEmpty) {
    p = mask + 1;
  } else {
    p = mix_id(key) & mask;
    for (;;) {
      // plain (L1-cacheable) load on purpose: thousands of duplicates of a hot id would
      // otherwise queue up at one L2 channel. A stale "empty" is harmless, the CAS below
      // then returns the real occupant; a slot never changes once it holds a key.
      int64_t k = keys[p];
      if (k == kSetEmpty) {
        k = static_cast<int64_t>(atomicCAS(reinterpret_cast<unsigned long long*>(&keys[p]),
                                           static_cast<unsigned long long>(kSetEmpty),
                                           static_cast<unsigned long long>(key)));
        if (k == kSetEmpty) break;
      }
      if (k == key) break;
      p = (p + 1) & mask;  // capacity >= 2n: an empty slot always exists
    }
  }
  // duplicates of a hot id arrive by the thousand: only those that can still lower the
  // minimum pay for the atomic (the stored value only ever decreases)
  if (minpos[p] > static_cast<int32_t>(i))  // plain load: a stale (larger) value only costs an atomic
    atomicMin(&minpos[p], static_cast<int32_t>(i));
  slotpos[i] = static_cast<int32_t>(p);
}

__device__ __forceinline__ void block_rank2(bool flag, int& rank, int& total) {
  __shared__ int wave_counts[kBlock / kWave];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const uint64_t ballot = __ballot(flag);
  const int prior = __popcll(ballot & ((uint64_t(1) << lane) - 1));
  if (lane == 0) wave_counts[wave] = __popcll(ballot);
  __syncthreads();
  int base = 0, tot = 0;
#pragma unroll
  for (int w = 0; w < kBlock / kWave; ++w) {
    if (w < wave) base += wave_counts[w];
    tot += wave_counts[w];
  }
  __syncthreads();
  rank = base + prior;
  total = tot;
}

__global__ void __launch_bounds__(kBlock)
first_count_kernel(const int32_t* __restrict__ minpos, const int32_t* __restrict__ slotpos, int64_t n,
                   int32_t* __restrict__ block_counts) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  const bool first = i < n && minpos[slotpos[i]] == static_cast<int32_t>(i);
  int rank, total;
  block_rank2(first, rank, total);
  if (threadIdx.x == 0) block_counts[blockIdx.x] = total;
}

__global__ void __launch_bounds__(1024)
scan_counts_kernel(int32_t* __restrict__ block_counts, int64_t nb, int64_t* __restrict__ total_out) {
  __shared__ int64_t partial[1024];
  const int t = threadIdx.x;
  const int64_t per = (nb + 1023) / 1024;
  const int64_t lo = std::min<int64_t>(t * per, nb), hi = std::min<int64_t>(lo + per, nb);
  int64_t sum = 0;
  for (int64_t b = lo; b < hi; ++b) sum += block_counts[b];
  partial[t] = sum;
  __syncthreads();
  for (int off = 1; off < 1024; off <<= 1) {
    int64_t add = t >= off ? partial[t - off] : 0;
    __syncthreads();
    partial[t] += add;
    __syncthreads();
  }
  int64_t run = t ? partial[t - 1] : 0;
  for (int64_t b = lo; b < hi; ++b) {
    int32_t c = block_counts[b];
    block_counts[b] = static_cast<int32_t>(run);
    run += c;
  }
  if (t == 1023) total_out[0] = partial[1023];
}

__global__ void __launch_bounds__(kBlock)
emit_unique_kernel(const int64_t* __restrict__ ids, const int32_t* __restrict__ minpos,
                   const int32_t* __restrict__ slotpos, int64_t n, const int32_t* __restrict__ block_prefix,
                   int64_t* __restrict__ unique_out, int32_t* __restrict__ uid) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  const int32_t sp = i < n ? slotpos[i] : 0;
  const bool first = i < n && minpos[sp] == static_cast<int32_t>(i);
  int rank, total;
  block_rank2(first, rank, total);
  if (!first) return;
  const int32_t u = block_prefix[blockIdx.x] + rank;
  unique_out[u] = ids[i];
  uid[sp] = u;
}

__global__ void __launch_bounds__(kBlock)
emit_inverse_kernel(const int32_t* __restrict__ slotpos, const int32_t* __restrict__ uid, int64_t n,
                    void* __restrict__ inverse, int inv64) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (i >= n) return;
  store_index(inverse, inv64, i, uid[slotpos[i]]);
}

}  // namespace
}  // namespace recis_hip

using namespace recis_hip;

extern "C" {

int recis_ids_encode(const int64_t* const* ids_ptrs, const int64_t* sizes, const int64_t* table_ids,
                     int64_t n_tensors, int64_t* out, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(n_tensors >= 0, "n_tensors must be >= 0");
  if (n_tensors == 0) return RECIS_OK;
  RECIS_REQUIRE(ids_ptrs && sizes && table_ids, "NULL argument");
  int64_t pos = 0;
  for (int64_t base = 0; base < n_tensors; base += kMaxJobs) {
    Jobs j;
    const int cnt = static_cast<int>(std::min<int64_t>(kMaxJobs, n_tensors - base));
    int64_t max_size = 0;
    for (int k = 0; k < cnt; ++k) {
      RECIS_REQUIRE(sizes[base + k] >= 0, "negative tensor size");
      RECIS_REQUIRE(table_ids[base + k] >= 0 && table_ids[base + k] < 4096, "table id %lld out of 12 bits",
                    (long long)table_ids[base + k]);
      RECIS_REQUIRE(sizes[base + k] == 0 || (ids_ptrs[base + k] && out), "NULL tensor pointer");
      j.in[k] = ids_ptrs[base + k];
      j.out[k] = out + pos;
      j.size[k] = sizes[base + k];
      j.param[k] = table_ids[base + k];
      pos += sizes[base + k];
      max_size = std::max(max_size, sizes[base + k]);
    }
    if (max_size == 0) continue;
    ids_encode_kernel<<<dim3(grid_x_for(max_size), cnt), dim3(kBlock), 0, stream>>>(j);
    RECIS_LAUNCH_CHECK();
  }
  return RECIS_OK;
}

int recis_merge_offsets(const void* const* offsets_ptrs, const int64_t* sizes, const int64_t* max_values,
                        int64_t n_tensors, int is64, void* out, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(n_tensors >= 0, "n_tensors must be >= 0");
  if (n_tensors == 0) return RECIS_OK;
  RECIS_REQUIRE(offsets_ptrs && sizes && max_values && out, "NULL argument");
  const int esz = is64 ? 8 : 4;
  int64_t pos = 0, prefix = 0;
  for (int64_t base = 0; base < n_tensors; base += kMaxJobs) {
    Jobs j;
    const int cnt = static_cast<int>(std::min<int64_t>(kMaxJobs, n_tensors - base));
    int64_t max_size = 0;
    for (int k = 0; k < cnt; ++k) {
      const int64_t t = base + k;
      RECIS_REQUIRE(sizes[t] >= 1 && offsets_ptrs[t], "every offsets tensor needs at least one entry");
      const int64_t take = (t < n_tensors - 1) ? sizes[t] - 1 : sizes[t];
      j.in[k] = offsets_ptrs[t];
      j.out[k] = static_cast<char*>(out) + pos * esz;
      j.size[k] = take;
      j.param[k] = prefix;
      pos += take;
      prefix += max_values[t];
      max_size = std::max(max_size, take);
    }
    if (max_size == 0) continue;
    if (is64)
      add_const_kernel<int64_t><<<dim3(grid_x_for(max_size), cnt), dim3(kBlock), 0, stream>>>(j);
    else
      add_const_kernel<int32_t><<<dim3(grid_x_for(max_size), cnt), dim3(kBlock), 0, stream>>>(j);
    RECIS_LAUNCH_CHECK();
  }
  return RECIS_OK;
}

int recis_unique(const int64_t* ids, int64_t n, int64_t* unique_out, void* inverse_out, int inverse_is64,
                 int64_t* count_out_dev, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(n >= 0 && n < (int64_t(1) << 30), "n out of range: %lld", (long long)n);
  RECIS_REQUIRE(count_out_dev != nullptr, "count_out_dev must not be NULL");
  int64_t cap = 1024;
  while (cap < 2 * n) cap <<= 1;
  const int64_t slots = cap + 1;
  const int64_t nb = std::max<int64_t>(1, (n + kBlock - 1) / kBlock);
  // workspace: keys[slots] | minpos[slots] | uid[slots] | slotpos[n] | block_counts[nb]
  size_t bytes = sizeof(int64_t) * slots + sizeof(int32_t) * (2 * slots + n + nb) + 64;
  void* ws = nullptr;
  if (int rc = get_workspace(stream, bytes, &ws)) return rc;
  int64_t* keys = static_cast<int64_t*>(ws);
  int32_t* minpos = reinterpret_cast<int32_t*>(keys + slots);
  int32_t* uid = minpos + slots;
  int32_t* slotpos = uid + slots;
  int32_t* block_counts = slotpos + n;
  RECIS_REQUIRE(n == 0 || (ids && unique_out && inverse_out), "NULL argument");
  set_init_kernel<<<dim3(std::min<int64_t>((slots + kBlock - 1) / kBlock, 256 * 16)), dim3(kBlock), 0, stream>>>(
      keys, minpos, slots);
  RECIS_LAUNCH_CHECK();
  if (n > 0) {
    set_insert_kernel<<<dim3(nb), dim3(kBlock), 0, stream>>>(keys, minpos, static_cast<uint64_t>(cap - 1), ids,
                                                             n, slotpos);
    RECIS_LAUNCH_CHECK();
    first_count_kernel<<<dim3(nb), dim3(kBlock), 0, stream>>>(minpos, slotpos, n, block_counts);
    RECIS_LAUNCH_CHECK();
  }
  scan_counts_kernel<<<1, 1024, 0, stream>>>(block_counts, n > 0 ? nb : 0, count_out_dev);
  RECIS_LAUNCH_CHECK();
  if (n > 0) {
    emit_unique_kernel<<<dim3(nb), dim3(kBlock), 0, stream>>>(ids, minpos, slotpos, n, block_counts,
                                                              unique_out, uid);
    RECIS_LAUNCH_CHECK();
    emit_inverse_kernel<<<dim3(nb), dim3(kBlock), 0, stream>>>(slotpos, uid, n, inverse_out, inverse_is64);
    RECIS_LAUNCH_CHECK();
  }
  return RECIS_OK;
}

}  // extern "C"
