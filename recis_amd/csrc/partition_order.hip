// The device ordering of the reference's ids_partition (ids_partition_kernel.cu:36-55): unique ids
// ascending by rotr64(id, 16) taken as unsigned, which is by shard slot (id & 0xFFFF) first.
//
// Two ways to the same result (sorted ids, the order, and its inverse: the rank of every input
// position), both the stable order of (rotated id, position):
//  * bins: the rotated ids are split by their top bits into bins of some 500 (a histogram, a scan of
//    the bin totals, a scatter of (key, position) records), and one workgroup per bin puts its
//    records in order in LDS (split once more by the next bits, then ranked by counting inside the
//    small groups). Five short kernels and one wait of the host for a word that says whether every
//    bin fits;
//  * a library sort of (rotated id, position) pairs, for small inputs, very large ones and inputs
//    whose shard slots are so unevenly spread that a bin overflows.
#include <hip/hip_runtime.h>

#include <rocprim/device/device_radix_sort.hpp>

#include <algorithm>
#include <type_traits>

#include "common.cuh"
#include "recis_hip.h"

namespace recis_hip {
namespace {

// The library's default configuration is kept on purpose: below 2^20 items it takes a merge sort, and
// forcing its one-sweep radix passes instead was measured slower at 0.9 M pairs (8 passes of 25 us and
// 17 buffer fills against 10 merge passes of 16 us).
using SortConfig = rocprim::default_config;

constexpr int kPoBlock = 1024;             // threads of the histogram / scatter kernels
constexpr int kPoPer = 8;                  // ids per thread there
constexpr int kPoTile = kPoBlock * kPoPer;
constexpr int kPoCap = 2048;               // most records of a bin the ranking kernel takes
constexpr int kPoTarget = 512;             // records per bin aimed at
constexpr int kPoMaxBinsLog2 = 13;         // the histogram of a workgroup lives in LDS
constexpr int64_t kPoMinIds = 32768;       // below this the library sort is a block sort and a few merges
constexpr int kRankBlock = 256;            // threads of the ranking kernel
constexpr int kRankPer = kPoCap / kRankBlock;

typedef uint32_t u4 __attribute__((ext_vector_type(4)));

struct PoItem {  // a record as it lies in memory, 16 bytes: one store, one load
  uint64_t key;
  int32_t pos;
  int32_t pad;
};

__device__ __forceinline__ uint64_t rotr16(uint64_t v) { return (v >> 16) | (v << 48); }
__device__ __forceinline__ uint64_t rotl16(uint64_t v) { return (v << 16) | (v >> 48); }
__device__ __forceinline__ int po_bin(uint64_t key, int nb_log2) {
  return nb_log2 == 0 ? 0 : static_cast<int>(key >> (64 - nb_log2));
}

__global__ void __launch_bounds__(kBlock) po_clear_kernel(int32_t* __restrict__ words, int n_words) {
  const int i = blockIdx.x * kBlock + threadIdx.x;
  if (i < n_words) words[i] = 0;
}

// records per bin: a histogram of the tile in LDS, one atomic per bin the tile has records for
__global__ void __launch_bounds__(kPoBlock)
po_hist_kernel(const int64_t* __restrict__ ids, int64_t n, int nb_log2, int32_t* __restrict__ bin_total) {
  extern __shared__ int32_t l_hist[];
  const int tid = threadIdx.x, nb = 1 << nb_log2;
  for (int b = tid; b < nb; b += kPoBlock) l_hist[b] = 0;
  __syncthreads();
  const int64_t lo = static_cast<int64_t>(blockIdx.x) * kPoTile;
#pragma unroll
  for (int x = 0; x < kPoPer; ++x) {
    const int64_t i = lo + x * kPoBlock + tid;
    if (i < n) atomicAdd(&l_hist[po_bin(rotr16(static_cast<uint64_t>(ids[i])), nb_log2)], 1);
  }
  __syncthreads();
  for (int b = tid; b < nb; b += kPoBlock) {
    const int32_t c = l_hist[b];
    if (c) atomicAdd(&bin_total[b], c);
  }
}

// bin_start [nb + 1] = exclusive scan of the totals; the host's word says whether a bin is too big.
// One workgroup.
__global__ void __launch_bounds__(kPoBlock)
po_starts_kernel(const int32_t* __restrict__ bin_total, int nb, int32_t* __restrict__ bin_start,
                 int64_t* __restrict__ too_big_host) {
  __shared__ int32_t s_sum[kPoBlock / kWave];
  __shared__ int32_t s_max[kPoBlock / kWave];
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const int per = (nb + kPoBlock - 1) / kPoBlock;
  const int lo = min(nb, tid * per), hi = min(nb, lo + per);
  int32_t sum = 0, mx = 0;
  for (int q = lo; q < hi; ++q) {
    const int32_t c = bin_total[q];
    sum += c;
    mx = max(mx, c);
  }
  int32_t incl = sum;
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    const int32_t y = __shfl_up(incl, o, kWave);
    if (lane >= o) incl += y;
    mx = max(mx, __shfl_xor(mx, o, kWave));
  }
  if (lane == kWave - 1) {
    s_sum[wave] = incl;
    s_max[wave] = mx;
  }
  __syncthreads();
  int32_t run = incl - sum, total = 0, all_max = 0;
#pragma unroll
  for (int w = 0; w < kPoBlock / kWave; ++w) {
    const int32_t c = s_sum[w];
    if (w < wave) run += c;
    total += c;
    all_max = max(all_max, s_max[w]);
  }
  for (int q = lo; q < hi; ++q) {
    bin_start[q] = run;
    run += bin_total[q];
  }
  if (tid == 0) {
    bin_start[nb] = total;
    *too_big_host = all_max > kPoCap ? 1 : 0;
  }
}

// (key, position) of every id goes to its bin: the tile's histogram again, one atomic per bin to
// reserve the tile's share of it, LDS counters for the places inside the share. Where a record
// lands inside its bin depends on the order the tiles arrive in; the ranking does not care.
__global__ void __launch_bounds__(kPoBlock)
po_scatter_kernel(const int64_t* __restrict__ ids, int64_t n, int nb_log2, const int32_t* __restrict__ bin_start,
                  int32_t* __restrict__ bin_cursor, u4* __restrict__ items) {
  extern __shared__ int32_t l_hist[];
  const int tid = threadIdx.x, nb = 1 << nb_log2;
  for (int b = tid; b < nb; b += kPoBlock) l_hist[b] = 0;
  __syncthreads();
  const int64_t lo = static_cast<int64_t>(blockIdx.x) * kPoTile;
  uint64_t k[kPoPer];
#pragma unroll
  for (int x = 0; x < kPoPer; ++x) {
    const int64_t i = lo + x * kPoBlock + tid;
    k[x] = i < n ? rotr16(static_cast<uint64_t>(ids[i])) : 0;
    if (i < n) atomicAdd(&l_hist[po_bin(k[x], nb_log2)], 1);
  }
  __syncthreads();
  for (int b = tid; b < nb; b += kPoBlock) {
    const int32_t c = l_hist[b];
    if (c) l_hist[b] = bin_start[b] + atomicAdd(&bin_cursor[b], c);
  }
  __syncthreads();
#pragma unroll
  for (int x = 0; x < kPoPer; ++x) {
    const int64_t i = lo + x * kPoBlock + tid;
    if (i >= n) continue;
    const int32_t p = atomicAdd(&l_hist[po_bin(k[x], nb_log2)], 1);
    if (p < 0 || static_cast<int64_t>(p) >= n) continue;  // cannot happen; never store out of bounds
    const u4 rec = {static_cast<uint32_t>(k[x]), static_cast<uint32_t>(k[x] >> 32), static_cast<uint32_t>(i), 0u};
    items[p] = rec;
  }
}

// One workgroup per bin. The bin's records are split once more in LDS, by the bits that follow the
// bin's (what is left of the shard slot, at most 8 bits), and inside such a group the rank of a
// record is the number of records of the group that come before it in the order of (key, position):
// a handful of comparisons per record instead of the whole bin's (counting over the whole bin was
// measured first: 170 us for 0.9 M ids, all of it 64-bit comparisons). The bits below the shard slot
// are the top bits of id >> 16, which real ids leave empty, so they do not help to split. The
// records then change places in LDS and leave in order.
constexpr int kSubMax = 256;
__global__ void __launch_bounds__(kRankBlock)
po_rank_kernel(const u4* __restrict__ items, const int32_t* __restrict__ bin_start, int64_t n, int nb_log2,
               int64_t* __restrict__ sorted_ids, int32_t* __restrict__ order, int32_t* __restrict__ rank_out) {
  __shared__ unsigned long long l_key[kPoCap];
  __shared__ int32_t l_pos[kPoCap];
  __shared__ int32_t s_start[kSubMax + 1];  // counts, then where each group starts
  __shared__ int32_t s_cur[kSubMax];
  __shared__ int32_t s_wave[kRankBlock / kWave];
  static_assert(kSubMax == kRankBlock, "one thread per group in the scan");
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const int32_t start = bin_start[blockIdx.x], cnt = bin_start[blockIdx.x + 1] - start;
  if (cnt <= 0 || cnt > kPoCap || start < 0 || static_cast<int64_t>(start) + cnt > n) return;  // uniform
  const int sub_bits = max(0, min(8, 16 - nb_log2));
  const int shift = 64 - nb_log2 - sub_bits;  // >= 40
  const unsigned sub_mask = (1u << sub_bits) - 1u;
  s_start[tid] = 0;
  if (tid == 0) s_start[kSubMax] = 0;
  __syncthreads();
  unsigned long long k[kRankPer];
  int32_t p[kRankPer], r[kRankPer];
  int sub[kRankPer];
#pragma unroll
  for (int x = 0; x < kRankPer; ++x) {
    const int i = tid + x * kRankBlock;
    k[x] = 0;
    p[x] = 0;
    r[x] = 0;
    sub[x] = 0;
    if (i < cnt) {
      const u4 rec = items[start + i];
      k[x] = static_cast<unsigned long long>(rec.x) | (static_cast<unsigned long long>(rec.y) << 32);
      p[x] = static_cast<int32_t>(rec.z);
      sub[x] = static_cast<int>(static_cast<unsigned>(k[x] >> shift) & sub_mask);
      atomicAdd(&s_start[sub[x]], 1);
    }
  }
  __syncthreads();
  {  // exclusive scan of the group counts, a thread per group
    const int32_t c = s_start[tid];
    int32_t incl = c;
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
      const int32_t y = __shfl_up(incl, o, kWave);
      if (lane >= o) incl += y;
    }
    if (lane == kWave - 1) s_wave[wave] = incl;
    __syncthreads();
    int32_t before = incl - c;
#pragma unroll
    for (int w = 0; w < kRankBlock / kWave; ++w) {
      if (w < wave) before += s_wave[w];
    }
    s_start[tid] = before;
    s_cur[tid] = before;
    if (tid == kRankBlock - 1) s_start[kSubMax] = before + c;
  }
  __syncthreads();
#pragma unroll
  for (int x = 0; x < kRankPer; ++x) {  // the groups, one after the other in LDS
    const int i = tid + x * kRankBlock;
    if (i >= cnt) continue;
    const int32_t at = atomicAdd(&s_cur[sub[x]], 1);
    if (at < 0 || at >= cnt) continue;  // cannot happen
    l_key[at] = k[x];
    l_pos[at] = p[x];
  }
  __syncthreads();
#pragma unroll
  for (int x = 0; x < kRankPer; ++x) {
    const int i = tid + x * kRankBlock;
    if (i >= cnt) continue;
    const int32_t lo = s_start[sub[x]], hi = min(cnt, s_start[sub[x] + 1]);
    int32_t before = 0;
    for (int32_t j = lo; j < hi; ++j) {
      const unsigned long long kj = l_key[j];
      const int32_t pj = l_pos[j];
      before += ((kj < k[x]) | ((kj == k[x]) & (pj < p[x]))) ? 1 : 0;
    }
    r[x] = lo + before;
  }
  __syncthreads();  // everybody has read the groups
#pragma unroll
  for (int x = 0; x < kRankPer; ++x) {
    const int i = tid + x * kRankBlock;
    if (i >= cnt || r[x] < 0 || r[x] >= cnt) continue;  // (a rank is below cnt by construction)
    l_key[r[x]] = k[x];
    l_pos[r[x]] = p[x];
    if (p[x] >= 0 && static_cast<int64_t>(p[x]) < n) rank_out[p[x]] = start + r[x];
  }
  __syncthreads();
  for (int i = tid; i < cnt; i += kRankBlock) {
    sorted_ids[start + i] = static_cast<int64_t>(rotl16(l_key[i]));
    order[start + i] = l_pos[i];
  }
}

__global__ void __launch_bounds__(kBlock)
partition_keys_kernel(const int64_t* __restrict__ ids, int64_t n, uint64_t* __restrict__ keys,
                      int32_t* __restrict__ pos) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (i >= n) return;
  keys[i] = rotr16(static_cast<uint64_t>(ids[i]));
  pos[i] = static_cast<int32_t>(i);
}

__global__ void __launch_bounds__(kBlock)
partition_finish_kernel(const uint64_t* __restrict__ keys, const int32_t* __restrict__ order, int64_t n,
                        int64_t* __restrict__ sorted_ids, int32_t* __restrict__ rank) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (i >= n) return;
  sorted_ids[i] = static_cast<int64_t>(rotl16(keys[i]));
  rank[order[i]] = static_cast<int32_t>(i);
}

// log2 of the number of bins for n ids, or -1 when the bins are not the way to take
int bins_log2_for(int64_t n) {
  if (n < kPoMinIds) return -1;
  int nb_log2 = 0;
  while (nb_log2 < kPoMaxBinsLog2 && ((n + (int64_t(1) << nb_log2) - 1) >> nb_log2) > kPoTarget) ++nb_log2;
  if (((n + (int64_t(1) << nb_log2) - 1) >> nb_log2) > kPoCap / 2) return -1;  // too many ids for the most bins
  return nb_log2;
}

}  // namespace
}  // namespace recis_hip

using namespace recis_hip;

extern "C" int recis_partition_order(const int64_t* ids, int64_t n, int64_t* sorted_ids, int32_t* order,
                                     int32_t* rank, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(n >= 0 && n <= INT32_MAX, "n must fit 32 bits");
  if (n == 0) return RECIS_OK;
  RECIS_REQUIRE(ids && sorted_ids && order && rank, "NULL argument");
  const size_t un = static_cast<size_t>(n);
  uint64_t* nil64 = nullptr;
  int32_t* nil32 = nullptr;
  size_t sort_bytes = 0;
  RECIS_CHECK_HIP(
      rocprim::radix_sort_pairs<SortConfig>(nullptr, sort_bytes, nil64, nil64, nil32, nil32, un, 0u, 64u, stream));
  // workspace of the library sort: keys_in[n] | keys_out[n] | pos[n] | the sort's own scratch;
  // of the bins: bin_total[nb] | bin_cursor[nb] | bin_start[nb + 1] | records[n]
  const size_t pos_off = 2 * sizeof(uint64_t) * un;
  const size_t sort_off = (pos_off + sizeof(int32_t) * un + 255) & ~size_t(255);
  const int nb_log2 = bins_log2_for(n);
  const size_t nb = nb_log2 >= 0 ? size_t(1) << nb_log2 : 0;
  const size_t items_off = (sizeof(int32_t) * (3 * nb + 1) + 255) & ~size_t(255);
  const size_t bins_bytes = nb_log2 >= 0 ? items_off + sizeof(PoItem) * un : 0;
  void* ws = nullptr;
  if (int rc = get_workspace(stream, std::max(sort_off + sort_bytes, bins_bytes) + 256, &ws)) return rc;

  if (nb_log2 >= 0) {
    int64_t* staged = nullptr;
    hipEvent_t staged_event = nullptr;
    if (int rc = get_count_staging(stream, &staged, &staged_event)) return rc;
    int64_t* too_big = staged + 2;  // (words 0 and 1 are the batch plan's)
    int32_t* bin_total = static_cast<int32_t*>(ws);
    int32_t* bin_cursor = bin_total + nb;
    int32_t* bin_start = bin_cursor + nb;
    u4* items = reinterpret_cast<u4*>(static_cast<char*>(ws) + items_off);
    const dim3 tiles(static_cast<unsigned>((n + kPoTile - 1) / kPoTile));
    const size_t lds = sizeof(int32_t) * nb;
    RECIS_TIME_KERNEL("partition_bins_hist", stream) {
      po_clear_kernel<<<dim3(static_cast<unsigned>((2 * nb + kBlock - 1) / kBlock)), dim3(kBlock), 0, stream>>>(
          bin_total, static_cast<int>(2 * nb));
      po_hist_kernel<<<tiles, dim3(kPoBlock), lds, stream>>>(ids, n, nb_log2, bin_total);
      po_starts_kernel<<<dim3(1), dim3(kPoBlock), 0, stream>>>(bin_total, static_cast<int>(nb), bin_start, too_big);
    }
    RECIS_LAUNCH_CHECK();
    // the one wait: whether every bin fits is a property of the ids
    RECIS_CHECK_HIP(hipStreamSynchronize(stream));
    if (*too_big == 0) {
      RECIS_TIME_KERNEL("partition_bins_scatter", stream)
      po_scatter_kernel<<<tiles, dim3(kPoBlock), lds, stream>>>(ids, n, nb_log2, bin_start, bin_cursor, items);
      RECIS_LAUNCH_CHECK();
      RECIS_TIME_KERNEL("partition_bins_rank", stream)
      po_rank_kernel<<<dim3(static_cast<unsigned>(nb)), dim3(kRankBlock), 0, stream>>>(items, bin_start, n, nb_log2,
                                                                                       sorted_ids, order, rank);
      RECIS_LAUNCH_CHECK();
      return RECIS_OK;
    }
  }

  uint64_t* keys_in = static_cast<uint64_t*>(ws);
  uint64_t* keys_out = keys_in + un;
  int32_t* pos = reinterpret_cast<int32_t*>(static_cast<char*>(ws) + pos_off);
  void* sort_ws = static_cast<char*>(ws) + sort_off;
  const dim3 grid(static_cast<unsigned>((n + kBlock - 1) / kBlock)), block(kBlock);
  RECIS_TIME_KERNEL("partition_keys_kernel", stream)
  partition_keys_kernel<<<grid, block, 0, stream>>>(ids, n, keys_in, pos);
  RECIS_LAUNCH_CHECK();
  RECIS_CHECK_HIP(
      rocprim::radix_sort_pairs<SortConfig>(sort_ws, sort_bytes, keys_in, keys_out, pos, order, un, 0u, 64u, stream));
  RECIS_TIME_KERNEL("partition_finish_kernel", stream)
  partition_finish_kernel<<<grid, block, 0, stream>>>(keys_out, order, n, sorted_ids, rank);
  RECIS_LAUNCH_CHECK();
  return RECIS_OK;
}
