// The device ordering of the reference's ids_partition (ids_partition_kernel.cu:36-55): unique ids
// ascending by rotr64(id, 16) taken as unsigned, which is by shard slot (id & 0xFFFF) first. One
// radix sort of (rotated id, position) pairs; the sorted ids, the order and its inverse (the rank of
// every input position) come out of one pass over the sorted pairs.
#include <hip/hip_runtime.h>

#include <rocprim/device/device_radix_sort.hpp>

#include "common.cuh"
#include "recis_hip.h"

namespace recis_hip {
namespace {

// The library's default configuration is kept on purpose: below 2^20 items it takes a merge sort, and
// forcing its one-sweep radix passes instead was measured slower at 0.9 M pairs (8 passes of 25 us and
// 17 buffer fills against 10 merge passes of 16 us).
using SortConfig = rocprim::default_config;

__global__ void __launch_bounds__(kBlock)
partition_keys_kernel(const int64_t* __restrict__ ids, int64_t n, uint64_t* __restrict__ keys,
                      int32_t* __restrict__ pos) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (i >= n) return;
  const uint64_t v = static_cast<uint64_t>(ids[i]);
  keys[i] = (v >> 16) | (v << 48);
  pos[i] = static_cast<int32_t>(i);
}

__global__ void __launch_bounds__(kBlock)
partition_finish_kernel(const uint64_t* __restrict__ keys, const int32_t* __restrict__ order, int64_t n,
                        int64_t* __restrict__ sorted_ids, int32_t* __restrict__ rank) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (i >= n) return;
  const uint64_t k = keys[i];
  sorted_ids[i] = static_cast<int64_t>((k << 16) | (k >> 48));
  rank[order[i]] = static_cast<int32_t>(i);
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
  RECIS_CHECK_HIP(rocprim::radix_sort_pairs<SortConfig>(nullptr, sort_bytes, nil64, nil64, nil32, nil32, un, 0u, 64u, stream));
  // workspace: keys_in[n] | keys_out[n] | pos[n] | the sort's own scratch
  const size_t pos_off = 2 * sizeof(uint64_t) * un;
  const size_t sort_off = (pos_off + sizeof(int32_t) * un + 255) & ~size_t(255);
  void* ws = nullptr;
  if (int rc = get_workspace(stream, sort_off + sort_bytes + 256, &ws)) return rc;
  uint64_t* keys_in = static_cast<uint64_t*>(ws);
  uint64_t* keys_out = keys_in + un;
  int32_t* pos = reinterpret_cast<int32_t*>(static_cast<char*>(ws) + pos_off);
  void* sort_ws = static_cast<char*>(ws) + sort_off;
  const dim3 grid(static_cast<unsigned>((n + kBlock - 1) / kBlock)), block(kBlock);
  RECIS_TIME_KERNEL("partition_keys_kernel", stream)
  partition_keys_kernel<<<grid, block, 0, stream>>>(ids, n, keys_in, pos);
  RECIS_LAUNCH_CHECK();
  RECIS_CHECK_HIP(rocprim::radix_sort_pairs<SortConfig>(sort_ws, sort_bytes, keys_in, keys_out, pos, order, un, 0u, 64u, stream));
  RECIS_TIME_KERNEL("partition_finish_kernel", stream)
  partition_finish_kernel<<<grid, block, 0, stream>>>(keys_out, order, n, sorted_ids, rank);
  RECIS_LAUNCH_CHECK();
  return RECIS_OK;
}
