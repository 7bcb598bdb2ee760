// EmbeddingBlocks row movement for gfx950: gather / insert / filter over a slot
// stored as a list of equally sized blocks.
//
// Stands in for the device branches of csrc/ops/block_ops.cc:262-397
// (kernels: csrc/ops/block_ops_kernel.cu:16-392). Differences in design:
//   * the block pointer table is a device array owned by the caller and reused
//     across calls (the reference rebuilds and uploads it on every launch and
//     synchronises the stream afterwards, block_ops_kernel.cu:100-116,263-266)
//   * rows are moved as raw bytes with 16-byte vectors, a power-of-two group of
//     lanes per row, so one instantiation serves every element type
//   * a row index outside the table raises a soft error instead of faulting
#include <hip/hip_runtime.h>

#include <algorithm>
#include <type_traits>

#include "common.cuh"

namespace recis_hip {
namespace {

template <int VB>
struct alignas(VB) Bytes {
  unsigned char b[VB];
};

struct BlockArgs {
  const int64_t* ids;
  char* const* blocks;
  int64_t n_blocks;
  int64_t block_size;
  int64_t n;
  int row_bytes;
  int64_t pitch_bytes;  // from one row of a block to the next (row_bytes when the rows are dense)
  int lpr_log2;
  int* err;
};

// row index -> address of the row; NULL (and a soft error) when out of range
__device__ __forceinline__ char* row_address(const BlockArgs& a, int64_t idx) {
  if (idx < 0) return nullptr;
  int64_t b, r;
  if (a.n_blocks == 1) {
    b = 0;
    r = idx;
    if (idx >= a.block_size) return nullptr;
  } else if ((static_cast<uint64_t>(idx) | static_cast<uint64_t>(a.block_size)) >> 32) {
    b = idx / a.block_size;
    r = idx - b * a.block_size;
  } else {
    const uint32_t bs = static_cast<uint32_t>(a.block_size);
    const uint32_t q = static_cast<uint32_t>(idx) / bs;
    b = q;
    r = static_cast<uint32_t>(idx) - q * bs;
  }
  if (b >= a.n_blocks) return nullptr;
  return a.blocks[b] + r * a.pitch_bytes;
}

template <int VB>
__global__ void __launch_bounds__(kBlock)
block_gather_kernel(BlockArgs a, int64_t default_key, int readonly, char* __restrict__ out) {
  const int rows_per_block = kBlock >> a.lpr_log2;
  const int64_t i = static_cast<int64_t>(blockIdx.x) * rows_per_block + (threadIdx.x >> a.lpr_log2);
  if (i >= a.n) return;
  const int cl = threadIdx.x & ((1 << a.lpr_log2) - 1);
  const int64_t idx = a.ids[i];
  const char* src = nullptr;
  if (!(readonly && idx == default_key)) {
    src = row_address(a, idx);
    if (!src) raise_device_error(a.err, RECIS_DEVERR_INDEX_RANGE);
  }
  char* dst = out + i * static_cast<int64_t>(a.row_bytes);
  for (int c = cl * VB; c < a.row_bytes; c += VB << a.lpr_log2) {
    Bytes<VB> v;
    if (src) {
      v = *reinterpret_cast<const Bytes<VB>*>(src + c);
    } else {
#pragma unroll
      for (int k = 0; k < VB; ++k) v.b[k] = 0;
    }
    *reinterpret_cast<Bytes<VB>*>(dst + c) = v;
  }
}

template <int VB>
__global__ void __launch_bounds__(kBlock)
block_insert_kernel(BlockArgs a, const char* __restrict__ emb, int broadcast,
                    const uint8_t* __restrict__ mask) {
  const int rows_per_block = kBlock >> a.lpr_log2;
  const int64_t i = static_cast<int64_t>(blockIdx.x) * rows_per_block + (threadIdx.x >> a.lpr_log2);
  if (i >= a.n) return;
  if (mask && !mask[i]) return;
  const int cl = threadIdx.x & ((1 << a.lpr_log2) - 1);
  char* dst = row_address(a, a.ids[i]);
  if (!dst) {
    raise_device_error(a.err, RECIS_DEVERR_INDEX_RANGE);
    return;
  }
  const char* src = emb + (broadcast ? 0 : i * static_cast<int64_t>(a.row_bytes));
  for (int c = cl * VB; c < a.row_bytes; c += VB << a.lpr_log2)
    *reinterpret_cast<Bytes<VB>*>(dst + c) = *reinterpret_cast<const Bytes<VB>*>(src + c);
}

// flat table gather: out[i] = emb[ids[i]]
template <int VB>
__global__ void __launch_bounds__(kBlock)
gather_kernel(const void* __restrict__ ids, int ids64, const char* __restrict__ emb, int64_t rows,
              char* __restrict__ out, int64_t n, int row_bytes, int lpr_log2, int* err) {
  const int rows_per_block = kBlock >> lpr_log2;
  const int64_t i = static_cast<int64_t>(blockIdx.x) * rows_per_block + (threadIdx.x >> lpr_log2);
  if (i >= n) return;
  const int cl = threadIdx.x & ((1 << lpr_log2) - 1);
  const int64_t idx = load_index(ids, ids64, i);
  const bool ok = static_cast<uint64_t>(idx) < static_cast<uint64_t>(rows);
  if (!ok) raise_device_error(err, RECIS_DEVERR_INDEX_RANGE);
  const char* src = emb + idx * static_cast<int64_t>(row_bytes);
  char* dst = out + i * static_cast<int64_t>(row_bytes);
  for (int c = cl * VB; c < row_bytes; c += VB << lpr_log2) {
    Bytes<VB> v;
    if (ok) {
      v = *reinterpret_cast<const Bytes<VB>*>(src + c);
    } else {
#pragma unroll
      for (int k = 0; k < VB; ++k) v.b[k] = 0;
    }
    *reinterpret_cast<Bytes<VB>*>(dst + c) = v;
  }
}

__global__ void __launch_bounds__(kBlock)
block_filter_kernel(BlockArgs a, int64_t threshold, int slot64, uint8_t* __restrict__ mask_out) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (i >= a.n) return;
  const char* p = row_address(a, a.ids[i]);
  if (!p) {
    raise_device_error(a.err, RECIS_DEVERR_INDEX_RANGE);
    mask_out[i] = 0;
    return;
  }
  const int64_t v = slot64 ? *reinterpret_cast<const int64_t*>(p)
                           : static_cast<int64_t>(*reinterpret_cast<const int32_t*>(p));
  mask_out[i] = v < threshold;
}

template <typename F>
int dispatch_vb(int vb, F&& f) {
  switch (vb) {
    case 16: return f(std::integral_constant<int, 16>{});
    case 8: return f(std::integral_constant<int, 8>{});
    case 4: return f(std::integral_constant<int, 4>{});
    case 2: return f(std::integral_constant<int, 2>{});
    case 1: return f(std::integral_constant<int, 1>{});
    default: return fail(RECIS_ERR_ARG, "bad vector bytes %d", vb);
  }
}

int fill_args(BlockArgs& a, const int64_t* ids, void* const* blocks_dev, int64_t n_blocks,
              int64_t block_size, int64_t row_pitch_bytes, int64_t n, int64_t row_bytes, int vb) {
  RECIS_REQUIRE(n >= 0, "n must be >= 0");
  RECIS_REQUIRE(n_blocks >= 1 && block_size >= 1, "need at least one block (n_blocks=%lld block_size=%lld)",
                (long long)n_blocks, (long long)block_size);
  RECIS_REQUIRE(row_bytes >= 1 && row_bytes <= (1 << 22), "row_bytes out of range: %lld", (long long)row_bytes);
  RECIS_REQUIRE(ids != nullptr && blocks_dev != nullptr, "ids / blocks must not be NULL");
  a.ids = ids;
  a.blocks = reinterpret_cast<char* const*>(blocks_dev);
  a.n_blocks = n_blocks;
  a.block_size = block_size;
  a.n = n;
  a.row_bytes = static_cast<int>(row_bytes);
  a.pitch_bytes = row_pitch_bytes > 0 ? row_pitch_bytes : row_bytes;
  RECIS_REQUIRE(a.pitch_bytes >= row_bytes && a.pitch_bytes % vb == 0,
                "row pitch %lld does not fit rows of %lld bytes moved %d bytes at a time", (long long)a.pitch_bytes,
                (long long)row_bytes, vb);
  a.lpr_log2 = std::min(6, ilog2_ceil((row_bytes + vb - 1) / vb));
  a.err = device_error_word(current_device());
  RECIS_REQUIRE(a.err != nullptr, "could not reach the device error word");
  return RECIS_OK;
}

}  // namespace
}  // namespace recis_hip

using namespace recis_hip;

extern "C" {

int recis_gather(const void* ids, int ids_is64, const void* emb, int64_t rows, void* out, int64_t n,
                 int64_t row_bytes, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(n >= 0 && rows >= 0, "negative size");
  if (n == 0) return RECIS_OK;
  RECIS_REQUIRE(ids && emb && out, "NULL argument");
  RECIS_REQUIRE(row_bytes >= 1 && row_bytes <= (1 << 22), "row_bytes out of range: %lld", (long long)row_bytes);
  const int vb = pick_vec_bytes(row_bytes, reinterpret_cast<uintptr_t>(emb) | reinterpret_cast<uintptr_t>(out));
  const int lpr_log2 = std::min(6, ilog2_ceil((row_bytes + vb - 1) / vb));
  int* err = device_error_word(current_device());
  RECIS_REQUIRE(err != nullptr, "could not reach the device error word");
  const int rows_per_block = kBlock >> lpr_log2;
  const int64_t grid = (n + rows_per_block - 1) / rows_per_block;
  return dispatch_vb(vb, [&](auto tag) {
    constexpr int VB = decltype(tag)::value;
    RECIS_TIME_KERNEL("gather_kernel", stream)
    gather_kernel<VB><<<dim3(grid), dim3(kBlock), 0, stream>>>(
        ids, ids_is64, static_cast<const char*>(emb), rows, static_cast<char*>(out), n,
        static_cast<int>(row_bytes), lpr_log2, err);
    RECIS_LAUNCH_CHECK();
    return RECIS_OK;
  });
}

int recis_block_gather(const int64_t* ids, void* const* blocks_dev, int64_t n_blocks,
                       int64_t block_size, int64_t row_pitch_bytes, int64_t default_key, int readonly, void* out,
                       int64_t n, int64_t row_bytes, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (n == 0) return RECIS_OK;
  RECIS_REQUIRE(out != nullptr, "out must not be NULL");
  const int vb = pick_vec_bytes(row_bytes, reinterpret_cast<uintptr_t>(out) | static_cast<uintptr_t>(row_pitch_bytes));
  BlockArgs a;
  if (int rc = fill_args(a, ids, blocks_dev, n_blocks, block_size, row_pitch_bytes, n, row_bytes, vb)) return rc;
  const int rows_per_block = kBlock >> a.lpr_log2;
  const int64_t grid = (n + rows_per_block - 1) / rows_per_block;
  return dispatch_vb(vb, [&](auto tag) {
    constexpr int VB = decltype(tag)::value;
    RECIS_TIME_KERNEL("block_gather_kernel", stream)
    block_gather_kernel<VB><<<dim3(grid), dim3(kBlock), 0, stream>>>(a, default_key, readonly,
                                                                    static_cast<char*>(out));
    RECIS_LAUNCH_CHECK();
    return RECIS_OK;
  });
}

int recis_block_insert(const int64_t* ids, const void* emb, int broadcast, const uint8_t* mask,
                       void* const* blocks_dev, int64_t n_blocks, int64_t block_size, int64_t row_pitch_bytes,
                       int64_t n, int64_t row_bytes, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (n == 0) return RECIS_OK;
  RECIS_REQUIRE(emb != nullptr, "emb must not be NULL");
  const int vb = pick_vec_bytes(row_bytes, reinterpret_cast<uintptr_t>(emb) | static_cast<uintptr_t>(row_pitch_bytes));
  BlockArgs a;
  if (int rc = fill_args(a, ids, blocks_dev, n_blocks, block_size, row_pitch_bytes, n, row_bytes, vb)) return rc;
  const int rows_per_block = kBlock >> a.lpr_log2;
  const int64_t grid = (n + rows_per_block - 1) / rows_per_block;
  return dispatch_vb(vb, [&](auto tag) {
    constexpr int VB = decltype(tag)::value;
    block_insert_kernel<VB><<<dim3(grid), dim3(kBlock), 0, stream>>>(a, static_cast<const char*>(emb),
                                                                    broadcast, mask);
    RECIS_LAUNCH_CHECK();
    return RECIS_OK;
  });
}

int recis_block_filter(const int64_t* ids, void* const* blocks_dev, int64_t n_blocks,
                       int64_t block_size, int64_t threshold, int slot_is64, uint8_t* mask_out,
                       int64_t n, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (n == 0) return RECIS_OK;
  RECIS_REQUIRE(mask_out != nullptr, "mask_out must not be NULL");
  BlockArgs a;
  if (int rc = fill_args(a, ids, blocks_dev, n_blocks, block_size, 0, n, slot_is64 ? 8 : 4, slot_is64 ? 8 : 4))
    return rc;
  block_filter_kernel<<<dim3((n + kBlock - 1) / kBlock), dim3(kBlock), 0, stream>>>(a, threshold, slot_is64,
                                                                                   mask_out);
  RECIS_LAUNCH_CHECK();
  return RECIS_OK;
}

}  // extern "C"
