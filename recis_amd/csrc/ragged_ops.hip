// Remaining ragged ops for gfx950: the unpooled padded gather (ragged_tile) with
// its backward, the sparse-mode pooling ops (segment_sum / segment_mean) and
// gen_segment_indices_by_offset.
//
// Stand in for csrc/ops/ragged_tile_kernel.cu:26-280, csrc/ops/segment_ops_kernel.cu:11-291
// and csrc/ops/embedding_segment_reduce_kernel.cu:395-423.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <type_traits>

#include "common.cuh"

namespace recis_hip {
namespace {

// One feature of ragged_tile: `batch` samples, `seq` output rows per sample.
// Output row (b, t) = table[value[off[b] + t]] if t < len_b else 0.
template <typename T, int VEC>
__global__ void __launch_bounds__(kBlock)
tile_fwd_kernel(const void* __restrict__ value, int val64, const void* __restrict__ offset, int off64,
                const T* __restrict__ table, int64_t table_rows, T* __restrict__ out, int64_t batch,
                int64_t seq, int64_t n_values, int D, int lpr_log2, int blocks_per_sample, int* err) {
  // one sample per group of `blocks_per_sample` workgroups: no per-lane division, the sample's
  // two offsets are uniform loads; most output rows are padding, written once and not read here
  const int rows_per_block = kBlock >> lpr_log2;
  const int64_t b = blockIdx.x / blocks_per_sample;
  const int64_t t = static_cast<int64_t>(blockIdx.x % blocks_per_sample) * rows_per_block + (threadIdx.x >> lpr_log2);
  if (t >= seq) return;
  const int cl = threadIdx.x & ((1 << lpr_log2) - 1);
  const int64_t start = load_index(offset, off64, b), end = load_index(offset, off64, b + 1);
  const T* src = nullptr;
  if (start < 0 || end < start || end > n_values) {
    raise_device_error(err, RECIS_DEVERR_OFFSETS);
  } else if (t < end - start) {
    const int64_t idx = load_index(value, val64, start + t);
    if (static_cast<uint64_t>(idx) < static_cast<uint64_t>(table_rows))
      src = table + idx * D;
    else
      raise_device_error(err, RECIS_DEVERR_INDEX_RANGE);
  }
  T* dst = out + (b * seq + t) * D;
  for (int c0 = cl * VEC; c0 < D; c0 += VEC << lpr_log2) {
    Pack<T, VEC> v;
    if (src) {
      v = *reinterpret_cast<const Pack<T, VEC>*>(src + c0);
    } else {
#pragma unroll
      for (int j = 0; j < VEC; ++j) v.v[j] = from_float<T>(0.f);
    }
    if constexpr (sizeof(T) * VEC == 16) {
      typedef uint32_t u4 __attribute__((ext_vector_type(4)));
      u4 raw;
      __builtin_memcpy(&raw, &v, 16);
      __builtin_nontemporal_store(raw, reinterpret_cast<u4*>(dst + c0));
    } else {
      *reinterpret_cast<Pack<T, VEC>*>(dst + c0) = v;
    }
  }
}

// d_table[value[off[b] + t]] += dy[(b, t)] for t < min(len_b, seq); fp32 atomics.
template <typename T, int VEC>
__global__ void __launch_bounds__(kBlock)
tile_bwd_kernel(const void* __restrict__ value, int val64, const void* __restrict__ offset, int off64,
                const T* __restrict__ dy, float* __restrict__ d_table, int64_t table_rows, int64_t batch,
                int64_t seq, int64_t n_values, int D, int lpr_log2, int* err) {
  const int rows_per_block = kBlock >> lpr_log2;
  const int64_t row = static_cast<int64_t>(blockIdx.x) * rows_per_block + (threadIdx.x >> lpr_log2);
  if (row >= batch * seq) return;
  const int cl = threadIdx.x & ((1 << lpr_log2) - 1);
  const int64_t b = row / seq, t = row - b * seq;
  const int64_t start = load_index(offset, off64, b), end = load_index(offset, off64, b + 1);
  if (start < 0 || end < start || end > n_values) {
    raise_device_error(err, RECIS_DEVERR_OFFSETS);
    return;
  }
  if (t >= end - start) return;
  const int64_t idx = load_index(value, val64, start + t);
  if (static_cast<uint64_t>(idx) >= static_cast<uint64_t>(table_rows)) {
    raise_device_error(err, RECIS_DEVERR_INDEX_RANGE);
    return;
  }
  const T* src = dy + row * D;
  float* dst = d_table + idx * D;
  for (int c0 = cl * VEC; c0 < D; c0 += VEC << lpr_log2) {
    float v[VEC];
    load_pack<T, VEC>(src + c0, v);
#pragma unroll
    for (int j = 0; j < VEC; ++j) unsafeAtomicAdd(dst + c0 + j, v[j]);
  }
}

__global__ void __launch_bounds__(kBlock) fill_f32_kernel(float* p, int64_t n, float v) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; i < n; i += stride) p[i] = v;
}

// sparse mode: out[seg[i]] += data[indices[i]] * w[i]  (segment_ops_kernel.cu:133-165)
template <typename T, int VEC>
__global__ void __launch_bounds__(kBlock)
segment_sum_kernel(const T* __restrict__ data, int64_t data_rows, const void* __restrict__ weight, int wdt,
                   int use_weight, const void* __restrict__ indices, const void* __restrict__ seg_ids,
                   int idx64, float* __restrict__ out, int64_t n, int64_t num_segments, int D, int lpr_log2,
                   int* err) {
  const int rows_per_block = kBlock >> lpr_log2;
  const int64_t i = static_cast<int64_t>(blockIdx.x) * rows_per_block + (threadIdx.x >> lpr_log2);
  if (i >= n) return;
  const int cl = threadIdx.x & ((1 << lpr_log2) - 1);
  const int64_t src_row = load_index(indices, idx64, i);
  const int64_t seg = load_index(seg_ids, idx64, i);
  if (static_cast<uint64_t>(src_row) >= static_cast<uint64_t>(data_rows) ||
      static_cast<uint64_t>(seg) >= static_cast<uint64_t>(num_segments)) {
    raise_device_error(err, RECIS_DEVERR_INDEX_RANGE);
    return;
  }
  const int64_t wi = use_weight ? i : 0;
  float w = 1.f;
  if (weight) {
    if (wdt == RECIS_F32) w = static_cast<const float*>(weight)[wi];
    else if (wdt == RECIS_BF16) w = to_float(static_cast<const bf16_t*>(weight)[wi]);
    else w = to_float(static_cast<const f16_t*>(weight)[wi]);
  }
  for (int c0 = cl * VEC; c0 < D; c0 += VEC << lpr_log2) {
    float v[VEC];
    load_pack<T, VEC>(data + src_row * D + c0, v);
#pragma unroll
    for (int j = 0; j < VEC; ++j) unsafeAtomicAdd(out + seg * D + c0 + j, v[j] * w);
  }
}

// weight normalisation of the sparse-mode mean (segment_ops_kernel.cu:74-108)
__global__ void __launch_bounds__(kBlock)
weight_sum_kernel(const float* __restrict__ weight, int use_weight, const void* __restrict__ seg_ids,
                  int idx64, float* __restrict__ weight_sum, int64_t n, int64_t num_segments) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (i >= n) return;
  const int64_t s = load_index(seg_ids, idx64, i);
  if (s < 0 || s >= num_segments) return;
  unsafeAtomicAdd(weight_sum + s, weight[use_weight ? i : 0]);
}

__global__ void __launch_bounds__(kBlock)
weight_norm_kernel(const float* __restrict__ weight, int use_weight, const void* __restrict__ seg_ids,
                   int idx64, const float* __restrict__ weight_sum, float* __restrict__ out, int64_t n,
                   int64_t num_segments) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (i >= n) return;
  const int64_t s = load_index(seg_ids, idx64, i);
  const float w = weight[use_weight ? i : 0];
  out[i] = (s < 0 || s >= num_segments) ? w : w / weight_sum[s];
}

// out[j] = s such that offsets[s] <= j < offsets[s + 1]
__global__ void __launch_bounds__(kBlock)
segment_indices_kernel(const void* __restrict__ offsets, int off64, int64_t S, void* __restrict__ out,
                       int64_t total) {
  const int64_t j = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (j >= total) return;
  // largest s in [0, S) with offsets[s] <= j (empty segments share a boundary:
  // take the last one, which is the segment that owns position j)
  int64_t lo = 0, hi = S;  // invariant: offsets[lo] <= j < offsets[hi]
  while (hi - lo > 1) {
    const int64_t mid = (lo + hi) >> 1;
    if (load_index(offsets, off64, mid) <= j)
      lo = mid;
    else
      hi = mid;
  }
  store_index(out, off64, j, lo);
}

template <typename F>
int dispatch_t_vec(int dtype, int vec, F&& f) {
  auto with_vec = [&](auto t) {
    using T = decltype(t);
    switch (vec) {
      case 8:
        if constexpr (sizeof(T) == 2) return f(t, std::integral_constant<int, 8>{});
        return fail(RECIS_ERR_ARG, "internal: vector too wide");
      case 4: return f(t, std::integral_constant<int, 4>{});
      case 2: return f(t, std::integral_constant<int, 2>{});
      case 1: return f(t, std::integral_constant<int, 1>{});
      default: return fail(RECIS_ERR_ARG, "bad vector width %d", vec);
    }
  };
  if (dtype == RECIS_F32) return with_vec(float{});
  if (dtype == RECIS_BF16) return with_vec(bf16_t{});
  if (dtype == RECIS_F16) return with_vec(f16_t{});
  return fail(RECIS_ERR_ARG, "invalid dtype %d", dtype);
}

}  // namespace
}  // namespace recis_hip

using namespace recis_hip;

extern "C" {

int recis_ragged_tile(const int64_t* batch, const int64_t* seq, int64_t n_features, const void* value,
                      int value_is64, int64_t n_values, const void* offset, int off_is64,
                      const void* table, int64_t table_rows, int dtype, void* out, int64_t D,
                      void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(n_features >= 0 && n_values >= 0 && table_rows >= 0, "negative size");
  RECIS_REQUIRE(D >= 1 && D <= (1 << 20), "embedding dim %lld out of range", (long long)D);
  if (n_features == 0) return RECIS_OK;
  RECIS_REQUIRE(batch && seq && offset, "NULL argument");
  const int esz = dtype_size(dtype);
  RECIS_REQUIRE(esz, "invalid dtype %d", dtype);
  int* err = device_error_word(current_device());
  RECIS_REQUIRE(err != nullptr, "could not reach the device error word");
  const int vb = pick_vec_bytes(D * esz, reinterpret_cast<uintptr_t>(table) | reinterpret_cast<uintptr_t>(out));
  const int vec = std::max(1, vb / esz);
  const int lpr_log2 = std::min(6, ilog2_ceil((D + vec - 1) / vec));
  const int rows_per_block = kBlock >> lpr_log2;
  int64_t obase = 0, rbase = 0;
  const int osz = off_is64 ? 8 : 4;
  for (int64_t f = 0; f < n_features; ++f) {
    RECIS_REQUIRE(batch[f] >= 0 && seq[f] >= 0, "negative batch/seq");
    const int64_t rows = batch[f] * seq[f];
    if (rows > 0) {
      RECIS_REQUIRE(out != nullptr, "out must not be NULL");
      const int64_t blocks_per_sample = (seq[f] + rows_per_block - 1) / rows_per_block;
      const int64_t grid = batch[f] * blocks_per_sample;
      RECIS_REQUIRE(grid < (int64_t(1) << 31) && blocks_per_sample < (int64_t(1) << 31), "padded output too large");
      const void* off_f = static_cast<const char*>(offset) + obase * osz;
      int rc = dispatch_t_vec(dtype, vec, [&](auto t, auto vtag) {
        using T = decltype(t);
        constexpr int VEC = decltype(vtag)::value;
        RECIS_TIME_KERNEL("tile_fwd_kernel", stream)
        tile_fwd_kernel<T, VEC><<<dim3(grid), dim3(kBlock), 0, stream>>>(
            value, value_is64, off_f, off_is64, static_cast<const T*>(table), table_rows,
            static_cast<T*>(out) + rbase * D, batch[f], seq[f], n_values, static_cast<int>(D), lpr_log2,
            static_cast<int>(blocks_per_sample), err);
        RECIS_LAUNCH_CHECK();
        return RECIS_OK;
      });
      if (rc) return rc;
    }
    obase += batch[f];
    rbase += rows;
  }
  return RECIS_OK;
}

int recis_ragged_tile_back(const int64_t* batch, const int64_t* seq, int64_t n_features, const void* value,
                           int value_is64, int64_t n_values, const void* offset, int off_is64,
                           const void* dy, int dtype, float* d_table, int64_t table_rows, int64_t D,
                           void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(n_features >= 0 && n_values >= 0 && table_rows >= 0, "negative size");
  RECIS_REQUIRE(D >= 1 && D <= (1 << 20), "embedding dim %lld out of range", (long long)D);
  const int esz = dtype_size(dtype);
  RECIS_REQUIRE(esz, "invalid dtype %d", dtype);
  if (table_rows == 0) return RECIS_OK;
  RECIS_REQUIRE(d_table != nullptr, "d_table must not be NULL");
  {
    const int64_t total = table_rows * D;
    fill_f32_kernel<<<dim3(std::min<int64_t>((total + kBlock - 1) / kBlock, 256 * 32)), dim3(kBlock), 0, stream>>>(
        d_table, total, 0.f);
    RECIS_LAUNCH_CHECK();
  }
  if (n_features == 0) return RECIS_OK;
  RECIS_REQUIRE(batch && seq && offset, "NULL argument");
  int* err = device_error_word(current_device());
  RECIS_REQUIRE(err != nullptr, "could not reach the device error word");
  const int vb = pick_vec_bytes(D * esz, reinterpret_cast<uintptr_t>(dy));
  const int vec = std::max(1, vb / esz);
  const int lpr_log2 = std::min(6, ilog2_ceil((D + vec - 1) / vec));
  const int rows_per_block = kBlock >> lpr_log2;
  int64_t obase = 0, rbase = 0;
  const int osz = off_is64 ? 8 : 4;
  for (int64_t f = 0; f < n_features; ++f) {
    RECIS_REQUIRE(batch[f] >= 0 && seq[f] >= 0, "negative batch/seq");
    const int64_t rows = batch[f] * seq[f];
    if (rows > 0) {
      RECIS_REQUIRE(dy != nullptr, "dy must not be NULL");
      const int64_t grid = (rows + rows_per_block - 1) / rows_per_block;
      const void* off_f = static_cast<const char*>(offset) + obase * osz;
      int rc = dispatch_t_vec(dtype, vec, [&](auto t, auto vtag) {
        using T = decltype(t);
        constexpr int VEC = decltype(vtag)::value;
        tile_bwd_kernel<T, VEC><<<dim3(grid), dim3(kBlock), 0, stream>>>(
            value, value_is64, off_f, off_is64, static_cast<const T*>(dy) + rbase * D, d_table, table_rows,
            batch[f], seq[f], n_values, static_cast<int>(D), lpr_log2, err);
        RECIS_LAUNCH_CHECK();
        return RECIS_OK;
      });
      if (rc) return rc;
    }
    obase += batch[f];
    rbase += rows;
  }
  return RECIS_OK;
}

int recis_segment_sum(const void* data, int dtype, int64_t data_rows, const void* weight, int weight_dtype,
                      int use_weight, const void* indices, const void* segment_ids, int idx_is64,
                      float* out, int64_t n, int64_t num_segments, int64_t D, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(n >= 0 && num_segments >= 0 && data_rows >= 0, "negative size");
  RECIS_REQUIRE(D >= 1 && D <= (1 << 20), "embedding dim %lld out of range", (long long)D);
  const int esz = dtype_size(dtype);
  RECIS_REQUIRE(esz, "invalid dtype %d", dtype);
  if (num_segments == 0) return RECIS_OK;
  RECIS_REQUIRE(out != nullptr, "out must not be NULL");
  const int64_t total = num_segments * D;
  fill_f32_kernel<<<dim3(std::min<int64_t>((total + kBlock - 1) / kBlock, 256 * 32)), dim3(kBlock), 0, stream>>>(
      out, total, 0.f);
  RECIS_LAUNCH_CHECK();
  if (n == 0) return RECIS_OK;
  RECIS_REQUIRE(data && indices && segment_ids, "NULL argument");
  RECIS_REQUIRE(weight == nullptr || dtype_size(weight_dtype), "invalid weight dtype");
  int* err = device_error_word(current_device());
  RECIS_REQUIRE(err != nullptr, "could not reach the device error word");
  const int vb = pick_vec_bytes(D * esz, reinterpret_cast<uintptr_t>(data));
  const int vec = std::max(1, vb / esz);
  const int lpr_log2 = std::min(6, ilog2_ceil((D + vec - 1) / vec));
  const int rows_per_block = kBlock >> lpr_log2;
  const int64_t grid = (n + rows_per_block - 1) / rows_per_block;
  return dispatch_t_vec(dtype, vec, [&](auto t, auto vtag) {
    using T = decltype(t);
    constexpr int VEC = decltype(vtag)::value;
    segment_sum_kernel<T, VEC><<<dim3(grid), dim3(kBlock), 0, stream>>>(
        static_cast<const T*>(data), data_rows, weight, weight_dtype, use_weight, indices, segment_ids,
        idx_is64, out, n, num_segments, static_cast<int>(D), lpr_log2, err);
    RECIS_LAUNCH_CHECK();
    return RECIS_OK;
  });
}

int recis_segment_mean_weight(const float* weight, int use_weight, const void* segment_ids, int idx_is64,
                              float* weight_sum, float* weight_norm, int64_t n, int64_t num_segments,
                              void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(n >= 0 && num_segments >= 0, "negative size");
  RECIS_REQUIRE(weight != nullptr, "weight must not be NULL (pass a one-element tensor of 1 when unweighted)");
  if (num_segments > 0) {
    RECIS_REQUIRE(weight_sum != nullptr, "weight_sum must not be NULL");
    fill_f32_kernel<<<dim3(std::min<int64_t>((num_segments + kBlock - 1) / kBlock, 256 * 32)), dim3(kBlock), 0,
                      stream>>>(weight_sum, num_segments, 0.f);
    RECIS_LAUNCH_CHECK();
  }
  if (n == 0) return RECIS_OK;
  RECIS_REQUIRE(segment_ids && weight_norm, "NULL argument");
  const int64_t grid = (n + kBlock - 1) / kBlock;
  weight_sum_kernel<<<dim3(grid), dim3(kBlock), 0, stream>>>(weight, use_weight, segment_ids, idx_is64,
                                                            weight_sum, n, num_segments);
  RECIS_LAUNCH_CHECK();
  weight_norm_kernel<<<dim3(grid), dim3(kBlock), 0, stream>>>(weight, use_weight, segment_ids, idx_is64,
                                                             weight_sum, weight_norm, n, num_segments);
  RECIS_LAUNCH_CHECK();
  return RECIS_OK;
}

int recis_gen_segment_indices(const void* offsets, int off_is64, int64_t S, void* out, int64_t total,
                              void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(S >= 0 && total >= 0, "negative size");
  if (total == 0) return RECIS_OK;
  RECIS_REQUIRE(offsets && out && S >= 1, "NULL argument / no segment");
  segment_indices_kernel<<<dim3((total + kBlock - 1) / kBlock), dim3(kBlock), 0, stream>>>(offsets, off_is64, S,
                                                                                          out, total);
  RECIS_LAUNCH_CHECK();
  return RECIS_OK;
}

}  // extern "C"
