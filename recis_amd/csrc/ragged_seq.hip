// Sequence ops on ragged tensors. (1) Truncation of lists of ragged tensors: the device side of fused_ragged_cutoff and
// fused_ragged_cutoff_3D (csrc/ops/fused_ragged_cutoff.cc:10-287, kernels
// fused_ragged_cutoff_kernel.cu:29-70, 260-371, 462-556, 634-728).
//
// Both shapes reduce to the same three steps over OUTPUT rows:
//   1. every output row gets a length and the position of its first element in the source values
//      (2-D: output row = input row, the first or last `keep` elements; 3-D: output row (s, j) is
//      inner row j of sequence s after dropping rows on one side, or an empty row of padding, so
//      that every sequence has exactly `keep` inner rows);
//   2. an exclusive scan of the lengths per tensor gives the output offsets and the value count;
//   3. the values are gathered row by row.
// One launch per step for the whole list (blockIdx.y = tensor). The scan is the classic three
// passes (sums of 2048-row blocks, one workgroup per tensor over the block sums, rescan with
// the block offset); no atomics, no host round trip before the value count is needed.
// (2) ragged_to_dense and dense_to_ragged (csrc/ops/ragged_to_dense_kernel.cu, dense_to_ragged_kernel.cu);
// the latter shares the scan and the row-wise copy of the truncation.
#include <algorithm>

#include "common.cuh"

namespace recis_hip {
namespace {

constexpr int kCutJobs = 24;  // tensors per launch: the job tables travel as kernel arguments (< 4 KB)
constexpr int kItems = 8;
constexpr int kRowsPerBlock = kBlock * kItems;  // 2048 output rows per workgroup

struct CutJobs {
  const void* outer[kCutJobs];   // 2-D: offsets [rows + 1]; 3-D: outer offsets [seqs + 1]
  const void* inner[kCutJobs];   // 3-D: inner offsets [inner_rows + 1]
  void* out_off[kCutJobs];       // [out_rows + 1]
  void* out_outer[kCutJobs];     // 3-D: [seqs + 1]
  void* drop_nums[kCutJobs];     // [rows] / [seqs], may be NULL
  void* pad_nums[kCutJobs];      // likewise
  int64_t* src[kCutJobs];        // [out_rows]: first source element of every output row
  int64_t rows[kCutJobs];        // input rows (2-D) / sequences (3-D)
  int64_t inner_rows[kCutJobs];  // 3-D: number of inner rows
  int64_t out_rows[kCutJobs];
  int64_t keep[kCutJobs];
  int64_t n_values[kCutJobs];
  int64_t sums_base[kCutJobs];   // first block sum of this tensor in the workspace
  uint8_t drop_left[kCutJobs];
  uint8_t pad_left[kCutJobs];
};

__device__ __forceinline__ int64_t block_sum(int64_t v, int64_t* lds) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_down(v, o, kWave);
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  if (lane == 0) lds[wave] = v;
  __syncthreads();
  int64_t total = 0;
#pragma unroll
  for (int w = 0; w < kBlock / kWave; ++w) total += lds[w];
  __syncthreads();
  return total;
}

// Step 1. Lengths go into out_off[r] (rescanned in place by step 2c).
template <bool THREE_D>
__global__ void __launch_bounds__(kBlock) cutoff_rows_kernel(CutJobs j, int is64, int64_t* block_sums, int* err) {
  __shared__ int64_t lds[kBlock / kWave];
  const int t = blockIdx.y;
  const int64_t out_rows = j.out_rows[t];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * kRowsPerBlock;
  if (base >= out_rows && !(THREE_D && base <= j.rows[t])) return;  // uniform per workgroup
  const int64_t keep = j.keep[t];
  int64_t sum = 0;
  for (int i = 0; i < kItems; ++i) {
    const int64_t r = base + static_cast<int64_t>(i) * kBlock + threadIdx.x;
    if (THREE_D && r <= j.rows[t]) store_index(j.out_outer[t], is64, r, r * keep);
    if (r >= out_rows) continue;
    int64_t len, src;
    if (!THREE_D) {
      // fused_ragged_cutoff_kernel.cu:55-69, 706-727
      const int64_t beg = load_index(j.outer[t], is64, r), end = load_index(j.outer[t], is64, r + 1);
      const int64_t src_len = end > beg ? end - beg : 0;
      const bool dropped = src_len >= keep;
      len = dropped ? keep : src_len;
      const int64_t drop = dropped ? src_len - keep : 0;
      if (j.drop_nums[t]) store_index(j.drop_nums[t], is64, r, drop);
      if (j.pad_nums[t]) store_index(j.pad_nums[t], is64, r, dropped ? 0 : keep - src_len);
      src = beg + (j.drop_left[t] ? drop : 0);
    } else {
      // fused_ragged_cutoff_kernel.cu:300-337
      const int64_t seq = r / keep, col = r % keep;
      const int64_t beg = load_index(j.outer[t], is64, seq), end = load_index(j.outer[t], is64, seq + 1);
      const int64_t seq_len = end > beg ? end - beg : 0;
      const int64_t drop = seq_len >= keep ? seq_len - keep : 0;
      const int64_t pad = seq_len >= keep ? 0 : keep - seq_len;
      if (col == 0) {
        if (j.drop_nums[t]) store_index(j.drop_nums[t], is64, seq, drop);
        if (j.pad_nums[t]) store_index(j.pad_nums[t], is64, seq, pad);
      }
      int64_t row = col;
      bool padded = false;
      if (drop > 0) {
        if (j.drop_left[t]) row += drop;
      } else if (pad > 0) {
        if (j.pad_left[t]) {
          padded = col < pad;
          row -= pad;
        } else {
          padded = keep <= pad + col;
        }
      }
      len = 0;
      src = 0;
      if (!padded) {
        const int64_t g = beg + row;
        if (g < 0 || g >= j.inner_rows[t]) {
          raise_device_error(err, RECIS_DEVERR_INDEX_RANGE);
        } else {
          const int64_t b = load_index(j.inner[t], is64, g), e = load_index(j.inner[t], is64, g + 1);
          len = e > b ? e - b : 0;
          src = b;
        }
      }
    }
    if (len > 0 && (src < 0 || src + len > j.n_values[t])) {
      raise_device_error(err, RECIS_DEVERR_INDEX_RANGE);
      len = 0;
    }
    store_index(j.out_off[t], is64, r, len);
    j.src[t][r] = src;
    sum += len;
  }
  if (base >= out_rows) return;
  const int64_t total = block_sum(sum, lds);
  if (threadIdx.x == 0) block_sums[j.sums_base[t] + blockIdx.x] = total;
}

// Step 2b. One workgroup per tensor: block sums -> exclusive block offsets, total.
__global__ void __launch_bounds__(kBlock) cutoff_scan_blocks_kernel(CutJobs j, int is64, int64_t* block_sums,
                                                                    int64_t* totals, int64_t totals_base) {
  __shared__ int64_t lds[kBlock];
  const int t = blockIdx.x;
  const int64_t nb = (j.out_rows[t] + kRowsPerBlock - 1) / kRowsPerBlock;
  int64_t* sums = block_sums + j.sums_base[t];
  int64_t carry = 0;
  for (int64_t b0 = 0; b0 < nb; b0 += kBlock) {
    const int64_t b = b0 + threadIdx.x;
    const int64_t v = b < nb ? sums[b] : 0;
    lds[threadIdx.x] = v;
    __syncthreads();
    for (int o = 1; o < kBlock; o <<= 1) {  // inclusive scan in LDS
      const int64_t add = threadIdx.x >= o ? lds[threadIdx.x - o] : 0;
      __syncthreads();
      lds[threadIdx.x] += add;
      __syncthreads();
    }
    if (b < nb) sums[b] = carry + lds[threadIdx.x] - v;
    carry += lds[kBlock - 1];
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    totals[totals_base + t] = carry;
    store_index(j.out_off[t], is64, j.out_rows[t], carry);
  }
}

// Step 2c. Lengths -> offsets, in place.
__global__ void __launch_bounds__(kBlock) cutoff_offsets_kernel(CutJobs j, int is64, const int64_t* block_sums) {
  __shared__ int64_t lds[kBlock / kWave];
  const int t = blockIdx.y;
  const int64_t out_rows = j.out_rows[t];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * kRowsPerBlock;
  if (base >= out_rows) return;
  // thread k owns rows base + k * kItems .. + kItems - 1
  const int64_t r0 = base + static_cast<int64_t>(threadIdx.x) * kItems;
  int64_t len[kItems];
  int64_t mine = 0;
#pragma unroll
  for (int i = 0; i < kItems; ++i) {
    len[i] = r0 + i < out_rows ? load_index(j.out_off[t], is64, r0 + i) : 0;
    mine += len[i];
  }
  // exclusive scan of `mine` over the workgroup: within the wave by shuffles, across waves through LDS
  int64_t incl = mine;
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    const int64_t up = __shfl_up(incl, o, kWave);
    if (lane >= o) incl += up;
  }
  if (lane == kWave - 1) lds[wave] = incl;
  __syncthreads();
  int64_t before = block_sums[j.sums_base[t] + blockIdx.x];
  for (int w = 0; w < wave; ++w) before += lds[w];
  int64_t at = before + incl - mine;
#pragma unroll
  for (int i = 0; i < kItems; ++i) {
    if (r0 + i < out_rows) store_index(j.out_off[t], is64, r0 + i, at);
    at += len[i];
  }
}

struct CopyJobs {
  const void* values[kCutJobs];
  void* out[kCutJobs];
  const void* out_off[kCutJobs];
  const int64_t* src[kCutJobs];
  int64_t out_rows[kCutJobs];
  int64_t total[kCutJobs];
};

// Step 3. A group of 2^g_log2 lanes per output row (g chosen by the host from the mean row length)
// copies the row's elements side by side: coalesced, no search.
template <typename T>
__global__ void __launch_bounds__(kBlock) cutoff_copy_kernel(CopyJobs j, int is64, int g_log2) {
  const int t = blockIdx.y;
  const T* in = static_cast<const T*>(j.values[t]);
  T* out = static_cast<T*>(j.out[t]);
  const int64_t rows = j.out_rows[t];
  const int g = 1 << g_log2;
  const int sub = threadIdx.x & (g - 1);
  const int64_t groups_per_grid = (static_cast<int64_t>(gridDim.x) * kBlock) >> g_log2;
  for (int64_t r = (static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x) >> g_log2; r < rows;
       r += groups_per_grid) {
    const int64_t beg = load_index(j.out_off[t], is64, r), end = load_index(j.out_off[t], is64, r + 1);
    const int64_t from = j.src[t][r] - beg;
    for (int64_t e = beg + sub; e < end; e += g) out[e] = in[from + e];
  }
}

// ---------------------------------------------------------------- dense <-> ragged
constexpr int kMaxRaggedDims = 5;

struct DenseArgs {
  const void* offsets[kMaxRaggedDims];
  int64_t width[kMaxRaggedDims];  // dense size of every ragged dimension
  int64_t n_off[kMaxRaggedDims];  // entries of every offsets array
  int n_dims;
  int64_t batch;
  int64_t folded;                 // product of the widths
  int64_t n_values;
};

// ragged_to_dense (ragged_to_dense_kernel.cu:34-84, walk of ragged_common.cuh:36-64): one thread
// per output element; its coordinates walk down the offsets, a coordinate beyond a row's length
// gives the default value.
template <typename T>
__global__ void __launch_bounds__(kBlock) ragged_to_dense_kernel(const T* values, T* out, DenseArgs a, int is64,
                                                                 T fill, int* err) {
  const int64_t total = a.batch * a.folded;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
  for (int64_t o = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; o < total; o += stride) {
    int64_t coord[kMaxRaggedDims];
    int64_t rest = o % a.folded;
    for (int d = a.n_dims - 1; d >= 0; --d) {
      coord[d] = rest % a.width[d];
      rest /= a.width[d];
    }
    int64_t at = o / a.folded;
    bool empty = false;
    for (int d = 0; d < a.n_dims; ++d) {
      if (at + 1 >= a.n_off[d]) {  // an outer offset points past the next level
        raise_device_error(err, RECIS_DEVERR_INDEX_RANGE);
        empty = true;
        break;
      }
      const int64_t beg = load_index(a.offsets[d], is64, at), end = load_index(a.offsets[d], is64, at + 1);
      if (coord[d] >= end - beg) {
        empty = true;
        break;
      }
      at = beg + coord[d];
    }
    if (!empty && (at < 0 || at >= a.n_values)) {
      raise_device_error(err, RECIS_DEVERR_INDEX_RANGE);
      empty = true;
    }
    out[o] = empty ? fill : values[at];
  }
}

// ragged_to_dense with one ragged level: a group of 2^g_log2 lanes per row streams the columns
// (offsets read once per row, no division per element).
template <typename T>
__global__ void __launch_bounds__(kBlock) ragged_to_dense_rows_kernel(const T* values, T* out, DenseArgs a, int is64,
                                                                      T fill, int g_log2, int* err) {
  const int g = 1 << g_log2;
  const int sub = threadIdx.x & (g - 1);
  const int64_t width = a.width[0];
  const int64_t groups_per_grid = (static_cast<int64_t>(gridDim.x) * kBlock) >> g_log2;
  for (int64_t r = (static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x) >> g_log2; r < a.batch;
       r += groups_per_grid) {
    const int64_t beg = load_index(a.offsets[0], is64, r), end = load_index(a.offsets[0], is64, r + 1);
    int64_t len = end > beg ? end - beg : 0;
    if (len > 0 && (beg < 0 || end > a.n_values)) {
      if (sub == 0) raise_device_error(err, RECIS_DEVERR_INDEX_RANGE);
      len = 0;
    }
    T* dst = out + r * width;
    for (int64_t c = sub; c < width; c += g) dst[c] = c < len ? values[beg + c] : fill;
  }
}

// dense_to_ragged, step 1 (dense_to_ragged_kernel.cu:16-30): the length of a row is the position
// after its last element that differs from `invalid`. A wave per row walks back from the end of
// the row, 64 columns at a time, and stops at the first chunk that holds such an element: the
// padding is read here, the rest of the row by the copy.
template <typename T>
__global__ void __launch_bounds__(kBlock) dense_row_lengths_kernel(const T* data, int64_t rows, int64_t cols,
                                                                   T invalid, int32_t* out_off, int64_t* src) {
  const int lane = threadIdx.x % kWave;
  const int64_t r = (static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x) / kWave;
  if (r >= rows) return;  // whole waves leave together
  int64_t last = -1;
  for (int64_t c0 = (cols - 1) / kWave * kWave; c0 >= 0 && last < 0; c0 -= kWave) {
    const int64_t c = c0 + lane;
    int64_t mine = (c < cols && data[r * cols + c] != invalid) ? c : -1;
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) {
      const int64_t other = __shfl_xor(mine, o, kWave);
      mine = other > mine ? other : mine;
    }
    last = mine;
  }
  if (lane == 0) {
    out_off[r] = static_cast<int32_t>(last + 1);
    src[r] = r * cols;
  }
}

// Sums of 2048-row blocks of lengths already stored in out_off (the input of the block scan).
__global__ void __launch_bounds__(kBlock) length_block_sums_kernel(const void* out_off, int is64, int64_t rows,
                                                                   int64_t* block_sums) {
  __shared__ int64_t lds[kBlock / kWave];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * kRowsPerBlock;
  int64_t sum = 0;
  for (int i = 0; i < kItems; ++i) {
    const int64_t r = base + static_cast<int64_t>(i) * kBlock + threadIdx.x;
    if (r < rows) sum += load_index(out_off, is64, r);
  }
  const int64_t total = block_sum(sum, lds);
  if (threadIdx.x == 0) block_sums[blockIdx.x] = total;
}

// ---------------------------------------------------------------- feature cross
// feature_cross_ragged (csrc/ops/feature_cross_ragged.cc:24-98, feature_cross_ragged_kernel.cu:
// 191-279): per segment, every distinct id of x paired with every distinct id of y; the pair's id is
// MurmurHash64A of the two 8-byte words (seed 0, ragged_common.cuh:105-125), its weight the
// product of the weights of the ids' first occurrences.

// Pass 1: rank[i] = 1 when element i is the first occurrence of its id in its row, else 0
// (a group of 2^g_log2 lanes per row; an element looks back over its row).
__global__ void __launch_bounds__(kBlock) cross_first_kernel(const int64_t* val, const void* off, int is64,
                                                             int64_t n_seg, int64_t n_val, int32_t* rank, int g_log2,
                                                             int* err) {
  const int g = 1 << g_log2;
  const int sub = threadIdx.x & (g - 1);
  const int64_t groups_per_grid = (static_cast<int64_t>(gridDim.x) * kBlock) >> g_log2;
  for (int64_t s = (static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x) >> g_log2; s < n_seg;
       s += groups_per_grid) {
    const int64_t beg = load_index(off, is64, s), end = load_index(off, is64, s + 1);
    if (beg < 0 || end > n_val || end < beg) {
      if (sub == 0) raise_device_error(err, RECIS_DEVERR_INDEX_RANGE);
      continue;
    }
    for (int64_t i = beg + sub; i < end; i += g) {
      const int64_t v = val[i];
      int32_t first = 1;
      for (int64_t k = beg; k < i; ++k)
        if (val[k] == v) {
          first = 0;
          break;
        }
      rank[i] = first;
    }
  }
}

// Pass 2: one thread per segment turns the flags into ranks (-1 for repeats), counts the distinct
// ids of both sides and stores the segment's output length.
__global__ void __launch_bounds__(kBlock) cross_rank_kernel(const void* x_off, const void* y_off, int is64,
                                                            int64_t n_seg, int64_t nx, int64_t ny, int32_t* x_rank,
                                                            int32_t* y_rank, int32_t* y_count, void* out_off) {
  const int64_t s = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (s >= n_seg) return;
  int64_t count[2];
  for (int side = 0; side < 2; ++side) {
    const void* off = side ? y_off : x_off;
    int32_t* rank = side ? y_rank : x_rank;
    const int64_t n = side ? ny : nx;
    const int64_t beg = load_index(off, is64, s), end = load_index(off, is64, s + 1);
    int32_t r = 0;
    if (beg >= 0 && end <= n)
      for (int64_t i = beg; i < end; ++i) rank[i] = rank[i] ? r++ : -1;
    count[side] = r;
  }
  y_count[s] = static_cast<int32_t>(count[1]);
  store_index(out_off, is64, s, count[0] * count[1]);
}

__device__ __forceinline__ uint64_t murmur_pair(uint64_t a, uint64_t b) {
  const uint64_t m = 0xc6a4a7935bd1e995ULL;
  uint64_t h = 0 ^ (16 * m);
  a *= m; a ^= a >> 47; a *= m; h ^= a; h *= m;
  b *= m; b ^= b >> 47; b *= m; h ^= b; h *= m;
  h ^= h >> 47;
  h *= m;
  h ^= h >> 47;
  return h;
}

// Pass 3: a lane group per segment walks the pairs of its rows; pairs of first occurrences land
// at offset + rank_x * distinct_y + rank_y.
template <typename W>
__global__ void __launch_bounds__(kBlock) cross_emit_kernel(const int64_t* xv, const void* x_off, const W* xw,
                                                            const int64_t* yv, const void* y_off, const W* yw,
                                                            int is64, int64_t n_seg, int64_t nx, int64_t ny,
                                                            const int32_t* x_rank, const int32_t* y_rank,
                                                            const int32_t* y_count, const void* out_off,
                                                            int64_t* out_val, W* out_w, int g_log2) {
  const int g = 1 << g_log2;
  const int sub = threadIdx.x & (g - 1);
  const int64_t groups_per_grid = (static_cast<int64_t>(gridDim.x) * kBlock) >> g_log2;
  for (int64_t s = (static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x) >> g_log2; s < n_seg;
       s += groups_per_grid) {
    const int64_t xb = load_index(x_off, is64, s), xe = load_index(x_off, is64, s + 1);
    const int64_t yb = load_index(y_off, is64, s), ye = load_index(y_off, is64, s + 1);
    if (xb < 0 || xe > nx || xe < xb || yb < 0 || ye > ny || ye < yb) continue;
    const int64_t ly = ye - yb, pairs = (xe - xb) * ly;
    const int64_t base = load_index(out_off, is64, s);
    const int64_t uy = y_count[s];
    for (int64_t p = sub; p < pairs; p += g) {
      const int64_t ix = xb + p / ly, iy = yb + p % ly;
      const int32_t rx = x_rank[ix], ry = y_rank[iy];
      if (rx < 0 || ry < 0) continue;
      const int64_t at = base + rx * uy + ry;
      out_val[at] = static_cast<int64_t>(murmur_pair(static_cast<uint64_t>(xv[ix]), static_cast<uint64_t>(yv[iy])));
      out_w[at] = (xw ? xw[ix] : W(1)) * (yw ? yw[iy] : W(1));
    }
  }
}

// ---------------------------------------------------------------- top-k index selection
// calc_ragged_index, drop left / pad right (csrc/ops/calc_ragged_index.cc:15-84): row r of
// topk [rows, cols] holds positions inside ragged row src = indicator[r], counted from the
// first element that a left truncation by drop_num[src] kept; position p stands for element
// offset[src] + drop_num[src] + p of the values and is kept when that lies inside the row.
// A wave per row: pass 1 counts the kept positions, pass 2 (after the scan) writes them in
// column order at out_off[r] + (kept positions before this column), by ballot and popcount.
struct TopkArgs {
  const void* drop_num;
  const void* offset;
  const void* topk;
  const void* indicator;
  int drop64, off64, topk64, ind64;
  int64_t rows, cols, src_rows;
};

template <bool EMIT>
__global__ void __launch_bounds__(kBlock) topk_index_kernel(TopkArgs a, void* out_off, void* out_index, int* err) {
  const int lane = threadIdx.x % kWave;
  const int64_t r = (static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x) / kWave;
  if (r >= a.rows) return;  // whole waves leave together
  const int64_t src = load_index(a.indicator, a.ind64, r);
  int64_t beg = 0, end = 0, drop = 0;
  if (src < 0 || src >= a.src_rows) {
    if (lane == 0) raise_device_error(err, RECIS_DEVERR_INDEX_RANGE);
  } else {
    beg = load_index(a.offset, a.off64, src);
    end = load_index(a.offset, a.off64, src + 1);
    drop = load_index(a.drop_num, a.drop64, src);
  }
  int64_t at = EMIT ? load_index(out_off, a.off64, r) : 0;
  for (int64_t c0 = 0; c0 < a.cols; c0 += kWave) {
    const int64_t c = c0 + lane;
    int64_t t = -1;
    bool keep = false;
    if (c < a.cols) {
      t = load_index(a.topk, a.topk64, r * a.cols + c) + beg + drop;
      keep = t >= beg && t < end;
    }
    const uint64_t mask = __ballot(keep);
    if constexpr (EMIT) {
      if (keep) store_index(out_index, a.topk64, at + __popcll(mask & ((uint64_t(1) << lane) - 1)), t);
    }
    at += __popcll(mask);
  }
  if constexpr (!EMIT) {
    if (lane == 0) store_index(out_off, a.off64, r, at);
  }
}

}  // namespace
}  // namespace recis_hip

using namespace recis_hip;

template <typename T>
static int ragged_to_dense_launch(const void* values, void* out, const DenseArgs& a, int is64, const void* fill,
                                  int* err, hipStream_t stream) {
  T f;
  __builtin_memcpy(&f, fill, sizeof(T));
  const int64_t total = a.batch * a.folded;
  if (a.n_dims == 1) {
    int g_log2 = 0;
    while (g_log2 < 6 && (int64_t(1) << g_log2) < a.width[0]) ++g_log2;
    const int64_t gx = std::min<int64_t>(((a.batch << g_log2) + kBlock - 1) / kBlock, 1 << 20);
    RECIS_TIME_KERNEL("ragged_to_dense_kernel", stream)
    ragged_to_dense_rows_kernel<T><<<dim3(static_cast<unsigned>(gx)), dim3(kBlock), 0, stream>>>(
        static_cast<const T*>(values), static_cast<T*>(out), a, is64, f, g_log2, err);
    RECIS_LAUNCH_CHECK();
    return RECIS_OK;
  }
  const int64_t gx = std::min<int64_t>((total + kBlock - 1) / kBlock, 1 << 20);
  RECIS_TIME_KERNEL("ragged_to_dense_kernel", stream)
  ragged_to_dense_kernel<T><<<dim3(static_cast<unsigned>(gx)), dim3(kBlock), 0, stream>>>(
      static_cast<const T*>(values), static_cast<T*>(out), a, is64, f, err);
  RECIS_LAUNCH_CHECK();
  return RECIS_OK;
}

extern "C" int recis_ragged_to_dense(const void* values, int elem_size, int64_t n_values,
                                     const void* const* offsets_ptrs, const int64_t* offsets_sizes, int off_is64,
                                     const int64_t* widths, int n_dims, const void* default_value, void* out,
                                     void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(n_dims >= 1 && n_dims <= kMaxRaggedDims, "ragged_to_dense: 1..%d ragged dimensions, got %d",
                kMaxRaggedDims, n_dims);
  RECIS_REQUIRE(offsets_ptrs && offsets_sizes && widths && default_value, "NULL argument");
  RECIS_REQUIRE(elem_size == 1 || elem_size == 2 || elem_size == 4 || elem_size == 8, "element size %d not supported",
                elem_size);
  DenseArgs a;
  a.n_dims = n_dims;
  a.folded = 1;
  for (int d = 0; d < n_dims; ++d) {
    RECIS_REQUIRE(offsets_ptrs[d] && offsets_sizes[d] >= 1 && widths[d] >= 0, "bad offsets in dimension %d", d);
    a.offsets[d] = offsets_ptrs[d];
    a.n_off[d] = offsets_sizes[d];
    a.width[d] = widths[d];
    a.folded *= widths[d];
  }
  a.batch = offsets_sizes[0] - 1;
  a.n_values = n_values;
  if (a.batch * a.folded == 0) return RECIS_OK;
  RECIS_REQUIRE(out && (n_values == 0 || values), "NULL tensor pointer");
  int* err = device_error_word(current_device());
  RECIS_REQUIRE(err != nullptr, "could not reach the device error word");
  switch (elem_size) {
    case 1: return ragged_to_dense_launch<uint8_t>(values, out, a, off_is64, default_value, err, stream);
    case 2: return ragged_to_dense_launch<uint16_t>(values, out, a, off_is64, default_value, err, stream);
    case 4: return ragged_to_dense_launch<uint32_t>(values, out, a, off_is64, default_value, err, stream);
    default: return ragged_to_dense_launch<uint64_t>(values, out, a, off_is64, default_value, err, stream);
  }
}

extern "C" int recis_dense_to_ragged_rows(const void* data, int dtype_kind, int64_t rows, int64_t cols,
                                          const void* invalid_value, int32_t* out_offsets, int64_t* src,
                                          int64_t* total_dev, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(rows >= 0 && cols >= 0, "negative size");
  RECIS_REQUIRE(out_offsets && total_dev && invalid_value && (rows == 0 || src), "NULL argument");
  RECIS_REQUIRE(rows * cols == 0 || data, "NULL data pointer");
  CutJobs j;
  j.out_off[0] = out_offsets;
  j.src[0] = src;
  j.out_rows[0] = rows;
  j.sums_base[0] = 0;
  const int64_t nb = (rows + kRowsPerBlock - 1) / kRowsPerBlock;
  void* ws = nullptr;
  int rc = get_workspace(stream, static_cast<size_t>(std::max<int64_t>(nb, 1)) * sizeof(int64_t), &ws);
  if (rc != RECIS_OK) return rc;
  int64_t* sums = static_cast<int64_t*>(ws);
  if (nb > 0) {
    const int64_t gw = (rows * kWave + kBlock - 1) / kBlock;
    RECIS_REQUIRE(gw < (int64_t(1) << 31), "too many rows");
    const dim3 grid(static_cast<unsigned>(gw));
    RECIS_TIME_KERNEL("dense_row_lengths_kernel", stream) {
      switch (dtype_kind) {  // comparison is by value: -0.0 == 0.0, NaN differs from everything
        case RECIS_SEQ_F32: {
          float x; __builtin_memcpy(&x, invalid_value, 4);
          dense_row_lengths_kernel<float><<<grid, dim3(kBlock), 0, stream>>>(static_cast<const float*>(data), rows, cols, x, out_offsets, src);
        } break;
        case RECIS_SEQ_F64: {
          double x; __builtin_memcpy(&x, invalid_value, 8);
          dense_row_lengths_kernel<double><<<grid, dim3(kBlock), 0, stream>>>(static_cast<const double*>(data), rows, cols, x, out_offsets, src);
        } break;
        case RECIS_SEQ_I32: {
          int32_t x; __builtin_memcpy(&x, invalid_value, 4);
          dense_row_lengths_kernel<int32_t><<<grid, dim3(kBlock), 0, stream>>>(static_cast<const int32_t*>(data), rows, cols, x, out_offsets, src);
        } break;
        case RECIS_SEQ_I64: {
          int64_t x; __builtin_memcpy(&x, invalid_value, 8);
          dense_row_lengths_kernel<int64_t><<<grid, dim3(kBlock), 0, stream>>>(static_cast<const int64_t*>(data), rows, cols, x, out_offsets, src);
        } break;
        default:
          return fail(RECIS_ERR_ARG, "dense_to_ragged: data must be float32, float64, int32 or int64");
      }
    }
    RECIS_LAUNCH_CHECK();
    length_block_sums_kernel<<<dim3(static_cast<unsigned>(nb)), dim3(kBlock), 0, stream>>>(out_offsets, 0, rows, sums);
    RECIS_LAUNCH_CHECK();
  }
  cutoff_scan_blocks_kernel<<<dim3(1), dim3(kBlock), 0, stream>>>(j, 0, sums, total_dev, 0);
  RECIS_LAUNCH_CHECK();
  if (nb > 0) {
    cutoff_offsets_kernel<<<dim3(static_cast<unsigned>(nb), 1), dim3(kBlock), 0, stream>>>(j, 0, sums);
    RECIS_LAUNCH_CHECK();
  }
  return RECIS_OK;
}

extern "C" int recis_ragged_cutoff_rows(const void* const* outer_ptrs, const void* const* inner_ptrs,
                                        int off_is64, const int64_t* n_rows, const int64_t* n_inner_rows,
                                        const int64_t* n_values, const int64_t* keep, const uint8_t* drop_left,
                                        const uint8_t* pad_left, int64_t n_tensors, void* const* out_offsets_ptrs,
                                        void* const* out_outer_ptrs, void* const* drop_nums_ptrs,
                                        void* const* pad_nums_ptrs, int64_t* const* src_ptrs,
                                        int64_t* totals_dev, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(n_tensors >= 0, "n_tensors must be >= 0");
  if (n_tensors == 0) return RECIS_OK;
  RECIS_REQUIRE(outer_ptrs && n_rows && n_values && keep && drop_left && pad_left && out_offsets_ptrs && src_ptrs &&
                    totals_dev, "NULL argument");
  const bool three_d = inner_ptrs != nullptr;
  RECIS_REQUIRE(!three_d || (n_inner_rows && out_outer_ptrs), "3-D cutoff needs inner row counts and outer outputs");
  int* err = device_error_word(current_device());
  RECIS_REQUIRE(err != nullptr, "could not reach the device error word");
  for (int64_t first = 0; first < n_tensors; first += kCutJobs) {
    CutJobs j;
    const int cnt = static_cast<int>(std::min<int64_t>(kCutJobs, n_tensors - first));
    int64_t max_rows = 0, n_sums = 0;
    for (int k = 0; k < cnt; ++k) {
      const int64_t t = first + k;
      RECIS_REQUIRE(n_rows[t] >= 0 && keep[t] >= 0 && n_values[t] >= 0, "negative size in tensor %lld", (long long)t);
      RECIS_REQUIRE(outer_ptrs[t] && out_offsets_ptrs[t], "NULL offsets pointer in tensor %lld", (long long)t);
      j.outer[k] = outer_ptrs[t];
      j.inner[k] = three_d ? inner_ptrs[t] : nullptr;
      j.out_off[k] = out_offsets_ptrs[t];
      j.out_outer[k] = three_d ? out_outer_ptrs[t] : nullptr;
      j.drop_nums[k] = drop_nums_ptrs ? drop_nums_ptrs[t] : nullptr;
      j.pad_nums[k] = pad_nums_ptrs ? pad_nums_ptrs[t] : nullptr;
      j.src[k] = src_ptrs[t];
      j.rows[k] = n_rows[t];
      j.inner_rows[k] = three_d ? n_inner_rows[t] : 0;
      j.out_rows[k] = three_d ? n_rows[t] * keep[t] : n_rows[t];
      RECIS_REQUIRE(!three_d || (inner_ptrs[t] && out_outer_ptrs[t] && n_inner_rows[t] >= 0),
                    "NULL inner offsets in tensor %lld", (long long)t);
      RECIS_REQUIRE(j.out_rows[k] == 0 || src_ptrs[t], "NULL scratch pointer in tensor %lld", (long long)t);
      j.keep[k] = keep[t];
      j.n_values[k] = n_values[t];
      j.drop_left[k] = drop_left[t];
      j.pad_left[k] = pad_left[t];
      j.sums_base[k] = n_sums;
      n_sums += (j.out_rows[k] + kRowsPerBlock - 1) / kRowsPerBlock;
      // the outer offsets of a 3-D output (rows + 1 entries) are written by the same grid
      max_rows = std::max(max_rows, std::max(j.out_rows[k], three_d ? j.rows[k] + 1 : 0));
    }
    void* ws = nullptr;
    int rc = get_workspace(stream, static_cast<size_t>(std::max<int64_t>(n_sums, 1)) * sizeof(int64_t), &ws);
    if (rc != RECIS_OK) return rc;
    int64_t* sums = static_cast<int64_t*>(ws);
    const int64_t gx = (max_rows + kRowsPerBlock - 1) / kRowsPerBlock;
    RECIS_REQUIRE(gx < (int64_t(1) << 31), "too many rows");
    if (gx > 0) {
      const dim3 grid(static_cast<unsigned>(gx), cnt);
      if (three_d) {
        RECIS_TIME_KERNEL("cutoff_rows_kernel", stream)
        cutoff_rows_kernel<true><<<grid, dim3(kBlock), 0, stream>>>(j, off_is64, sums, err);
      } else {
        RECIS_TIME_KERNEL("cutoff_rows_kernel", stream)
        cutoff_rows_kernel<false><<<grid, dim3(kBlock), 0, stream>>>(j, off_is64, sums, err);
      }
      RECIS_LAUNCH_CHECK();
    }
    cutoff_scan_blocks_kernel<<<dim3(cnt), dim3(kBlock), 0, stream>>>(j, off_is64, sums, totals_dev, first);
    RECIS_LAUNCH_CHECK();
    if (gx > 0) {
      RECIS_TIME_KERNEL("cutoff_offsets_kernel", stream)
      cutoff_offsets_kernel<<<dim3(static_cast<unsigned>(gx), cnt), dim3(kBlock), 0, stream>>>(j, off_is64, sums);
      RECIS_LAUNCH_CHECK();
    }
  }
  return RECIS_OK;
}

extern "C" int recis_ragged_cutoff_copy(const void* const* values_ptrs, int elem_size,
                                        const void* const* out_offsets_ptrs, int off_is64,
                                        const int64_t* n_out_rows, const int64_t* const* src_ptrs,
                                        const int64_t* totals, void* const* out_values_ptrs, int64_t n_tensors,
                                        void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(n_tensors >= 0, "n_tensors must be >= 0");
  if (n_tensors == 0) return RECIS_OK;
  RECIS_REQUIRE(values_ptrs && out_offsets_ptrs && n_out_rows && src_ptrs && totals && out_values_ptrs, "NULL argument");
  RECIS_REQUIRE(elem_size == 1 || elem_size == 2 || elem_size == 4 || elem_size == 8, "element size %d not supported",
                elem_size);
  for (int64_t first = 0; first < n_tensors; first += kCutJobs) {
    CopyJobs j;
    const int cnt = static_cast<int>(std::min<int64_t>(kCutJobs, n_tensors - first));
    int64_t max_total = 0;
    for (int k = 0; k < cnt; ++k) {
      const int64_t t = first + k;
      RECIS_REQUIRE(totals[t] >= 0 && n_out_rows[t] >= 0, "negative size in tensor %lld", (long long)t);
      RECIS_REQUIRE(totals[t] == 0 || (values_ptrs[t] && out_values_ptrs[t] && src_ptrs[t] && out_offsets_ptrs[t] &&
                                       n_out_rows[t] > 0), "NULL pointer in tensor %lld", (long long)t);
      j.values[k] = values_ptrs[t];
      j.out[k] = out_values_ptrs[t];
      j.out_off[k] = out_offsets_ptrs[t];
      j.src[k] = src_ptrs[t];
      j.out_rows[k] = n_out_rows[t];
      j.total[k] = totals[t];
      max_total = std::max(max_total, totals[t]);
    }
    if (max_total == 0) continue;
    int64_t sum_total = 0, sum_rows = 0, max_rows = 0;
    for (int k = 0; k < cnt; ++k) {
      sum_total += j.total[k];
      sum_rows += j.out_rows[k];
      max_rows = std::max(max_rows, j.out_rows[k]);
    }
    int g_log2 = 0;  // lanes per row: the power of two at or above the mean row length, at most a wave
    while (g_log2 < 6 && (int64_t(1) << g_log2) * sum_rows < sum_total) ++g_log2;
    const int64_t gx = std::min<int64_t>(((max_rows << g_log2) + kBlock - 1) / kBlock, 1 << 20);
    const dim3 grid(static_cast<unsigned>(std::max<int64_t>(gx, 1)), cnt);
    RECIS_TIME_KERNEL("cutoff_copy_kernel", stream) {
      switch (elem_size) {
        case 1: cutoff_copy_kernel<uint8_t><<<grid, dim3(kBlock), 0, stream>>>(j, off_is64, g_log2); break;
        case 2: cutoff_copy_kernel<uint16_t><<<grid, dim3(kBlock), 0, stream>>>(j, off_is64, g_log2); break;
        case 4: cutoff_copy_kernel<uint32_t><<<grid, dim3(kBlock), 0, stream>>>(j, off_is64, g_log2); break;
        default: cutoff_copy_kernel<uint64_t><<<grid, dim3(kBlock), 0, stream>>>(j, off_is64, g_log2); break;
      }
    }
    RECIS_LAUNCH_CHECK();
  }
  return RECIS_OK;
}

static int group_log2(int64_t total, int64_t rows) {
  int g = 0;
  while (g < 6 && (int64_t(1) << g) * rows < total) ++g;
  return g;
}

extern "C" int recis_feature_cross_rows(const int64_t* x_val, const void* x_off, int64_t nx, const int64_t* y_val,
                                        const void* y_off, int64_t ny, int off_is64, int64_t n_seg,
                                        int32_t* x_rank, int32_t* y_rank, int32_t* y_count, void* out_offsets,
                                        int64_t* total_dev, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(n_seg >= 0 && nx >= 0 && ny >= 0, "negative size");
  RECIS_REQUIRE(out_offsets && total_dev, "NULL argument");
  RECIS_REQUIRE(n_seg == 0 || (x_off && y_off && y_count), "NULL offsets pointer");
  RECIS_REQUIRE((nx == 0 || (x_val && x_rank)) && (ny == 0 || (y_val && y_rank)), "NULL values pointer");
  int* err = device_error_word(current_device());
  RECIS_REQUIRE(err != nullptr, "could not reach the device error word");
  CutJobs j;
  j.out_off[0] = out_offsets;
  j.out_rows[0] = n_seg;
  j.sums_base[0] = 0;
  const int64_t nb = (n_seg + kRowsPerBlock - 1) / kRowsPerBlock;
  void* ws = nullptr;
  int rc = get_workspace(stream, static_cast<size_t>(std::max<int64_t>(nb, 1)) * sizeof(int64_t), &ws);
  if (rc != RECIS_OK) return rc;
  int64_t* sums = static_cast<int64_t*>(ws);
  if (n_seg > 0) {
    for (int side = 0; side < 2; ++side) {
      const int64_t n = side ? ny : nx;
      if (n == 0) continue;
      const int g = group_log2(n, n_seg);
      const int64_t gx = std::min<int64_t>(((n_seg << g) + kBlock - 1) / kBlock, 1 << 20);
      RECIS_TIME_KERNEL("cross_first_kernel", stream)
      cross_first_kernel<<<dim3(static_cast<unsigned>(gx)), dim3(kBlock), 0, stream>>>(
          side ? y_val : x_val, side ? y_off : x_off, off_is64, n_seg, n, side ? y_rank : x_rank, g, err);
      RECIS_LAUNCH_CHECK();
    }
    const int64_t gr = (n_seg + kBlock - 1) / kBlock;
    RECIS_REQUIRE(gr < (int64_t(1) << 31), "too many segments");
    RECIS_TIME_KERNEL("cross_rank_kernel", stream)
    cross_rank_kernel<<<dim3(static_cast<unsigned>(gr)), dim3(kBlock), 0, stream>>>(
        x_off, y_off, off_is64, n_seg, nx, ny, x_rank, y_rank, y_count, out_offsets);
    RECIS_LAUNCH_CHECK();
    length_block_sums_kernel<<<dim3(static_cast<unsigned>(nb)), dim3(kBlock), 0, stream>>>(out_offsets, off_is64, n_seg,
                                                                                          sums);
    RECIS_LAUNCH_CHECK();
  }
  cutoff_scan_blocks_kernel<<<dim3(1), dim3(kBlock), 0, stream>>>(j, off_is64, sums, total_dev, 0);
  RECIS_LAUNCH_CHECK();
  if (nb > 0) {
    cutoff_offsets_kernel<<<dim3(static_cast<unsigned>(nb), 1), dim3(kBlock), 0, stream>>>(j, off_is64, sums);
    RECIS_LAUNCH_CHECK();
  }
  return RECIS_OK;
}

extern "C" int recis_feature_cross_emit(const int64_t* x_val, const void* x_off, const void* x_weight, int64_t nx,
                                        const int64_t* y_val, const void* y_off, const void* y_weight, int64_t ny,
                                        int off_is64, int weight_is_f64, int64_t n_seg, const int32_t* x_rank,
                                        const int32_t* y_rank, const int32_t* y_count, const void* out_offsets,
                                        int64_t total, int64_t* out_val, void* out_weight, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(n_seg >= 0 && nx >= 0 && ny >= 0 && total >= 0, "negative size");
  if (total == 0 || n_seg == 0) return RECIS_OK;
  RECIS_REQUIRE(x_val && x_off && y_val && y_off && x_rank && y_rank && y_count && out_offsets && out_val && out_weight,
                "NULL argument");
  // pairs examined per segment on average decide the lanes per segment
  const int g = group_log2(std::max<int64_t>(total, (nx / std::max<int64_t>(n_seg, 1)) * ny), n_seg);
  const int64_t gx = std::min<int64_t>(((n_seg << g) + kBlock - 1) / kBlock, 1 << 20);
  const dim3 grid(static_cast<unsigned>(gx));
  RECIS_TIME_KERNEL("cross_emit_kernel", stream) {
    if (weight_is_f64)
      cross_emit_kernel<double><<<grid, dim3(kBlock), 0, stream>>>(
          x_val, x_off, static_cast<const double*>(x_weight), y_val, y_off, static_cast<const double*>(y_weight),
          off_is64, n_seg, nx, ny, x_rank, y_rank, y_count, out_offsets, out_val, static_cast<double*>(out_weight), g);
    else
      cross_emit_kernel<float><<<grid, dim3(kBlock), 0, stream>>>(
          x_val, x_off, static_cast<const float*>(x_weight), y_val, y_off, static_cast<const float*>(y_weight),
          off_is64, n_seg, nx, ny, x_rank, y_rank, y_count, out_offsets, out_val, static_cast<float*>(out_weight), g);
  }
  RECIS_LAUNCH_CHECK();
  return RECIS_OK;
}

extern "C" int recis_ragged_topk_index(const void* drop_num, int drop_is64, const void* offset, int off_is64,
                                       int64_t src_rows, const void* topk, int topk_is64, const void* indicator,
                                       int indicator_is64, int64_t rows, int64_t cols, void* out_index,
                                       void* out_offsets, int64_t* total_dev, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(rows >= 0 && cols >= 0 && src_rows >= 0, "negative size");
  RECIS_REQUIRE(out_offsets && total_dev, "NULL argument");
  RECIS_REQUIRE(rows == 0 || (drop_num && offset && indicator), "NULL argument");
  RECIS_REQUIRE(rows * cols == 0 || (topk && out_index), "NULL topk / out_index pointer");
  TopkArgs a;
  a.drop_num = drop_num; a.offset = offset; a.topk = topk; a.indicator = indicator;
  a.drop64 = drop_is64; a.off64 = off_is64; a.topk64 = topk_is64; a.ind64 = indicator_is64;
  a.rows = rows; a.cols = cols; a.src_rows = src_rows;
  CutJobs j;
  j.out_off[0] = out_offsets;
  j.out_rows[0] = rows;
  j.sums_base[0] = 0;
  const int64_t nb = (rows + kRowsPerBlock - 1) / kRowsPerBlock;
  void* ws = nullptr;
  int rc = get_workspace(stream, static_cast<size_t>(std::max<int64_t>(nb, 1)) * sizeof(int64_t), &ws);
  if (rc != RECIS_OK) return rc;
  int64_t* sums = static_cast<int64_t*>(ws);
  const int64_t gw = (rows * kWave + kBlock - 1) / kBlock;
  RECIS_REQUIRE(gw < (int64_t(1) << 31), "too many rows");
  int* err = device_error_word(current_device());
  RECIS_REQUIRE(err != nullptr, "could not reach the device error word");
  if (nb > 0) {
    RECIS_TIME_KERNEL("topk_index_kernel(count)", stream) {
      topk_index_kernel<false><<<dim3(static_cast<unsigned>(gw)), dim3(kBlock), 0, stream>>>(a, out_offsets, nullptr, err);
    }
    RECIS_LAUNCH_CHECK();
    length_block_sums_kernel<<<dim3(static_cast<unsigned>(nb)), dim3(kBlock), 0, stream>>>(out_offsets, off_is64, rows, sums);
    RECIS_LAUNCH_CHECK();
  }
  cutoff_scan_blocks_kernel<<<dim3(1), dim3(kBlock), 0, stream>>>(j, off_is64, sums, total_dev, 0);
  RECIS_LAUNCH_CHECK();
  if (nb > 0) {
    cutoff_offsets_kernel<<<dim3(static_cast<unsigned>(nb), 1), dim3(kBlock), 0, stream>>>(j, off_is64, sums);
    RECIS_LAUNCH_CHECK();
    if (cols > 0) {
      RECIS_TIME_KERNEL("topk_index_kernel(emit)", stream) {
        topk_index_kernel<true><<<dim3(static_cast<unsigned>(gw)), dim3(kBlock), 0, stream>>>(a, out_offsets, out_index, err);
      }
      RECIS_LAUNCH_CHECK();
    }
  }
  return RECIS_OK;
}
