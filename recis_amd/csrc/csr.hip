// Consumers of the batch plan for gfx950: per-row work driven by the plan's occurrence lists.
//
//   gather-reduce  out[u] = sum over the list entries k of unique id u of coef[k] * rows[src[k]]
//                  (the backward of pooling and of the padded gather), optionally ending in the
//                  optimizer's update of table row row_index[u] instead of a store
//   expand         out[dst[k]] = w[dst[k]] * row(u): the forward of the lookup, each table row
//                  read once and written per occurrence
//   fill_lists     the src / coef arrays of the gather-reduce for the two pooling shapes
//
// The reference scatters gradients back to unique rows with one global atomic per element
// (csrc/ops/embedding_segment_reduce_kernel.cu:79-120, segment_ops_kernel.cu:133-165); here every
// unique row is summed by the lanes that own it, rows with very many occurrences are cut into
// work items whose partial sums a second small kernel folds, and nothing is atomic.
#include "csr_rows.cuh"

namespace recis_hip {
namespace {

// ------------------------------------------------------------------ expand (transpose of the gather-reduce)
// out[dst[k], :] = w[dst[k]] * row(u) for every list entry k of every unique id u: the forward
// of pooling when every segment holds exactly one id, and of the unpooled (tile) output. Each
// unique row is read ONCE and stored to all its occurrences; stores do not wait for anything,
// where the occurrence-major kernels chase index -> row index -> row for every output row.
struct ExpArgs {
  const int32_t* row_start;  // [U + 1]
  const int32_t* dst;        // [n] output row per list entry
  const void* weight;        // [n_out] per output row, or NULL
  int wdt;
  int64_t U, n_out;
  int D;
  int lpr_log2;
  int* err;
  const int64_t* row_index;  // rows in a block list: unique row u is row row_index[u] (negative = zeros)
  const void* const* blocks;
  int64_t block_rows, n_blocks;
  int64_t pitch;  // elements from one row of a block to the next
  int32_t hot_len;
  const int32_t* hot_items;
  const int64_t* counts;
  int64_t hot_cap;
  int64_t cold_blocks;
  // rows in a block list only: every row that is read also gets *stamp_value written into an
  // int64 slot of the same table (same blocks of block_rows rows), or NULL
  void* const* stamp_blocks;
  const int64_t* stamp_value;
};

// A row of zeros as long as any row (D <= 8192 of at most 4 bytes): what a unique id reads whose
// key the table does not hold, so that the row loads need no branch around them.
__device__ __align__(256) const unsigned char g_expand_zero_row[8192 * 4] = {};

constexpr int kExpandRows = 2;  // unique rows a lane group works at a time: their loads are in flight together (4: slower)

// STREAM: the rows are read with the streaming hint (a table larger than the caches keep, and any
// dense array of rows: each row is read once here); without it for a small table, whose rows the
// update at the end of the step and the next step's lookups find in the caches again.
template <typename TIn, typename TOut, int VEC, bool BLK, bool STREAM = true>
__global__ void __launch_bounds__(kBlock, 8)
csr_expand_kernel(const TIn* __restrict__ rows, TOut* __restrict__ out, ExpArgs a) {
  const int D = a.D;
  const int cl = threadIdx.x & ((1 << a.lpr_log2) - 1);
  const int lane = threadIdx.x & (kWave - 1);
  const int groups = kWave >> a.lpr_log2;  // lane groups of a wave
  const int g = lane >> a.lpr_log2;        // this lane's group in its wave

  auto load_row = [&](int64_t u, int c0, float (&v)[VEC], bool stamp_here) {
    const TIn* src = nullptr;
    if constexpr (BLK) {
      const int64_t ri = a.row_index[u];
      if (ri >= 0) {
        int64_t b = 0, r = ri;
        if (a.n_blocks > 1) {
          b = ri / a.block_rows;
          r = ri - b * a.block_rows;
        }
        if (b >= a.n_blocks || r >= a.block_rows) {
          raise_device_error(a.err, RECIS_DEVERR_INDEX_RANGE);
        } else {
          src = static_cast<const TIn*>(a.blocks[b]) + r * a.pitch;
          if (a.stamp_blocks && c0 == 0 && stamp_here) static_cast<int64_t*>(a.stamp_blocks[b])[r] = a.stamp_value[0];
        }
      }
    } else {
      src = rows + u * D;
    }
    if (src) {
      if constexpr (STREAM)
        load_pack_stream<TIn, VEC>(src + c0, v);  // every row is read once here
      else
        load_pack<TIn, VEC>(src + c0, v);
    } else {
#pragma unroll
      for (int j = 0; j < VEC; ++j) v[j] = 0.f;
    }
  };
  auto store_to = [&](int64_t d, int c0, const float (&v)[VEC]) {
    if (static_cast<uint64_t>(d) >= static_cast<uint64_t>(a.n_out)) {
      raise_device_error(a.err, RECIS_DEVERR_INDEX_RANGE);
      return;
    }
    float o[VEC];
    const float w = a.weight ? load_coef(a.weight, a.wdt, d) : 1.0f;
#pragma unroll
    for (int j = 0; j < VEC; ++j) o[j] = fmaf(v[j], w, 0.f);  // the pooled kernels' rounding
    store_pack_stream<TOut, VEC>(out + d * D + c0, o);
  };
  // stores to the list entries first, first + step, ... < last; the destinations of four entries
  // are fetched together so that their latencies overlap (more would cost resident waves)
  auto store_list = [&](int32_t first, int32_t last, int32_t step, int c0, const float (&v)[VEC]) {
    for (int32_t k = first; k < last; k += 4 * step) {
      int32_t d[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) d[i] = k + i * step < last ? a.dst[k + i * step] : -1;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (k + i * step < last) store_to(d[i], c0, v);
    }
  };

  const int64_t hot_blocks = static_cast<int64_t>(gridDim.x) - a.cold_blocks;
  if (static_cast<int64_t>(blockIdx.x) < hot_blocks) {
    // ---- hot work items: a workgroup per (row, chunk); all its lane groups hold the row
    int64_t n_items = a.counts[1];
    if (n_items > a.hot_cap) n_items = a.hot_cap;
    const int groups_per_block = kBlock >> a.lpr_log2;
    const int gb = threadIdx.x >> a.lpr_log2;
    for (int64_t item = blockIdx.x; item < n_items; item += hot_blocks) {
      const int32_t u = a.hot_items[2 * item];
      const int32_t chunk = a.hot_items[2 * item + 1];
      const int32_t start = a.row_start[u] + chunk * kHotChunk;
      const int32_t end = min(a.row_start[u + 1], start + kHotChunk);
      for (int c0 = cl * VEC; c0 < D; c0 += VEC << a.lpr_log2) {
        float v[VEC];
        load_row(u, c0, v, chunk == 0 && gb == 0);  // a hot row is stamped once: by its first work item
        store_list(start + gb, end, groups_per_block, c0, v);
      }
    }
    return;
  }

  // ---- cold rows: kExpandRows of them per lane group. The kernel is a chain of dependent accesses
  // per row (list bounds -> row index -> row -> destinations -> stores) with 16 bytes per lane in
  // flight; with every resident wave busy that is still too little to fill the memory system, so a
  // group walks the chain for two rows at once, and the cold workgroups stride over the batches of
  // rows with the NEXT batch's list bounds and table rows asked for before this batch is worked
  // (their round trip runs under this batch's row reads and stores).
  const int groups_per_block = kBlock >> a.lpr_log2;
  const int32_t per_batch = kExpandRows * groups_per_block;
  const void* base0 = nullptr;
  void* stamp_base0 = nullptr;
  if constexpr (BLK) {
    base0 = a.blocks[0];
    if (a.stamp_blocks) stamp_base0 = a.stamp_blocks[0];
  }
  // U may be the caller's upper bound (the plan's own count decides which rows exist): the arrays
  // hold U entries, so a row below U is safe to read.
  const int32_t n_unique = static_cast<int32_t>(min(a.U, a.counts[0]));
  const int32_t n_batches = (n_unique + per_batch - 1) / per_batch;
  const int32_t stride = static_cast<int32_t>(a.cold_blocks);
  int32_t start_n[kExpandRows], end_n[kExpandRows];
  int64_t ri_n[kExpandRows];
  auto ask = [&](int32_t bt) {
#pragma unroll
    for (int r = 0; r < kExpandRows; ++r) {
      const int32_t un = bt * per_batch + (threadIdx.x >> a.lpr_log2) + r * groups_per_block;
      const int32_t at = un < n_unique ? un : 0;
      start_n[r] = a.row_start[at];
      end_n[r] = a.row_start[at + 1];
      ri_n[r] = BLK ? a.row_index[at] : 0;
    }
  };
  int32_t batch = static_cast<int32_t>(static_cast<int64_t>(blockIdx.x) - hot_blocks);
  if (batch < n_batches) ask(batch);
  for (; batch < n_batches; batch += stride) {
  int64_t u[kExpandRows];
  int32_t start[kExpandRows], end[kExpandRows];
  int64_t ri_read[kExpandRows];
  bool is_long[kExpandRows], is_short[kExpandRows];
#pragma unroll
  for (int r = 0; r < kExpandRows; ++r) {
    u[r] = static_cast<int64_t>(batch) * per_batch + (threadIdx.x >> a.lpr_log2) + r * groups_per_block;
    start[r] = start_n[r];
    end[r] = end_n[r];
    ri_read[r] = ri_n[r];
    if (u[r] >= n_unique) start[r] = end[r] = 0;
  }
  if (batch + stride < n_batches) ask(batch + stride);
#pragma unroll
  for (int r = 0; r < kExpandRows; ++r) {
    if (end[r] - start[r] > a.hot_len) end[r] = start[r];  // written by the work items
    is_long[r] = a.lpr_log2 < 6 && end[r] - start[r] > kCoopLen;
    is_short[r] = !is_long[r] && end[r] > start[r];
  }
  // short rows: where the rows lie first (no branch around a load: a missing row reads zeros), then
  // the rows, then the stores
  const TIn* src[kExpandRows];
  if constexpr (BLK) {
    // in stages, each stage's loads of all the rows in flight together and no branch around any of
    // them: block pointers (of block 0 for a row that reads zeros; none for a table in one block),
    // then the rows
    int64_t ri[kExpandRows], off[kExpandRows], blk[kExpandRows];
    int32_t ok[kExpandRows];
    const int64_t stamp = a.stamp_blocks ? a.stamp_value[0] : 0;  // (uniform)
#pragma unroll
    for (int r = 0; r < kExpandRows; ++r) ri[r] = is_short[r] ? ri_read[r] : -1;
    bool bad_any = false;
#pragma unroll
    for (int r = 0; r < kExpandRows; ++r) {
      int64_t b = 0;
      off[r] = ri[r];
      if (a.n_blocks > 1) {  // (uniform)
        b = ri[r] >= 0 ? ri[r] / a.block_rows : 0;
        off[r] = ri[r] - b * a.block_rows;
      }
      const bool bad = (ri[r] >= 0) & ((b >= a.n_blocks) | (off[r] >= a.block_rows));
      bad_any = bad_any | bad;
      ok[r] = (ri[r] >= 0) & !bad;
      blk[r] = ok[r] ? b : 0;
    }
    const void* base[kExpandRows];
    void* stamp_base[kExpandRows];
#pragma unroll
    for (int r = 0; r < kExpandRows; ++r) {
      if (a.n_blocks == 1) {  // (uniform) one block: its address came with the first round trip
        base[r] = base0;
        stamp_base[r] = stamp_base0;
      } else {
        base[r] = a.blocks[blk[r]];
        stamp_base[r] = a.stamp_blocks ? a.stamp_blocks[blk[r]] : nullptr;  // (uniform choice)
      }
    }
#pragma unroll
    for (int r = 0; r < kExpandRows; ++r) {
      src[r] = ok[r] ? static_cast<const TIn*>(base[r]) + off[r] * a.pitch : reinterpret_cast<const TIn*>(g_expand_zero_row);
      if (a.stamp_blocks && cl == 0 && ok[r]) static_cast<int64_t*>(stamp_base[r])[off[r]] = stamp;
    }
    if (bad_any) raise_device_error(a.err, RECIS_DEVERR_INDEX_RANGE);
  } else {
#pragma unroll
    for (int r = 0; r < kExpandRows; ++r)
      src[r] = is_short[r] ? rows + u[r] * D : reinterpret_cast<const TIn*>(g_expand_zero_row);
  }
  for (int c0 = cl * VEC; c0 < D; c0 += VEC << a.lpr_log2) {
    float v[kExpandRows][VEC];
#pragma unroll
    for (int r = 0; r < kExpandRows; ++r) {
      if constexpr (STREAM)
        load_pack_stream<TIn, VEC>(src[r] + c0, v[r]);  // every row is read once here
      else
        load_pack<TIn, VEC>(src[r] + c0, v[r]);
    }
#pragma unroll
    for (int r = 0; r < kExpandRows; ++r)
      if (is_short[r]) store_list(start[r], end[r], 1, c0, v[r]);
  }
  // long rows of this wave, one after the other: the owner's row reaches every group by shuffles
#pragma unroll
  for (int r = 0; r < kExpandRows; ++r) {
    uint64_t todo = __ballot(is_long[r]);
    while (todo) {
      const int owner = __ffsll(static_cast<unsigned long long>(todo)) - 1;
      todo &= ~(((uint64_t(1) << (1 << a.lpr_log2)) - 1) << owner);
      const int32_t r_start = __shfl(start[r], owner, kWave), r_end = __shfl(end[r], owner, kWave);
      const int64_t row = u[r] - g + (owner >> a.lpr_log2);  // rows of a wave are consecutive
      for (int cbase = 0; cbase < D; cbase += VEC << a.lpr_log2) {  // uniform: shuffles inside
        const int c0 = cbase + cl * VEC;
        const bool col_ok = c0 < D;
        float mine[VEC], v[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) mine[j] = 0.f;
        if (lane >> a.lpr_log2 == owner >> a.lpr_log2 && col_ok) load_row(row, c0, mine, true);
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[j] = __shfl(mine[j], owner + cl, kWave);
        if (col_ok) store_list(r_start + g, r_end, groups, c0, v);
      }
    }
  }
  }  // batches
}

// src / coef of every list entry, for the backward of pooled segments and of the padded gather over
// the same occurrences. Entry k lists occurrence i = list[k], which lies in segment s (the largest
// s with offsets[s] <= i, found by bisection: the offsets of a batch stay in the caches) at place
// t = i - offsets[s]:
//   pooled segments  src = s, coef = w_i (divided by the segment length for mean)
//   padded gather    segment s is sample b = s - seg_lo[f] of feature f, and place t of it is padded
//                    row rbase[f] + b * seq[f] + t, or nothing (-1) when t >= seq[f]
// Reads and writes go by list entry, so every array is streamed; one launch serves both shapes.
constexpr int kFillFeatures = 32;  // features of the padded gather per launch
struct FillArgs {
  const int32_t* list;
  int64_t n;
  const void* offsets;
  int off64;
  int64_t S;
  const void* weight;
  int wdt;
  int mean;
  int32_t* src_pool;  // or NULL
  float* coef;        // or NULL
  int32_t* src_tile;  // or NULL
  int n_features;
  int first_group;    // this launch also marks the entries that no segment covers
  int64_t seg_lo[kFillFeatures + 1];
  int64_t seq[kFillFeatures];
  int64_t rbase[kFillFeatures];
  int64_t coarse_stride;  // every coarse_stride-th offset goes into the workgroup's LDS table
  int n_coarse;
};
// The bisection runs in two stages: over every coarse_stride-th offset, in LDS (a workgroup loads
// that table once for the kFillPer entries of each of its threads), then over the few offsets in
// between, in memory. A bisection of the whole array out of the caches is a dozen dependent loads
// per entry (27 us for the 1.6 M entries and 8193 offsets of the sequence workload; 2 - 3 loads now).
constexpr int kFillCoarse = 2048;
constexpr int kFillPer = 4;
__global__ void __launch_bounds__(kBlock)
fill_lists_kernel(FillArgs a) {
  __shared__ int32_t s_coarse[kFillCoarse];
  for (int c = threadIdx.x; c < a.n_coarse; c += kBlock) {
    const int64_t v = load_index(a.offsets, a.off64, c * a.coarse_stride);
    s_coarse[c] = static_cast<int32_t>(min(v, static_cast<int64_t>(INT32_MAX)));  // places are below 2^30
  }
  __syncthreads();
  const int64_t first = load_index(a.offsets, a.off64, 0), last = load_index(a.offsets, a.off64, a.S);
#pragma unroll 1
  for (int x = 0; x < kFillPer; ++x) {
  const int64_t k = (static_cast<int64_t>(blockIdx.x) * kFillPer + x) * kBlock + threadIdx.x;
  if (k >= a.n) return;
  const int64_t i = a.list[k];
  if (i < first || i >= last) {
    if (a.first_group) {
      if (a.src_pool) a.src_pool[k] = -1;
      if (a.coef) a.coef[k] = 0.f;
      if (a.src_tile) a.src_tile[k] = -1;
    }
    continue;
  }
  int64_t lo, hi;
  {
    int c_lo = 0, c_hi = a.n_coarse;  // s_coarse[c_lo] <= i < s_coarse[c_hi] (the end counts as larger)
    while (c_hi - c_lo > 1) {
      const int mid = (c_lo + c_hi) >> 1;
      if (s_coarse[mid] <= i)
        c_lo = mid;
      else
        c_hi = mid;
    }
    lo = c_lo * a.coarse_stride;
    hi = min(a.S, lo + a.coarse_stride);
  }
  while (hi - lo > 1) {
    const int64_t mid = (lo + hi) >> 1;
    if (load_index(a.offsets, a.off64, mid) <= i)
      lo = mid;
    else
      hi = mid;
  }
  const int64_t begin = load_index(a.offsets, a.off64, lo);
  if (a.first_group) {
    if (a.src_pool) a.src_pool[k] = static_cast<int32_t>(lo);
    if (a.coef) {
      float w = a.weight ? load_coef(a.weight, a.wdt, i) : 1.0f;
      if (a.mean) w /= static_cast<float>(load_index(a.offsets, a.off64, lo + 1) - begin);
      a.coef[k] = w;
    }
  }
  if (a.src_tile && lo >= a.seg_lo[0] && lo < a.seg_lo[a.n_features]) {
    int f = 0;
#pragma unroll 4
    for (int x = 1; x < kFillFeatures; ++x) f += (x < a.n_features && lo >= a.seg_lo[x]) ? 1 : 0;
    const int64_t t = i - begin;
    a.src_tile[k] = t < a.seq[f] ? static_cast<int32_t>(a.rbase[f] + (lo - a.seg_lo[f]) * a.seq[f] + t) : -1;
  }
  }
}

}  // namespace
}  // namespace recis_hip

using namespace recis_hip;

extern "C" {

int recis_csr_fill_lists(const int32_t* list, int64_t n, const void* offsets, int off_is64, int64_t S,
                         const void* weight, int weight_dtype, int mean, int32_t* src_pool_out, float* coef_out,
                         const int64_t* batch, const int64_t* seq, int64_t n_features, int32_t* src_tile_out,
                         void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(n >= 0 && S >= 0 && n_features >= 0, "negative size");
  if (n == 0) return RECIS_OK;
  RECIS_REQUIRE(list && offsets, "NULL argument");
  RECIS_REQUIRE(S >= 1, "occurrences without a segment");
  RECIS_REQUIRE(src_pool_out || src_tile_out, "nothing to fill");
  RECIS_REQUIRE(coef_out == nullptr || src_pool_out, "coef_out goes with src_pool_out");
  RECIS_REQUIRE(!src_pool_out || coef_out || (!weight && !mean), "coef_out is needed for weights or mean");
  RECIS_REQUIRE(weight == nullptr || dtype_size(weight_dtype), "invalid weight dtype");
  RECIS_REQUIRE(!src_tile_out || (batch && seq && n_features >= 1), "the padded gather needs its features");
  FillArgs a{};
  a.list = list;
  a.n = n;
  a.offsets = offsets;
  a.off64 = off_is64;
  a.S = S;
  a.weight = weight;
  a.wdt = weight_dtype;
  a.mean = mean;
  a.src_pool = src_pool_out;
  a.coef = coef_out;
  a.src_tile = src_tile_out;
  a.coarse_stride = (S + 1 + kFillCoarse - 1) / kFillCoarse;
  a.n_coarse = static_cast<int>((S + a.coarse_stride) / a.coarse_stride);  // offsets 0, stride, ... <= S
  const dim3 grid(static_cast<unsigned>((n + kFillPer * kBlock - 1) / (kFillPer * kBlock)));
  if (!src_tile_out) {
    a.first_group = 1;
    fill_lists_kernel<<<grid, dim3(kBlock), 0, stream>>>(a);
    RECIS_LAUNCH_CHECK();
    return RECIS_OK;
  }
  int64_t seg = 0, row = 0;
  for (int64_t f = 0; f < n_features; ++f) {
    RECIS_REQUIRE(batch[f] >= 0 && seq[f] >= 0, "negative batch/seq");
    seg += batch[f];
  }
  RECIS_REQUIRE(seg == S, "the features hold %lld segments, the offsets %lld", (long long)seg, (long long)S);
  seg = 0;
  for (int64_t f0 = 0; f0 < n_features; f0 += kFillFeatures) {  // kFillFeatures features per launch
    a.n_features = static_cast<int>(std::min<int64_t>(kFillFeatures, n_features - f0));
    a.first_group = f0 == 0;
    for (int x = 0; x < a.n_features; ++x) {
      a.seg_lo[x] = seg;
      a.seq[x] = seq[f0 + x];
      a.rbase[x] = row;
      seg += batch[f0 + x];
      row += batch[f0 + x] * seq[f0 + x];
    }
    a.seg_lo[a.n_features] = seg;
    fill_lists_kernel<<<grid, dim3(kBlock), 0, stream>>>(a);
    RECIS_LAUNCH_CHECK();
  }
  return RECIS_OK;
}

static CsrRequest one_input_request(const void* rows, int rows_dtype, int64_t n_rows, const int32_t* src,
                                    const void* coef, int coef_dtype, const int32_t* row_start,
                                    const int32_t* hot_items, int64_t hot_cap, const int64_t* counts_dev, int64_t U,
                                    int64_t D, const void* cover_offsets, int cover_is64, int64_t cover_S,
                                    void* stream_) {
  CsrRequest r;
  r.in1 = CsrInput{rows, rows_dtype, n_rows, src, coef, coef_dtype};
  r.row_start = row_start;
  r.hot_items = hot_items;
  r.hot_cap = hot_cap;
  r.counts_dev = counts_dev;
  r.U = U;
  r.D = D;
  r.cover = cover_offsets;
  r.cover64 = cover_is64;
  r.cover_S = cover_S;
  r.stream = static_cast<hipStream_t>(stream_);
  return r;
}

int recis_csr_gather_reduce(const void* rows, int rows_dtype, int64_t n_rows, const int32_t* src, const void* coef,
                            int coef_dtype, const int32_t* row_start, const int32_t* hot_items, int64_t hot_cap,
                            const int64_t* counts_dev, void* out, int out_dtype, int64_t U, int64_t D,
                            int accumulate, const void* cover_offsets, int cover_is64, int64_t cover_S,
                            void* stream_) {
  CsrRequest r = one_input_request(rows, rows_dtype, n_rows, src, coef, coef_dtype, row_start, hot_items, hot_cap,
                                   counts_dev, U, D, cover_offsets, cover_is64, cover_S, stream_);
  r.out = out;
  r.out_dtype = out_dtype;
  r.accumulate = accumulate;
  return csr_gather_reduce_run<false>(r);
}

int recis_csr_gather_reduce_mapped(const void* rows, int rows_dtype, int64_t n_rows, const int32_t* src,
                                   const void* coef, int coef_dtype, const int32_t* row_start,
                                   const int32_t* hot_items, int64_t hot_cap, const int64_t* counts_dev, void* out,
                                   int out_dtype, int64_t U, int64_t D, int accumulate, const void* cover_offsets,
                                   int cover_is64, int64_t cover_S, const int32_t* out_rows, void* stream_) {
  RECIS_REQUIRE(out_rows != nullptr || U == 0, "out_rows must not be NULL");
  CsrRequest r = one_input_request(rows, rows_dtype, n_rows, src, coef, coef_dtype, row_start, hot_items, hot_cap,
                                   counts_dev, U, D, cover_offsets, cover_is64, cover_S, stream_);
  r.out = out;
  r.out_dtype = out_dtype;
  r.accumulate = accumulate;
  r.out_rows = out_rows;
  return csr_gather_reduce_run<false>(r);
}

int recis_csr_gather_reduce_parts(const void* const* part_rows, const int64_t* part_counts, int n_parts,
                                  int rows_dtype, const int32_t* src, const int32_t* row_start,
                                  const int32_t* hot_items, int64_t hot_cap, const int64_t* counts_dev, void* out,
                                  int64_t U, int64_t D, int accumulate, void* stream_) {
  RECIS_REQUIRE(n_parts >= 1 && n_parts <= kMaxParts, "1 to %d parts (got %d)", kMaxParts, n_parts);
  RECIS_REQUIRE(part_rows && part_counts, "NULL argument");
  int64_t n_rows = 0;
  for (int f = 0; f < n_parts; ++f) {
    RECIS_REQUIRE(part_counts[f] >= 0 && (part_rows[f] != nullptr || part_counts[f] == 0), "bad part %d", f);
    n_rows += part_counts[f];
  }
  CsrRequest r = one_input_request(nullptr, rows_dtype, n_rows, src, nullptr, 0, row_start, hot_items, hot_cap,
                                   counts_dev, U, D, nullptr, 0, 0, stream_);
  r.part_rows = part_rows;
  r.part_counts = part_counts;
  r.n_parts = n_parts;
  r.out = out;
  r.out_dtype = RECIS_F32;
  r.accumulate = accumulate;
  return csr_gather_reduce_run<false>(r);
}

int recis_csr_gather_reduce_adamw(const void* rows, int rows_dtype, int64_t n_rows, const int32_t* src,
                                  const void* coef, int coef_dtype, const int32_t* row_start,
                                  const int32_t* hot_items, int64_t hot_cap, const int64_t* counts_dev, int64_t U,
                                  int64_t D, const void* cover_offsets, int cover_is64, int64_t cover_S,
                                  const int64_t* row_index, void* const* emb_blocks_dev,
                                  void* const* exp_avg_blocks_dev, void* const* exp_avg_sq_blocks_dev,
                                  int64_t n_blocks, int64_t block_size, int64_t row_pitch_bytes, int row_dtype,
                                  void* beta1_t, void* beta2_t, int beta_is_f64, double lr, double beta1, double beta2,
                                  double weight_decay, double eps, void* stream_) {
  RECIS_REQUIRE(beta1_t != nullptr && beta2_t != nullptr, "beta1_t / beta2_t must not be NULL");
  FuseArgs f{};
  if (U > 0) {
    if (int rc = fill_fuse_args(f, row_index, emb_blocks_dev, exp_avg_blocks_dev, exp_avg_sq_blocks_dev, true, n_blocks,
                                block_size, row_pitch_bytes, D, row_dtype))
      return rc;
  }
  CsrRequest r = one_input_request(rows, rows_dtype, n_rows, src, coef, coef_dtype, row_start, hot_items, hot_cap,
                                   counts_dev, U, D, cover_offsets, cover_is64, cover_S, stream_);
  r.out_dtype = row_dtype;
  r.epi = kEpiAdam;
  r.fuse = &f;
  return run_with_alpha<false>(r, f, beta1_t, beta2_t, beta_is_f64, lr, beta1, beta2, weight_decay, eps);
}

int recis_csr_gather_reduce_adagrad(const void* rows, int rows_dtype, int64_t n_rows, const int32_t* src,
                                    const void* coef, int coef_dtype, const int32_t* row_start,
                                    const int32_t* hot_items, int64_t hot_cap, const int64_t* counts_dev, int64_t U,
                                    int64_t D, const void* cover_offsets, int cover_is64, int64_t cover_S,
                                    const int64_t* row_index, void* const* emb_blocks_dev,
                                    void* const* accum_blocks_dev, int64_t n_blocks, int64_t block_size,
                                    int64_t row_pitch_bytes, int row_dtype, double lr, double eps, void* stream_) {
  if (U == 0) return RECIS_OK;
  FuseArgs f;
  if (int rc = fill_fuse_args(f, row_index, emb_blocks_dev, accum_blocks_dev, nullptr, false, n_blocks, block_size,
                              row_pitch_bytes, D, row_dtype))
    return rc;
  f.lr = static_cast<float>(lr);
  f.eps = static_cast<float>(eps);
  CsrRequest r = one_input_request(rows, rows_dtype, n_rows, src, coef, coef_dtype, row_start, hot_items, hot_cap,
                                   counts_dev, U, D, cover_offsets, cover_is64, cover_S, stream_);
  r.out_dtype = row_dtype;
  r.epi = kEpiAdagrad;
  r.fuse = &f;
  return csr_gather_reduce_run<false>(r);
}


int recis_csr_expand_rows(const void* rows, void* const* emb_blocks_dev, int64_t n_blocks, int64_t block_rows,
                          int64_t row_pitch_bytes, const int64_t* row_index, int rows_dtype, const void* weight, int weight_dtype,
                          const int32_t* row_start, const int32_t* dst, const int32_t* hot_items, int64_t hot_cap,
                          const int64_t* counts_dev, void* out, int out_dtype, int64_t U, int64_t n_out, int64_t D,
                          void* stream_) {
  return recis_csr_expand_rows_stamped(rows, emb_blocks_dev, n_blocks, block_rows, row_pitch_bytes, row_index, rows_dtype, weight,
                                       weight_dtype, row_start, dst, hot_items, hot_cap, counts_dev, out, out_dtype, U,
                                       n_out, D, nullptr, nullptr, stream_);
}

int recis_csr_expand_rows_stamped(const void* rows, void* const* emb_blocks_dev, int64_t n_blocks, int64_t block_rows,
                                  int64_t row_pitch_bytes, const int64_t* row_index, int rows_dtype, const void* weight, int weight_dtype,
                                  const int32_t* row_start, const int32_t* dst, const int32_t* hot_items,
                                  int64_t hot_cap, const int64_t* counts_dev, void* out, int out_dtype, int64_t U,
                                  int64_t n_out, int64_t D, void* const* stamp_blocks_dev,
                                  const int64_t* stamp_value_dev, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE((stamp_blocks_dev == nullptr) == (stamp_value_dev == nullptr), "stamp blocks and stamp value go together");
  RECIS_REQUIRE(stamp_blocks_dev == nullptr || emb_blocks_dev != nullptr, "rows are stamped in a block list only");
  RECIS_REQUIRE(U >= 0 && n_out >= 0, "negative size");
  RECIS_REQUIRE(D >= 1 && D <= 8192, "embedding dim %lld out of range", (long long)D);
  if (U == 0 || n_out == 0) return RECIS_OK;
  const bool blk = emb_blocks_dev != nullptr;
  RECIS_REQUIRE(row_start && dst && out && counts_dev, "NULL argument");
  RECIS_REQUIRE(blk ? (row_index != nullptr && n_blocks >= 1 && block_rows >= 1) : rows != nullptr,
                "rows: a dense array or a block list with row_index");
  RECIS_REQUIRE(hot_cap == 0 || hot_items, "hot_items must not be NULL");
  const int in_sz = dtype_size(rows_dtype), out_sz = dtype_size(out_dtype);
  RECIS_REQUIRE(in_sz && out_sz, "invalid dtype");
  RECIS_REQUIRE(weight == nullptr || dtype_size(weight_dtype), "invalid weight dtype");
  // block bases are allocator-aligned; a dense array brings its own alignment
  const int vb_in = pick_vec_bytes(D * in_sz, blk ? 0 : reinterpret_cast<uintptr_t>(rows));
  const int vb_out = pick_vec_bytes(D * out_sz, reinterpret_cast<uintptr_t>(out));
  const int vec = std::max(1, std::min(vb_in / in_sz, vb_out / out_sz));
  ExpArgs a;
  a.row_start = row_start;
  a.dst = dst;
  a.weight = weight;
  a.wdt = weight_dtype;
  a.U = U;
  a.n_out = n_out;
  a.D = static_cast<int>(D);
  a.lpr_log2 = std::min(6, ilog2_ceil((D + vec - 1) / vec));
  a.err = device_error_word(current_device());
  RECIS_REQUIRE(a.err != nullptr, "could not reach the device error word");
  a.row_index = row_index;
  a.blocks = emb_blocks_dev;
  a.block_rows = block_rows;
  a.pitch = blk ? pitch_elements(row_pitch_bytes, D, in_sz, vb_in) : D;
  RECIS_REQUIRE(a.pitch >= D, "row pitch of %lld bytes does not fit rows of %lld elements", (long long)row_pitch_bytes,
                (long long)D);
  a.n_blocks = n_blocks;
  a.hot_len = hot_cap > 0 ? kHotLen : INT_MAX;
  a.hot_items = hot_items;
  a.counts = counts_dev;
  a.hot_cap = hot_cap;
  a.stamp_blocks = stamp_blocks_dev;
  a.stamp_value = stamp_value_dev;
  const int rows_per_block = kExpandRows * (kBlock >> a.lpr_log2);
  RECIS_REQUIRE(U <= INT32_MAX, "more unique rows than 32-bit list entries name");
  // the cold workgroups stride over the batches of rows: as many as the device holds at once
  a.cold_blocks = std::min<int64_t>((U + rows_per_block - 1) / rows_per_block, cold_grid_blocks());
  const int64_t hot_blocks = hot_cap > 0 ? std::min<int64_t>(hot_cap, 4096) : 0;
  const dim3 grid(static_cast<unsigned>(a.cold_blocks + hot_blocks));
  auto with_types = [&](auto tin, auto tout) {
    using TIn = decltype(tin);
    using TOut = decltype(tout);
    return dispatch_vec(vec, [&](auto vtag) {
      constexpr int VEC = decltype(vtag)::value;
      if constexpr (VEC * sizeof(TIn) > 16 || VEC * sizeof(TOut) > 16) {
        return fail(RECIS_ERR_ARG, "internal: vector too wide");
      } else {
        RECIS_TIME_KERNEL("csr_expand_kernel", stream)
        if (blk && stream_table_rows(RowBlocks{n_blocks, block_rows, a.D, a.pitch}, sizeof(TIn), 1))
          csr_expand_kernel<TIn, TOut, VEC, true><<<grid, dim3(kBlock), 0, stream>>>(nullptr, static_cast<TOut*>(out), a);
        else if (blk)
          csr_expand_kernel<TIn, TOut, VEC, true, false><<<grid, dim3(kBlock), 0, stream>>>(nullptr,
                                                                                           static_cast<TOut*>(out), a);
        else
          csr_expand_kernel<TIn, TOut, VEC, false><<<grid, dim3(kBlock), 0, stream>>>(static_cast<const TIn*>(rows),
                                                                                    static_cast<TOut*>(out), a);
        RECIS_LAUNCH_CHECK();
        return RECIS_OK;
      }
    });
  };
  if (rows_dtype == RECIS_F32 && out_dtype == RECIS_F32) return with_types(float{}, float{});
  if (rows_dtype == RECIS_BF16 && out_dtype == RECIS_BF16) return with_types(bf16_t{}, bf16_t{});
  if (rows_dtype == RECIS_F16 && out_dtype == RECIS_F16) return with_types(f16_t{}, f16_t{});
  if (rows_dtype == RECIS_BF16 && out_dtype == RECIS_F32) return with_types(bf16_t{}, float{});
  if (rows_dtype == RECIS_F16 && out_dtype == RECIS_F32) return with_types(f16_t{}, float{});
  return fail(RECIS_ERR_ARG, "unsupported dtype pair (rows=%d, out=%d)", rows_dtype, out_dtype);
}

}  // extern "C"
