// Batch plan for gfx950: dedup of a batch of ids together with the transposed index
// (for every unique id, the list of occurrences that carry it).
//
// The reference scatters gradients back to unique rows with one global atomic per
// element (csrc/ops/embedding_segment_reduce_kernel.cu:79-120, segment_ops_kernel.cu:133-165)
// and dedups with a radix sort (csrc/ops/ids_partition_kernel.cu:86-131). On MI355X fp32
// atomics run at a few percent of HBM speed and ids of low-cardinality features repeat
// tens of thousands of times per batch, so this build never scatters rows: the plan below
// groups the occurrences by unique id once per batch, after which the gradient of a
// unique row is a gather-reduce over its own list, written once.
//
//   insert   one workgroup dedups its 1024 ids in an LDS hash first (LDS atomics), so an id
//            repeated k times in the block costs ONE probe of the global scratch set, one
//            atomicMin (first occurrence) and one atomicAdd (occurrence count, whose return
//            value hands every occurrence its rank inside the id's list)
//   unique   first occurrences are ranked in input order by a scan: unique ids come out in
//            order of first occurrence (deterministic)
//   lists    exclusive scan of the per-unique counts -> row_start; occurrence i goes to
//            list[row_start[u] + rank_i]
//   hot      unique ids with more than kHotLen occurrences are listed as (row, chunk) work
//            items for a workgroup-per-chunk reduction; everything else is one small team
//            of lanes per row
#include <hip/hip_runtime.h>

#include <algorithm>
#include <type_traits>

#include "common.cuh"

namespace recis_hip {
namespace {

constexpr int kPlanBlock = 1024;
constexpr int kLdsSlots = 2048;  // LDS hash entries per workgroup (load <= 1/2)
constexpr int64_t kSetEmpty = -1;
constexpr int32_t kNoPos = 0x7fffffff;
constexpr int kHotLen = 256;      // rows with more occurrences than this are "hot"
constexpr int kHotChunk = 8192;   // occurrences per hot work item

__device__ __forceinline__ uint64_t mix_id(int64_t key) {
  uint64_t x = static_cast<uint64_t>(key);
  x ^= x >> 33;
  x *= 0xff51afd7ed558ccdULL;
  x ^= x >> 33;
  x *= 0xc4ceb9fe1a85ec53ULL;
  x ^= x >> 33;
  return x;
}

// One 16-byte slot of the global scratch set: everything a unique id needs sits in one
// cache line, so the probe, the first-occurrence atomicMin and the count atomicAdd of an id
// touch HBM once. `cnt` is reused for the unique index once the count has been consumed.
struct alignas(16) PSlot {
  int64_t key;
  int32_t minpos;
  int32_t cnt;
};

__global__ void __launch_bounds__(kBlock)
plan_init_kernel(PSlot* tab, int64_t slots, int64_t* counts) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
  PSlot empty;
  empty.key = kSetEmpty;
  empty.minpos = kNoPos;
  empty.cnt = 0;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; i < slots; i += stride) tab[i] = empty;
  if (blockIdx.x == 0 && threadIdx.x < 2) counts[threadIdx.x] = 0;
}

// Global scratch set of `cap` probed slots (any size: the start slot is the high half of
// hash * cap); slot `cap` is reserved for the id that equals the empty marker.
__device__ __forceinline__ uint32_t global_slot(PSlot* tab, uint64_t cap, int64_t key) {
  if (key == kSetEmpty) return static_cast<uint32_t>(cap);
  uint64_t p = __umul64hi(mix_id(key), cap);
  for (;;) {
    // plain (L1-cacheable) load: a stale "empty" is corrected by the CAS, a slot never
    // changes once it holds a key
    int64_t k = tab[p].key;
    if (k == kSetEmpty) {
      k = static_cast<int64_t>(atomicCAS(reinterpret_cast<unsigned long long*>(&tab[p].key),
                                         static_cast<unsigned long long>(kSetEmpty),
                                         static_cast<unsigned long long>(key)));
      if (k == kSetEmpty) break;
    }
    if (k == key) break;
    if (++p == cap) p = 0;  // cap >= 2n: an empty slot always exists
  }
  return static_cast<uint32_t>(p);
}

__global__ void __launch_bounds__(kPlanBlock)
plan_insert_kernel(PSlot* __restrict__ tab, uint64_t cap, const int64_t* __restrict__ ids, int64_t n,
                   int32_t* __restrict__ slotpos, int32_t* __restrict__ rank) {
  __shared__ int64_t l_key[kLdsSlots + 1];
  __shared__ int32_t l_min[kLdsSlots + 1];
  __shared__ int32_t l_cnt[kLdsSlots + 1];
  __shared__ uint32_t l_slot[kLdsSlots + 1];
  __shared__ int32_t l_base[kLdsSlots + 1];
  const int tid = threadIdx.x;
  for (int e = tid; e <= kLdsSlots; e += kPlanBlock) {
    l_key[e] = kSetEmpty;
    l_min[e] = kNoPos;
    l_cnt[e] = 0;
  }
  __syncthreads();
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kPlanBlock + tid;
  const bool live = i < n;
  int64_t key = 0;
  int e = 0, local_rank = 0;
  if (live) {
    key = ids[i];
    if (key == kSetEmpty) {
      e = kLdsSlots;
    } else {
      e = static_cast<int>(mix_id(key) >> 40) & (kLdsSlots - 1);
      for (;;) {
        int64_t k = l_key[e];
        if (k == kSetEmpty) {
          k = static_cast<int64_t>(atomicCAS(reinterpret_cast<unsigned long long*>(&l_key[e]),
                                             static_cast<unsigned long long>(kSetEmpty),
                                             static_cast<unsigned long long>(key)));
          if (k == kSetEmpty) break;
        }
        if (k == key) break;
        e = (e + 1) & (kLdsSlots - 1);  // at most 1024 distinct ids in 2048 entries
      }
    }
    local_rank = atomicAdd(&l_cnt[e], 1);
    atomicMin(&l_min[e], tid);
  }
  __syncthreads();
  if (live && l_min[e] == tid) {  // the block's first occurrence speaks for all of them
    const uint32_t p = global_slot(tab, cap, key);
    atomicMin(&tab[p].minpos, static_cast<int32_t>(i));
    l_base[e] = atomicAdd(&tab[p].cnt, l_cnt[e]);
    l_slot[e] = p;
  }
  __syncthreads();
  if (live) {
    slotpos[i] = static_cast<int32_t>(l_slot[e]);
    rank[i] = l_base[e] + local_rank;
  }
}

__device__ __forceinline__ void block_rank256(bool flag, int& rank, int& total) {
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
plan_first_count_kernel(const PSlot* __restrict__ tab, const int32_t* __restrict__ slotpos, int64_t n,
                        int32_t* __restrict__ block_counts) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  const bool first = i < n && tab[slotpos[i]].minpos == static_cast<int32_t>(i);
  int rank, total;
  block_rank256(first, rank, total);
  if (threadIdx.x == 0) block_counts[blockIdx.x] = total;
}

// Single-workgroup exclusive scan of up to millions of int32 partials (in place), total out.
__global__ void __launch_bounds__(1024)
scan_partials_kernel(int32_t* __restrict__ v, int64_t n, int64_t* __restrict__ total_out) {
  __shared__ int64_t partial[1024];
  const int t = threadIdx.x;
  const int64_t per = (n + 1023) / 1024;
  const int64_t lo = std::min<int64_t>(t * per, n), hi = std::min<int64_t>(lo + per, n);
  int64_t sum = 0;
  for (int64_t b = lo; b < hi; ++b) sum += v[b];
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
    int32_t c = v[b];
    v[b] = static_cast<int32_t>(run);
    run += c;
  }
  if (t == 1023 && total_out) total_out[0] = partial[1023];
}

__global__ void __launch_bounds__(kBlock)
plan_emit_unique_kernel(const int64_t* __restrict__ ids, PSlot* __restrict__ tab,
                        const int32_t* __restrict__ slotpos, int64_t n,
                        const int32_t* __restrict__ block_prefix, int64_t* __restrict__ unique_out,
                        int32_t* __restrict__ row_start) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  const int32_t sp = i < n ? slotpos[i] : 0;
  const bool first = i < n && tab[sp].minpos == static_cast<int32_t>(i);
  int rank, total;
  block_rank256(first, rank, total);
  if (!first) return;
  const int32_t u = block_prefix[blockIdx.x] + rank;
  unique_out[u] = ids[i];
  row_start[u] = tab[sp].cnt;  // counts for now; scanned in place afterwards
  tab[sp].cnt = u;             // from here on the field holds the unique index
}

// Device-wide exclusive scan of row_start[0 .. U) (U read from device memory), three phases
// over tiles of 1024; entries U .. n are set to the grand total.
__global__ void __launch_bounds__(1024)
tile_sum_kernel(const int32_t* __restrict__ v, const int64_t* __restrict__ count, int32_t* __restrict__ tile_sums) {
  __shared__ int wave_sums[16];
  const int64_t U = count[0];
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 1024 + threadIdx.x;
  int x = i < U ? v[i] : 0;
  for (int off = 32; off > 0; off >>= 1) x += __shfl_down(x, off, kWave);
  if ((threadIdx.x & 63) == 0) wave_sums[threadIdx.x >> 6] = x;
  __syncthreads();
  if (threadIdx.x == 0) {
    int s = 0;
    for (int w = 0; w < 16; ++w) s += wave_sums[w];
    tile_sums[blockIdx.x] = s;
  }
}

__global__ void __launch_bounds__(1024)
tile_scan_kernel(int32_t* __restrict__ v, const int64_t* __restrict__ count, const int32_t* __restrict__ tile_prefix,
                 int64_t n_plus_1, int32_t total) {
  __shared__ int wave_sums[16];
  const int64_t U = count[0];
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 1024 + threadIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int x = i < U ? v[i] : 0;
  int incl = x;
  for (int off = 1; off < 64; off <<= 1) {
    int y = __shfl_up(incl, off, kWave);
    if (lane >= off) incl += y;
  }
  if (lane == 63) wave_sums[wave] = incl;
  __syncthreads();
  int base = tile_prefix[blockIdx.x];
  for (int w = 0; w < wave; ++w) base += wave_sums[w];
  if (i < n_plus_1) v[i] = i < U ? base + incl - x : total;
}

__global__ void __launch_bounds__(kBlock)
plan_emit_lists_kernel(const int32_t* __restrict__ slotpos, const int32_t* __restrict__ rank,
                       const PSlot* __restrict__ tab, const int32_t* __restrict__ row_start, int64_t n,
                       int32_t* __restrict__ inverse, int32_t* __restrict__ list, int32_t* __restrict__ pos_out) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (i >= n) return;
  const int32_t u = tab[slotpos[i]].cnt;
  const int32_t pos = row_start[u] + rank[i];
  inverse[i] = u;
  list[pos] = static_cast<int32_t>(i);
  if (pos_out) pos_out[i] = pos;
}

// (row, chunk) work items for rows with more than kHotLen occurrences.
__global__ void __launch_bounds__(kBlock)
plan_hot_items_kernel(const int32_t* __restrict__ row_start, int64_t* __restrict__ counts,
                      int32_t* __restrict__ hot_items, int64_t hot_cap) {
  const int64_t U = counts[0];
  const int64_t u = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (u >= U) return;
  const int32_t len = row_start[u + 1] - row_start[u];
  if (len <= kHotLen) return;
  const int n_items = (len + kHotChunk - 1) / kHotChunk;
  const int64_t base = static_cast<int64_t>(atomicAdd(reinterpret_cast<unsigned long long*>(&counts[1]),
                                                      static_cast<unsigned long long>(n_items)));
  for (int k = 0; k < n_items; ++k) {
    if (base + k < hot_cap) {
      hot_items[2 * (base + k)] = static_cast<int32_t>(u);
      hot_items[2 * (base + k) + 1] = k;
    }
  }
}

// ---------------------------------------------------------------- consumers
__device__ __forceinline__ float load_coef(const void* w, int wdt, int64_t i) {
  if (wdt == RECIS_F32) return static_cast<const float*>(w)[i];
  if (wdt == RECIS_BF16) return to_float(static_cast<const bf16_t*>(w)[i]);
  return to_float(static_cast<const f16_t*>(w)[i]);
}

struct CsrArgs {
  const int32_t* row_start;  // [U + 1]
  const int32_t* src;        // [n] input row per list entry (negative = skip)
  const void* coef;          // [n] per list entry, or NULL
  int coef_dt;
  int64_t U, n_rows;
  int D;
  int lpr_log2;
  int accumulate;
  int* err;
};

// One group of LPR lanes per unique row (cold rows); hot rows are cleared here and summed by
// csr_hot_kernel.
template <typename TIn, typename TOut, int VEC>
__global__ void __launch_bounds__(kBlock)
csr_cold_kernel(const TIn* __restrict__ rows, TOut* __restrict__ out, CsrArgs a) {
  const int rows_per_block = kBlock >> a.lpr_log2;
  const int64_t u = static_cast<int64_t>(blockIdx.x) * rows_per_block + (threadIdx.x >> a.lpr_log2);
  if (u >= a.U) return;
  const int cl = threadIdx.x & ((1 << a.lpr_log2) - 1);
  const int32_t start = a.row_start[u], end = a.row_start[u + 1];
  const bool hot = end - start > kHotLen;
  const int D = a.D;

  auto fetch = [&](int32_t k, int c0, float (&v)[VEC], float& w) {
    const int32_t s = a.src[k];
    w = a.coef ? load_coef(a.coef, a.coef_dt, k) : 1.0f;
    if (s < 0 || static_cast<int64_t>(s) >= a.n_rows) {
      if (s >= 0) raise_device_error(a.err, RECIS_DEVERR_INDEX_RANGE);
#pragma unroll
      for (int j = 0; j < VEC; ++j) v[j] = 0.f;
      w = 0.f;
      return;
    }
    load_pack<TIn, VEC>(rows + static_cast<int64_t>(s) * D + c0, v);
  };

  for (int c0 = cl * VEC; c0 < D; c0 += VEC << a.lpr_log2) {
    float acc[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) acc[j] = 0.f;
    if (!hot) {
      int32_t k = start;
      for (; k + 3 < end; k += 4) {
        float v0[VEC], v1[VEC], v2[VEC], v3[VEC];
        float w0, w1, w2, w3;
        fetch(k, c0, v0, w0);
        fetch(k + 1, c0, v1, w1);
        fetch(k + 2, c0, v2, w2);
        fetch(k + 3, c0, v3, w3);
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          acc[j] = fmaf(v0[j], w0, acc[j]);
          acc[j] = fmaf(v1[j], w1, acc[j]);
          acc[j] = fmaf(v2[j], w2, acc[j]);
          acc[j] = fmaf(v3[j], w3, acc[j]);
        }
      }
      for (; k < end; ++k) {
        float v0[VEC];
        float w0;
        fetch(k, c0, v0, w0);
#pragma unroll
        for (int j = 0; j < VEC; ++j) acc[j] = fmaf(v0[j], w0, acc[j]);
      }
    }
    TOut* dst = out + u * D + c0;
    if (a.accumulate) {
      if (hot) continue;  // keep what is there; the hot kernel adds to it
      float old[VEC];
      load_pack<TOut, VEC>(dst, old);
#pragma unroll
      for (int j = 0; j < VEC; ++j) acc[j] += old[j];
    }
    store_pack<TOut, VEC>(dst, acc);
  }
}

// One workgroup per (hot row, chunk): row groups stride over the chunk, partial sums are
// combined through LDS and added to the (cleared) output row with a handful of atomics.
template <typename TIn, int VEC>
__global__ void __launch_bounds__(kPlanBlock)
csr_hot_kernel(const TIn* __restrict__ rows, float* __restrict__ out, CsrArgs a,
               const int32_t* __restrict__ hot_items, const int64_t* __restrict__ counts, int64_t hot_cap) {
  extern __shared__ float s_part[];  // [waves][D]
  int64_t n_items = counts[1];
  if (n_items > hot_cap) n_items = hot_cap;
  const int D = a.D;
  const int groups = kPlanBlock >> a.lpr_log2;
  const int g = threadIdx.x >> a.lpr_log2;
  const int cl = threadIdx.x & ((1 << a.lpr_log2) - 1);
  const int wave = threadIdx.x / kWave;
  constexpr int n_waves = kPlanBlock / kWave;
  for (int64_t item = blockIdx.x; item < n_items; item += gridDim.x) {
    const int32_t u = hot_items[2 * item];
    const int32_t chunk = hot_items[2 * item + 1];
    const int32_t start = a.row_start[u] + chunk * kHotChunk;
    const int32_t end = min(a.row_start[u + 1], start + kHotChunk);
    for (int c0 = cl * VEC; c0 < D; c0 += VEC << a.lpr_log2) {
      float acc[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) acc[j] = 0.f;
      for (int32_t k = start + g; k < end; k += groups) {
        const int32_t s = a.src[k];
        if (s < 0 || static_cast<int64_t>(s) >= a.n_rows) continue;
        const float w = a.coef ? load_coef(a.coef, a.coef_dt, k) : 1.0f;
        float v[VEC];
        load_pack<TIn, VEC>(rows + static_cast<int64_t>(s) * D + c0, v);
#pragma unroll
        for (int j = 0; j < VEC; ++j) acc[j] = fmaf(v[j], w, acc[j]);
      }
      // groups of one wave share columns when lpr < 64: fold them with shuffles
      for (int off = 1 << a.lpr_log2; off < kWave; off <<= 1) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) acc[j] += __shfl_xor(acc[j], off, kWave);
      }
      if ((threadIdx.x & (kWave - 1)) < (1 << a.lpr_log2)) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) s_part[wave * D + c0 + j] = acc[j];
      }
    }
    __syncthreads();
    for (int d = threadIdx.x; d < D; d += kPlanBlock) {
      float s = 0.f;
      for (int w = 0; w < n_waves; ++w) s += s_part[w * D + d];
      unsafeAtomicAdd(out + static_cast<int64_t>(u) * D + d, s);
    }
    __syncthreads();
  }
}

// src / coef of every list entry for pooled segments: occurrence i of segment s gets
// src = s and coef = w_i (divided by the segment length for mean).
__global__ void __launch_bounds__(kBlock)
fill_pool_kernel(const void* __restrict__ offsets, int off64, int64_t S, int64_t n, const void* __restrict__ weight,
                 int wdt, const int32_t* __restrict__ pos, int mean, int32_t* __restrict__ src,
                 float* __restrict__ coef) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (i >= n) return;
  // segment of occurrence i: largest s with offsets[s] <= i
  int64_t lo = 0, hi = S;
  const int64_t first = load_index(offsets, off64, 0), last = load_index(offsets, off64, S);
  const int32_t p = pos[i];
  if (i < first || i >= last) {
    src[p] = -1;
    if (coef) coef[p] = 0.f;
    return;
  }
  while (hi - lo > 1) {
    const int64_t mid = (lo + hi) >> 1;
    if (load_index(offsets, off64, mid) <= i)
      lo = mid;
    else
      hi = mid;
  }
  src[p] = static_cast<int32_t>(lo);
  if (coef) {
    float w = weight ? load_coef(weight, wdt, i) : 1.0f;
    if (mean) w /= static_cast<float>(load_index(offsets, off64, lo + 1) - load_index(offsets, off64, lo));
    coef[p] = w;
  }
}

// src of every list entry for the padded gather of one feature: occurrence t of sample b
// maps to padded row rbase + b * seq + t, or to "skip" when t >= seq.
__global__ void __launch_bounds__(kBlock)
fill_tile_kernel(const void* __restrict__ offsets, int off64, int64_t batch, int64_t seq, int64_t rbase,
                 const int32_t* __restrict__ pos, int32_t* __restrict__ src) {
  const int64_t first = load_index(offsets, off64, 0), last = load_index(offsets, off64, batch);
  const int64_t i = first + static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (i >= last) return;
  int64_t lo = 0, hi = batch;
  while (hi - lo > 1) {
    const int64_t mid = (lo + hi) >> 1;
    if (load_index(offsets, off64, mid) <= i)
      lo = mid;
    else
      hi = mid;
  }
  const int64_t t = i - load_index(offsets, off64, lo);
  src[pos[i]] = t < seq ? static_cast<int32_t>(rbase + lo * seq + t) : -1;
}

template <typename F>
int dispatch_vec(int vec, F&& f) {
  switch (vec) {
    case 8: return f(std::integral_constant<int, 8>{});
    case 4: return f(std::integral_constant<int, 4>{});
    case 2: return f(std::integral_constant<int, 2>{});
    case 1: return f(std::integral_constant<int, 1>{});
    default: return fail(RECIS_ERR_ARG, "unsupported vector width %d", vec);
  }
}

}  // namespace
}  // namespace recis_hip

using namespace recis_hip;

extern "C" {

int recis_unique_plan(const int64_t* ids, int64_t n, int64_t* unique_out, int32_t* inverse_out,
                      int32_t* row_start_out, int32_t* list_out, int32_t* pos_out, int32_t* hot_items_out,
                      int64_t hot_cap, int64_t* counts_out_dev, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(n >= 0 && n < (int64_t(1) << 30), "n out of range: %lld", (long long)n);
  RECIS_REQUIRE(counts_out_dev && row_start_out, "counts_out_dev / row_start_out must not be NULL");
  RECIS_REQUIRE(hot_cap == 0 || (hot_items_out && hot_cap >= n / kHotLen + n / kHotChunk + 2),
                "hot_items_out must hold at least n/%d + n/%d + 2 items", kHotLen, kHotChunk);
  RECIS_REQUIRE(n == 0 || (ids && unique_out && inverse_out && list_out), "NULL argument");
  const int64_t cap = std::max<int64_t>(1024, 2 * n);
  const int64_t slots = cap + 1;
  const int64_t nb = std::max<int64_t>(1, (n + kBlock - 1) / kBlock);
  const int64_t n_tiles = (n + 1 + 1023) / 1024;
  // workspace: tab[slots] | slotpos[n] | rank[n] | block_counts[nb] | tile sums
  const size_t bytes = sizeof(PSlot) * slots + sizeof(int32_t) * (2 * n + nb + n_tiles) + 256;
  void* ws = nullptr;
  if (int rc = get_workspace(stream, bytes, &ws)) return rc;
  PSlot* tab = static_cast<PSlot*>(ws);
  int32_t* slotpos = reinterpret_cast<int32_t*>(tab + slots);
  int32_t* rank = slotpos + n;
  int32_t* block_counts = rank + n;
  int32_t* tile_sums = block_counts + nb;

  RECIS_TIME_KERNEL("plan_init_kernel", stream)

  plan_init_kernel<<<dim3(std::min<int64_t>((slots + kBlock - 1) / kBlock, 256 * 16)), dim3(kBlock), 0, stream>>>(
      tab, slots, counts_out_dev);
  RECIS_LAUNCH_CHECK();
  if (n > 0) {
    RECIS_TIME_KERNEL("plan_insert_kernel", stream)
    plan_insert_kernel<<<dim3((n + kPlanBlock - 1) / kPlanBlock), dim3(kPlanBlock), 0, stream>>>(
        tab, static_cast<uint64_t>(cap), ids, n, slotpos, rank);
    RECIS_LAUNCH_CHECK();
    RECIS_TIME_KERNEL("plan_first_count_kernel", stream)
    plan_first_count_kernel<<<dim3(nb), dim3(kBlock), 0, stream>>>(tab, slotpos, n, block_counts);
    RECIS_LAUNCH_CHECK();
  }
  scan_partials_kernel<<<1, 1024, 0, stream>>>(block_counts, n > 0 ? nb : 0, counts_out_dev);
  RECIS_LAUNCH_CHECK();
  if (n > 0) {
    RECIS_TIME_KERNEL("plan_emit_unique_kernel", stream)
    plan_emit_unique_kernel<<<dim3(nb), dim3(kBlock), 0, stream>>>(ids, tab, slotpos, n, block_counts, unique_out,
                                                                   row_start_out);
    RECIS_LAUNCH_CHECK();
  }
  tile_sum_kernel<<<dim3(n_tiles), dim3(1024), 0, stream>>>(row_start_out, counts_out_dev, tile_sums);
  RECIS_LAUNCH_CHECK();
  scan_partials_kernel<<<1, 1024, 0, stream>>>(tile_sums, n_tiles, nullptr);
  RECIS_LAUNCH_CHECK();
  tile_scan_kernel<<<dim3(n_tiles), dim3(1024), 0, stream>>>(row_start_out, counts_out_dev, tile_sums, n + 1,
                                                            static_cast<int32_t>(n));
  RECIS_LAUNCH_CHECK();
  if (n > 0) {
    RECIS_TIME_KERNEL("plan_emit_lists_kernel", stream)
    plan_emit_lists_kernel<<<dim3(nb), dim3(kBlock), 0, stream>>>(slotpos, rank, tab, row_start_out, n,
                                                                  inverse_out, list_out, pos_out);
    RECIS_LAUNCH_CHECK();
    if (hot_cap > 0) {
      plan_hot_items_kernel<<<dim3(nb), dim3(kBlock), 0, stream>>>(row_start_out, counts_out_dev, hot_items_out,
                                                                   hot_cap);
      RECIS_LAUNCH_CHECK();
    }
  }
  return RECIS_OK;
}

int recis_csr_fill_pool(const void* offsets, int off_is64, int64_t S, int64_t n, const void* weight,
                        int weight_dtype, const int32_t* pos, int mean, int32_t* src_out, float* coef_out,
                        void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(n >= 0 && S >= 0, "negative size");
  if (n == 0) return RECIS_OK;
  RECIS_REQUIRE(offsets && pos && src_out, "NULL argument");
  RECIS_REQUIRE(S >= 1, "occurrences without a segment");
  RECIS_REQUIRE(coef_out || (!weight && !mean), "coef_out is needed for weights or mean");
  RECIS_REQUIRE(weight == nullptr || dtype_size(weight_dtype), "invalid weight dtype");
  fill_pool_kernel<<<dim3((n + kBlock - 1) / kBlock), dim3(kBlock), 0, stream>>>(
      offsets, off_is64, S, n, weight, weight_dtype, pos, mean, src_out, coef_out);
  RECIS_LAUNCH_CHECK();
  return RECIS_OK;
}

int recis_csr_fill_tile(const int64_t* batch, const int64_t* seq, int64_t n_features, const void* offsets,
                        int off_is64, int64_t n, const int32_t* pos, int32_t* src_out, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(n_features >= 0 && n >= 0, "negative size");
  if (n_features == 0 || n == 0) return RECIS_OK;
  RECIS_REQUIRE(batch && seq && offsets && pos && src_out, "NULL argument");
  int64_t obase = 0, rbase = 0;
  const int osz = off_is64 ? 8 : 4;
  for (int64_t f = 0; f < n_features; ++f) {
    RECIS_REQUIRE(batch[f] >= 0 && seq[f] >= 0, "negative batch/seq");
    if (batch[f] > 0) {
      // upper bound of this feature's occurrences is n; the kernel stops at its last offset
      const void* off_f = static_cast<const char*>(offsets) + obase * osz;
      fill_tile_kernel<<<dim3((n + kBlock - 1) / kBlock), dim3(kBlock), 0, stream>>>(off_f, off_is64, batch[f],
                                                                                    seq[f], rbase, pos, src_out);
      RECIS_LAUNCH_CHECK();
    }
    obase += batch[f];
    rbase += batch[f] * seq[f];
  }
  return RECIS_OK;
}

int recis_csr_gather_reduce(const void* rows, int rows_dtype, int64_t n_rows, const int32_t* src, const void* coef,
                            int coef_dtype, const int32_t* row_start, const int32_t* hot_items, int64_t hot_cap,
                            const int64_t* counts_dev, void* out, int out_dtype, int64_t U, int64_t D,
                            int accumulate, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(U >= 0 && n_rows >= 0, "negative size");
  RECIS_REQUIRE(D >= 1 && D <= 8192, "embedding dim %lld out of range", (long long)D);
  if (U == 0) return RECIS_OK;
  RECIS_REQUIRE(src && row_start && out && counts_dev, "NULL argument");
  RECIS_REQUIRE(rows != nullptr || n_rows == 0, "rows must not be NULL");
  RECIS_REQUIRE(hot_cap == 0 || hot_items, "hot_items must not be NULL");
  RECIS_REQUIRE(hot_cap == 0 || out_dtype == RECIS_F32, "hot rows are accumulated in fp32: out must be fp32");
  RECIS_REQUIRE(hot_cap == 0 || D <= 1024, "hot-row reduction supports D <= 1024 (got %lld)", (long long)D);
  const int in_sz = dtype_size(rows_dtype), out_sz = dtype_size(out_dtype);
  RECIS_REQUIRE(in_sz && out_sz, "invalid dtype");
  RECIS_REQUIRE(coef == nullptr || dtype_size(coef_dtype), "invalid coef dtype");
  const int vb_in = pick_vec_bytes(D * in_sz, reinterpret_cast<uintptr_t>(rows));
  const int vb_out = pick_vec_bytes(D * out_sz, reinterpret_cast<uintptr_t>(out));
  const int vec = std::max(1, std::min(vb_in / in_sz, vb_out / out_sz));
  CsrArgs a;
  a.row_start = row_start;
  a.src = src;
  a.coef = coef;
  a.coef_dt = coef_dtype;
  a.U = U;
  a.n_rows = n_rows;
  a.D = static_cast<int>(D);
  a.lpr_log2 = std::min(6, ilog2_ceil((D + vec - 1) / vec));
  a.accumulate = accumulate;
  a.err = device_error_word(current_device());
  RECIS_REQUIRE(a.err != nullptr, "could not allocate the device error word");
  const int rows_per_block = kBlock >> a.lpr_log2;
  const int64_t grid = (U + rows_per_block - 1) / rows_per_block;
  auto with_types = [&](auto tin, auto tout) {
    using TIn = decltype(tin);
    using TOut = decltype(tout);
    return dispatch_vec(vec, [&](auto vtag) {
      constexpr int VEC = decltype(vtag)::value;
      if constexpr (VEC * sizeof(TIn) > 16 || VEC * sizeof(TOut) > 16) {
        return fail(RECIS_ERR_ARG, "internal: vector too wide");
      } else {
        RECIS_TIME_KERNEL("csr_cold_kernel", stream)
        csr_cold_kernel<TIn, TOut, VEC><<<dim3(grid), dim3(kBlock), 0, stream>>>(
            static_cast<const TIn*>(rows), static_cast<TOut*>(out), a);
        RECIS_LAUNCH_CHECK();
        if constexpr (std::is_same<TOut, float>::value) {
          if (hot_cap > 0) {
            const int64_t hot_grid = std::min<int64_t>(hot_cap, 2048);
            const size_t lds = sizeof(float) * (kPlanBlock / kWave) * static_cast<size_t>(D);
            RECIS_TIME_KERNEL("csr_hot_kernel", stream)
            csr_hot_kernel<TIn, VEC><<<dim3(hot_grid), dim3(kPlanBlock), lds, stream>>>(
                static_cast<const TIn*>(rows), static_cast<float*>(out), a, hot_items, counts_dev, hot_cap);
            RECIS_LAUNCH_CHECK();
          }
        }
        return RECIS_OK;
      }
    });
  };
  if (rows_dtype == RECIS_F32 && out_dtype == RECIS_F32) return with_types(float{}, float{});
  if (rows_dtype == RECIS_BF16 && out_dtype == RECIS_F32) return with_types(bf16_t{}, float{});
  if (rows_dtype == RECIS_F16 && out_dtype == RECIS_F32) return with_types(f16_t{}, float{});
  if (rows_dtype == RECIS_BF16 && out_dtype == RECIS_BF16) return with_types(bf16_t{}, bf16_t{});
  if (rows_dtype == RECIS_F16 && out_dtype == RECIS_F16) return with_types(f16_t{}, f16_t{});
  return fail(RECIS_ERR_ARG, "unsupported dtype pair (rows=%d, out=%d)", rows_dtype, out_dtype);
}

}  // extern "C"
