// Batch plan for gfx950: dedup of a batch of ids together with the transposed index
// (for every unique id, the list of occurrences that carry it).
//
// The reference scatters gradients back to unique rows with one global atomic per
// element (csrc/ops/embedding_segment_reduce_kernel.cu:79-120, segment_ops_kernel.cu:133-165)
// and dedups with a radix sort (csrc/ops/ids_partition_kernel.cu:86-131). On MI355X
// device-scope atomics run at some 3e10 per second whatever they touch (a few percent of
// HBM speed) and ids of low-cardinality features repeat tens of thousands of times per
// batch, so this build never scatters rows and never builds the plan with global atomics:
// ids are partitioned by hash into buckets small enough to be deduplicated in LDS.
//
//   tile     a workgroup dedups tiles of 1024 ids in an LDS hash: an id repeated k times in
//            a tile becomes ONE record {id, first position, k}; records per bucket are
//            counted in an LDS histogram (one row per workgroup)
//   colscan  exclusive scan of every histogram column -> where each workgroup's records of
//            each bucket go; bucket sizes
//   scatter  records move to their bucket (bucket = top bits of the mixed id)
//   bucket   one workgroup per bucket: LDS hash over the bucket's records gives every unique
//            id its first position and its count; unique ids are ranked by first position
//            inside the bucket, counts are scanned into list offsets
//   scan     bucket totals -> first unique index and first list entry of every bucket
//   emit     one launch: per occurrence unique index (inverse) and list position; per unique
//            id the id, row_start, hot work items
//
// Unique ids come out ordered by (bucket, first occurrence): a function of the input only.
// The order of the occurrences inside one id's list is not specified.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <climits>
#include <mutex>
#include <type_traits>

#include "common.cuh"

namespace recis_hip {
namespace {

constexpr int kPlanBlock = 1024;  // ids per tile == threads of the tile / scatter / hot kernels
constexpr int kLdsSlots = 2048;   // LDS hash entries of a tile (load <= 1/2)
constexpr int kBucketBlock = 256;
constexpr int kBucketSlots = 1024;  // LDS hash entries of a bucket round
constexpr int kMaxBuckets = 8192;
constexpr int kMinBuckets = 32;
constexpr int kMaxRows = 512;  // histogram rows (= workgroups of the tile and scatter kernels)
constexpr int64_t kSetEmpty = -1;
constexpr int32_t kNoPos = 0x7fffffff;
constexpr int kHotLen = RECIS_PLAN_HOT_LEN;  // rows with more occurrences than this are "hot"
constexpr int kHotChunk = RECIS_PLAN_HOT_CHUNK;  // occurrences per hot work item

__device__ __forceinline__ uint64_t mix_id(int64_t key) {
  uint64_t x = static_cast<uint64_t>(key);
  x ^= x >> 33;
  x *= 0xff51afd7ed558ccdULL;
  x ^= x >> 33;
  x *= 0xc4ceb9fe1a85ec53ULL;
  x ^= x >> 33;
  return x;
}

// One deduplicated run of a tile: `word` = (count - 1) << 10 | index of the record in its tile.
struct alignas(16) Rec {
  int64_t key;
  int32_t pos;  // first position of the id in its tile (absolute)
  uint32_t word;
};

// A unique id of a bucket, in bucket-local terms.
struct alignas(16) URec {
  int64_t key;
  int32_t list_off;  // first list entry, relative to the bucket's first
  int32_t cnt;
};

struct PlanGeom {
  int64_t n;
  int tiles;         // ceil(n / 1024)
  int tiles_per_wg;  // tiles a workgroup of the tile / scatter kernels walks
  int rows;          // workgroups of those kernels == histogram rows
  int nb_log2;       // buckets = 1 << nb_log2
};

__device__ __forceinline__ int bucket_of(int64_t key, int nb_log2) {
  return static_cast<int>(mix_id(key) >> (64 - nb_log2));
}

// Rank of the set flags among the 1024 threads of a workgroup (by thread index) and their total.
__device__ __forceinline__ void block_rank1024(bool flag, int& rank, int& total, int* wave_counts /*[16]*/) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const uint64_t ballot = __ballot(flag);
  const int prior = __popcll(ballot & ((uint64_t(1) << lane) - 1));
  if (lane == 0) wave_counts[wave] = __popcll(ballot);
  __syncthreads();
  int base = 0, tot = 0;
#pragma unroll
  for (int w = 0; w < kPlanBlock / kWave; ++w) {
    const int c = wave_counts[w];
    if (w < wave) base += c;
    tot += c;
  }
  __syncthreads();
  rank = base + prior;
  total = tot;
}

// tile: LDS dedup of tiles of 1024 ids -> records, per-occurrence (record, rank in run), histogram row
__global__ void __launch_bounds__(kPlanBlock)
plan_tile_kernel(const int64_t* __restrict__ ids, PlanGeom g, Rec* __restrict__ tile_rec,
                 int32_t* __restrict__ tile_nrec, uint32_t* __restrict__ occ_rec, uint16_t* __restrict__ hist,
                 int64_t* __restrict__ counts) {
  __shared__ int64_t l_key[kLdsSlots + 1];
  __shared__ int32_t l_min[kLdsSlots + 1];
  __shared__ int32_t l_cnt[kLdsSlots + 1];
  __shared__ uint32_t l_hist[kMaxBuckets / 2];  // two 16-bit counters per word
  __shared__ int wave_counts[kPlanBlock / kWave];
  const int tid = threadIdx.x;
  const int nb = 1 << g.nb_log2;
  if (blockIdx.x == 0 && tid < 2) counts[tid] = 0;
  for (int w = tid; w < nb / 2; w += kPlanBlock) l_hist[w] = 0;
  const int t_lo = blockIdx.x * g.tiles_per_wg;
  const int t_hi = min(g.tiles, t_lo + g.tiles_per_wg);
  int64_t key_next = 0;
  if (static_cast<int64_t>(t_lo) * kPlanBlock + tid < g.n) key_next = ids[static_cast<int64_t>(t_lo) * kPlanBlock + tid];
  for (int t = t_lo; t < t_hi; ++t) {
    for (int e = tid; e <= kLdsSlots; e += kPlanBlock) {
      l_key[e] = kSetEmpty;
      l_min[e] = kNoPos;
      l_cnt[e] = 0;
    }
    __syncthreads();
    const int64_t i = static_cast<int64_t>(t) * kPlanBlock + tid;
    const bool live = i < g.n;
    const int64_t key = key_next;
    if (t + 1 < t_hi && i + kPlanBlock < g.n) key_next = ids[i + kPlanBlock];  // in flight while this tile is worked
    int e = 0, local_rank = 0;
    if (live) {
      if (key == kSetEmpty) {
        e = kLdsSlots;  // reserved entry for the id that equals the empty marker
      } else {
        e = static_cast<int>(mix_id(key) >> 20) & (kLdsSlots - 1);
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
    const bool first = live && l_min[e] == tid;
    int j, total;
    block_rank1024(first, j, total, wave_counts);
    if (first) {
      Rec r;
      r.key = key;
      r.pos = static_cast<int32_t>(i);
      r.word = (static_cast<uint32_t>(l_cnt[e] - 1) << 10) | static_cast<uint32_t>(j);
      tile_rec[static_cast<int64_t>(t) * kPlanBlock + j] = r;
      l_min[e] = j;  // every occurrence of the run reads its record index here
      const int b = bucket_of(key, g.nb_log2);
      atomicAdd(&l_hist[b >> 1], 1u << ((b & 1) * 16));
    }
    if (tid == 0) tile_nrec[t] = total;
    __syncthreads();
    if (live) occ_rec[i] = (static_cast<uint32_t>(local_rank) << 10) | static_cast<uint32_t>(l_min[e]);
    __syncthreads();
  }
  uint32_t* row = reinterpret_cast<uint32_t*>(hist + static_cast<int64_t>(blockIdx.x) * nb);
  for (int w = tid; w < nb / 2; w += kPlanBlock) row[w] = l_hist[w];
}

// colscan: for every bucket, exclusive scan of its histogram column over the rows.
// Workgroup = 32 buckets x 32 groups of rows.
__global__ void __launch_bounds__(1024)
plan_colscan_kernel(const uint16_t* __restrict__ hist, PlanGeom g, int32_t* __restrict__ off,
                    int32_t* __restrict__ bucket_total) {
  __shared__ int32_t part[32][33];
  const int nb = 1 << g.nb_log2;
  const int bl = threadIdx.x & 31, rg = threadIdx.x >> 5;
  const int b = blockIdx.x * 32 + bl;
  const int per = (g.rows + 31) / 32;
  const int r_lo = min(g.rows, rg * per), r_hi = min(g.rows, r_lo + per);
  int32_t sum = 0;
  for (int r = r_lo; r < r_hi; ++r) sum += hist[static_cast<int64_t>(r) * nb + b];
  part[rg][bl] = sum;
  __syncthreads();
  int32_t run = 0;
  for (int q = 0; q < rg; ++q) run += part[q][bl];
  for (int r = r_lo; r < r_hi; ++r) {
    const int64_t at = static_cast<int64_t>(r) * nb + b;
    const int32_t c = hist[at];
    off[at] = run;
    run += c;
  }
  if (rg == 31) bucket_total[b] = run;
}

// Exclusive scan of one or two int32 arrays of nb <= 8192 entries by one workgroup;
// out arrays have nb + 1 entries (the last one is the total); total of the first to total_out.
__global__ void __launch_bounds__(1024)
plan_scan_kernel(const int32_t* __restrict__ in0, int32_t* __restrict__ out0, const int32_t* __restrict__ in1,
                 int32_t* __restrict__ out1, int nb, int64_t* __restrict__ total_out,
                 volatile int64_t* total_host, const int* __restrict__ err) {
  __shared__ int32_t partial[1024];
  const int t = threadIdx.x;
  const int per = (nb + 1023) / 1024;
  const int lo = min(nb, t * per), hi = min(nb, lo + per);
  for (int pass = 0; pass < 2; ++pass) {
    const int32_t* in = pass ? in1 : in0;
    int32_t* out = pass ? out1 : out0;
    if (in == nullptr) break;
    int32_t sum = 0;
    for (int b = lo; b < hi; ++b) sum += in[b];
    partial[t] = sum;
    __syncthreads();
    for (int o = 1; o < 1024; o <<= 1) {
      const int32_t add = t >= o ? partial[t - o] : 0;
      __syncthreads();
      partial[t] += add;
      __syncthreads();
    }
    int32_t run = t ? partial[t - 1] : 0;
    for (int b = lo; b < hi; ++b) {
      const int32_t c = in[b];
      out[b] = run;
      run += c;
    }
    if (t == 1023) {
      out[nb] = partial[1023];
      if (pass == 0 && total_out) total_out[0] = partial[1023];
      if (pass == 0 && total_host) {  // pinned host words: no copy kernel needed
        total_host[1] = err ? __hip_atomic_load(err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0;
        total_host[0] = partial[1023];
      }
    }
    __syncthreads();
  }
}

// scatter: records of a workgroup's tiles go to their buckets
__global__ void __launch_bounds__(kPlanBlock)
plan_scatter_kernel(const Rec* __restrict__ tile_rec, const int32_t* __restrict__ tile_nrec, PlanGeom g,
                    const int32_t* __restrict__ off, const int32_t* __restrict__ bucket_start,
                    Rec* __restrict__ bucket_rec) {
  __shared__ int32_t cursor[kMaxBuckets];
  const int nb = 1 << g.nb_log2;
  const int32_t* off_row = off + static_cast<int64_t>(blockIdx.x) * nb;
  for (int b = threadIdx.x; b < nb; b += kPlanBlock) cursor[b] = bucket_start[b] + off_row[b];
  __syncthreads();
  const int t_lo = blockIdx.x * g.tiles_per_wg;
  const int t_hi = min(g.tiles, t_lo + g.tiles_per_wg);
  for (int t0 = t_lo; t0 < t_hi; t0 += 4) {  // four tiles' loads in flight
    Rec r[4];
    bool have[4];
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      const int t = t0 + x;
      have[x] = t < t_hi && static_cast<int>(threadIdx.x) < tile_nrec[t];
      if (have[x]) r[x] = tile_rec[static_cast<int64_t>(t) * kPlanBlock + threadIdx.x];
    }
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      if (have[x]) bucket_rec[atomicAdd(&cursor[bucket_of(r[x].key, g.nb_log2)], 1)] = r[x];
    }
  }
}

// bucket: dedup of the records of one bucket in LDS. A bucket normally holds a few hundred
// distinct ids (its records can be many more: a hot id brings one record per tile). When the
// distinct ids do not fit the LDS table, the bucket is started over in twice as many rounds:
// round r admits the ids whose hash falls in its share, so every id is handled in exactly one
// round. The first kBucketRegs
// records of a thread stay in registers between the two passes over the records; further
// ones (rare: hot buckets) go through `result` in global memory.
constexpr int kBucketRegs = 4;

__device__ __forceinline__ bool in_round(int64_t key, uint32_t rounds, uint32_t round) {
  return rounds == 1 || static_cast<uint32_t>((mix_id(key) >> 8) & 0xffffff) % rounds == round;
}

__global__ void __launch_bounds__(kBucketBlock)
plan_bucket_kernel(const Rec* __restrict__ bucket_rec, const int32_t* __restrict__ bucket_start, PlanGeom g,
                   int2* __restrict__ result, URec* __restrict__ bucket_uniq, int32_t* __restrict__ ucnt,
                   int32_t* __restrict__ ocnt, int* __restrict__ err) {
  constexpr int kPad = 16;  // d_min is read 16 entries at a time
  __shared__ int64_t l_key[kBucketSlots + 1];
  __shared__ int32_t l_min[kBucketSlots + 1];
  __shared__ int32_t l_cnt[kBucketSlots + 1];
  __shared__ uint16_t l_rank[kBucketSlots + 2];
  __shared__ uint16_t d_ent[kBucketSlots + 2];
  __shared__ __attribute__((aligned(16))) int32_t d_min[kBucketSlots + 1 + kPad];
  __shared__ int32_t s_cnt[kBucketSlots + 1];
  __shared__ int wave_counts[kBucketBlock / kWave];
  __shared__ int s_n_ent, s_total, s_overflow;
  const int tid = threadIdx.x;
  const int b = blockIdx.x;
  const int32_t r_lo = bucket_start[b], r_hi = bucket_start[b + 1];
  const int nrec = r_hi - r_lo;
  uint32_t rounds = 1;
  Rec reg[kBucketRegs];
#pragma unroll
  for (int x = 0; x < kBucketRegs; ++x) {
    const int32_t q = r_lo + tid + x * kBucketBlock;
    if (q < r_hi) reg[x] = bucket_rec[q];
  }
  int32_t u_done = 0, occ_done = 0;

  // inserts one record; returns the entry (or -1) and the offset of the record's run in the id's list
  auto insert = [&](const Rec& r, int& e, int& base) {
    if (r.key == kSetEmpty) {
      e = kBucketSlots;
    } else {
      e = static_cast<int>(mix_id(r.key) >> 32) & (kBucketSlots - 1);
      int probes = 0;
      for (;;) {
        int64_t k = l_key[e];
        if (k == kSetEmpty) {
          k = static_cast<int64_t>(atomicCAS(reinterpret_cast<unsigned long long*>(&l_key[e]),
                                             static_cast<unsigned long long>(kSetEmpty),
                                             static_cast<unsigned long long>(r.key)));
          if (k == kSetEmpty) break;
        }
        if (k == r.key) break;
        e = (e + 1) & (kBucketSlots - 1);
        if (++probes >= kBucketSlots) {  // table full: more distinct ids than a round can take
          e = -1;
          base = 0;
          s_overflow = 1;
          return;
        }
      }
    }
    base = atomicAdd(&l_cnt[e], static_cast<int>(r.word >> 10) + 1);
    atomicMin(&l_min[e], r.pos);
    if (base == 0) {  // first run of the id: list the entry
      const int k = atomicAdd(&s_n_ent, 1);
      d_ent[k] = static_cast<uint16_t>(e);
      if (k >= kBucketSlots * 7 / 8) s_overflow = 1;  // too loaded to go on probing
    }
  };
  auto origin_of = [](const Rec& r) { return (static_cast<int64_t>(r.pos) >> 10 << 10) | (r.word & 1023u); };

  for (uint32_t round = 0; round < rounds; ++round) {
    for (int e = tid; e <= kBucketSlots; e += kBucketBlock) {
      l_key[e] = kSetEmpty;
      l_min[e] = kNoPos;
      l_cnt[e] = 0;
      l_rank[e] = 0;
    }
    if (tid == 0) {
      s_n_ent = 0;
      s_overflow = 0;
    }
    __syncthreads();
    // A: insert the round's records
    int e_reg[kBucketRegs], base_reg[kBucketRegs];
#pragma unroll
    for (int x = 0; x < kBucketRegs; ++x) {
      e_reg[x] = -2;  // not of this round
      base_reg[x] = 0;
      const int32_t q = r_lo + tid + x * kBucketBlock;
      if (q < r_hi && in_round(reg[x].key, rounds, round)) insert(reg[x], e_reg[x], base_reg[x]);
    }
    for (int32_t q = r_lo + tid + kBucketRegs * kBucketBlock; q < r_hi; q += kBucketBlock) {
      const Rec r = bucket_rec[q];
      if (!in_round(r.key, rounds, round)) continue;
      int e, base;
      insert(r, e, base);
      result[origin_of(r)] = make_int2(e, base);
    }
    __syncthreads();
    if (s_overflow) {  // start the bucket over with twice the rounds
      __syncthreads();
      if (rounds >= (1u << 16)) {
        if (tid == 0) raise_device_error(err, RECIS_DEVERR_PLAN_OVERFLOW);
        break;
      }
      rounds *= 2;
      round = static_cast<uint32_t>(-1);  // ++ makes it 0
      u_done = 0;
      occ_done = 0;
      continue;
    }
    const int n_ent = s_n_ent;
    for (int k = tid; k < n_ent + kPad; k += kBucketBlock) d_min[k] = k < n_ent ? l_min[d_ent[k]] : kNoPos;
    __syncthreads();
    // rank by first position (positions are distinct), counts in rank order
    for (int k = tid; k < n_ent; k += kBucketBlock) {
      const int32_t m = d_min[k];
      int rnk = 0;
      for (int q = 0; q < n_ent; q += kPad) {
        const int4 a0 = *reinterpret_cast<const int4*>(&d_min[q]);
        const int4 a1 = *reinterpret_cast<const int4*>(&d_min[q + 4]);
        const int4 a2 = *reinterpret_cast<const int4*>(&d_min[q + 8]);
        const int4 a3 = *reinterpret_cast<const int4*>(&d_min[q + 12]);
        rnk += (a0.x < m) + (a0.y < m) + (a0.z < m) + (a0.w < m) + (a1.x < m) + (a1.y < m) + (a1.z < m) + (a1.w < m) +
               (a2.x < m) + (a2.y < m) + (a2.z < m) + (a2.w < m) + (a3.x < m) + (a3.y < m) + (a3.z < m) + (a3.w < m);
      }
      const int e = d_ent[k];
      l_rank[e] = static_cast<uint16_t>(rnk);
      s_cnt[rnk] = l_cnt[e];
    }
    __syncthreads();
    // exclusive scan of s_cnt[0 .. n_ent) in place (n_ent <= 1025): 5 consecutive entries per thread
    {
      constexpr int kPer = (kBucketSlots + 1 + kBucketBlock - 1) / kBucketBlock;
      int32_t v[kPer];
      int32_t sum = 0;
#pragma unroll
      for (int x = 0; x < kPer; ++x) {
        const int k = tid * kPer + x;
        v[x] = k < n_ent ? s_cnt[k] : 0;
        sum += v[x];
      }
      const int lane = tid & (kWave - 1), wave = tid / kWave;
      int32_t incl = sum;
      for (int o = 1; o < kWave; o <<= 1) {
        const int32_t y = __shfl_up(incl, o, kWave);
        if (lane >= o) incl += y;
      }
      if (lane == kWave - 1) wave_counts[wave] = incl;
      __syncthreads();
      int32_t run = incl - sum;
      int32_t tot = 0;
#pragma unroll
      for (int w = 0; w < kBucketBlock / kWave; ++w) {
        if (w < wave) run += wave_counts[w];
        tot += wave_counts[w];
      }
      if (tid == 0) s_total = tot;
#pragma unroll
      for (int x = 0; x < kPer; ++x) {
        const int k = tid * kPer + x;
        if (k < n_ent) s_cnt[k] = run;
        run += v[x];
      }
    }
    __syncthreads();
    for (int k = tid; k < n_ent; k += kBucketBlock) {
      const int e = d_ent[k];
      const int rnk = l_rank[e];
      URec u;
      u.key = e == kBucketSlots ? kSetEmpty : l_key[e];
      u.list_off = occ_done + s_cnt[rnk];
      u.cnt = l_cnt[e];
      bucket_uniq[r_lo + u_done + rnk] = u;
    }
    // B: every record learns its unique id (bucket-local) and the list offset of its run
#pragma unroll
    for (int x = 0; x < kBucketRegs; ++x) {
      if (e_reg[x] == -2) continue;
      int2 out = make_int2(0, 0);  // overflow (flagged): keep the indices in range
      if (e_reg[x] >= 0) {
        const int rnk = l_rank[e_reg[x]];
        out = make_int2(u_done + rnk, occ_done + s_cnt[rnk] + base_reg[x]);
      }
      result[origin_of(reg[x])] = out;
    }
    for (int32_t q = r_lo + tid + kBucketRegs * kBucketBlock; q < r_hi; q += kBucketBlock) {
      const Rec r = bucket_rec[q];
      if (!in_round(r.key, rounds, round)) continue;
      const int64_t origin = origin_of(r);
      const int2 eb = result[origin];
      int2 out = make_int2(0, 0);
      if (eb.x >= 0) {
        const int rnk = l_rank[eb.x];
        out = make_int2(u_done + rnk, occ_done + s_cnt[rnk] + eb.y);
      }
      result[origin] = out;
    }
    __syncthreads();
    u_done += n_ent;
    occ_done += s_total;
    __syncthreads();
  }
  if (tid == 0) {
    ucnt[b] = u_done;
    ocnt[b] = occ_done;
  }
}

__global__ void plan_empty_kernel(int64_t* __restrict__ counts, int32_t* __restrict__ row_start,
                                  volatile int64_t* total_host, const int* __restrict__ err) {
  if (threadIdx.x < 2) counts[threadIdx.x] = 0;
  if (threadIdx.x == 0) {
    row_start[0] = 0;
    if (total_host) {
      total_host[1] = err ? __hip_atomic_load(err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0;
      total_host[0] = 0;
    }
  }
}

// emit, per occurrence: inverse, list entry, position in the list
__device__ __forceinline__ void
emit_occ_block(int64_t vblock, const int64_t* __restrict__ ids, const uint32_t* __restrict__ occ_rec,
               const int2* __restrict__ result, const int32_t* __restrict__ ubase,
               const int32_t* __restrict__ lbase, const PlanGeom& g, int32_t* __restrict__ inverse,
               int32_t* __restrict__ list, int32_t* __restrict__ pos_out) {
  const int64_t i = vblock * kBlock + threadIdx.x;
  if (i >= g.n) return;
  const uint32_t w = occ_rec[i];
  const int2 r = result[(i >> 10 << 10) | (w & 1023u)];
  const int b = bucket_of(ids[i], g.nb_log2);
  const int32_t pos = lbase[b] + r.y + static_cast<int32_t>(w >> 10);
  inverse[i] = ubase[b] + r.x;
  if (static_cast<uint32_t>(pos) < static_cast<uint64_t>(g.n)) list[pos] = static_cast<int32_t>(i);  // else: overflow flagged
  if (pos_out) pos_out[i] = pos;
}

// emit, per unique id (workgroups 0 .. buckets-1: one bucket each): id, row_start, hot work
// items; the remaining workgroups set row_start[U .. n] = n.
__device__ __forceinline__ void
emit_uniq_block(int64_t vblock, const URec* __restrict__ bucket_uniq, const int32_t* __restrict__ bucket_start,
                const int32_t* __restrict__ ubase, const int32_t* __restrict__ lbase, const PlanGeom& g,
                int64_t* __restrict__ unique_out, int32_t* __restrict__ row_start,
                int64_t* __restrict__ counts, int32_t* __restrict__ hot_items, int64_t hot_cap) {
  const int nb = 1 << g.nb_log2;
  if (vblock >= nb) {
    const int64_t U = ubase[nb];
    const int64_t chunk = static_cast<int64_t>(kBlock) * 16;
    const int64_t lo = U + (vblock - nb) * chunk;
    const int64_t hi = min(lo + chunk, g.n + 1);
    for (int64_t x = lo + threadIdx.x; x < hi; x += kBlock) row_start[x] = static_cast<int32_t>(g.n);
    return;
  }
  const int b = static_cast<int>(vblock);
  const int32_t u0 = ubase[b], cnt = ubase[b + 1] - u0, l0 = lbase[b];
  const URec* src = bucket_uniq + bucket_start[b];
  for (int k = threadIdx.x; k < cnt; k += kBlock) {
    const URec u = src[k];
    unique_out[u0 + k] = u.key;
    row_start[u0 + k] = l0 + u.list_off;
    if (hot_cap > 0 && u.cnt > kHotLen) {
      const int n_items = (u.cnt + kHotChunk - 1) / kHotChunk;
      const int64_t base = static_cast<int64_t>(atomicAdd(reinterpret_cast<unsigned long long*>(&counts[1]),
                                                          static_cast<unsigned long long>(n_items)));
      for (int c = 0; c < n_items; ++c) {
        if (base + c < hot_cap) {
          hot_items[2 * (base + c)] = u0 + k;
          hot_items[2 * (base + c) + 1] = c;
        }
      }
    }
  }
}

// emit, one launch: the first `uniq_blocks` workgroups work per unique id (a bucket each, then
// the row_start tail), the rest per occurrence.
__global__ void __launch_bounds__(kBlock)
plan_emit_kernel(int64_t uniq_blocks, const int64_t* __restrict__ ids, const uint32_t* __restrict__ occ_rec,
                 const int2* __restrict__ result, const URec* __restrict__ bucket_uniq,
                 const int32_t* __restrict__ bucket_start, const int32_t* __restrict__ ubase,
                 const int32_t* __restrict__ lbase, PlanGeom g, int64_t* __restrict__ unique_out,
                 int32_t* __restrict__ inverse, int32_t* __restrict__ row_start, int32_t* __restrict__ list,
                 int32_t* __restrict__ pos_out, int64_t* __restrict__ counts, int32_t* __restrict__ hot_items,
                 int64_t hot_cap) {
  const int64_t vb = blockIdx.x;
  if (vb < uniq_blocks)
    emit_uniq_block(vb, bucket_uniq, bucket_start, ubase, lbase, g, unique_out, row_start, counts, hot_items,
                    hot_cap);
  else
    emit_occ_block(vb - uniq_blocks, ids, occ_rec, result, ubase, lbase, g, inverse, list, pos_out);
}

// ---------------------------------------------------------------- consumers
__device__ __forceinline__ float load_coef(const void* w, int wdt, int64_t i) {
  if (wdt == RECIS_F32) return static_cast<const float*>(w)[i];
  if (wdt == RECIS_BF16) return to_float(static_cast<const bf16_t*>(w)[i]);
  return to_float(static_cast<const f16_t*>(w)[i]);
}

constexpr int kMaxParts = 8;  // input arrays of one gather-reduce launch (PARTS kernels)

struct CsrArgs {
  const int32_t* row_start;  // [U + 1]
  const int32_t* src;        // [n] input row per list entry (negative = skip)
  const void* coef;          // [n] per list entry, or NULL
  int coef_dt;
  int64_t U, n_rows;
  int D;
  int lpr_log2;
  int accumulate;
  int nt_in;  // the gathered rows are too many to stay cached: non-temporal loads
  int* err;
  const void* cover;  // offsets [cover_S + 1] or NULL: entries whose src lies outside
  int cover64;        // [cover[0], cover[cover_S]) are skipped
  int64_t cover_S;
  // hot rows (more than hot_len occurrences): (row, chunk) work items, partial sums per item
  int32_t hot_len;           // INT_MAX when the caller brings no work items: every row is "cold"
  const int32_t* hot_items;  // [2 * hot_cap]
  const int64_t* counts;     // counts[1] = number of items
  int64_t hot_cap;
  float* hot_part;           // [hot_cap, D]
  int64_t cold_blocks;       // the last cold_blocks workgroups work per row, the ones before per hot item
  // PARTS kernels: the input rows are n_parts arrays laid end to end in src's numbering; part f
  // holds rows [part_lo[f], part_lo[f + 1])
  int n_parts;
  const void* part_rows[kMaxParts];
  int64_t part_lo[kMaxParts + 1];
};

// Row s of the input: of the one array, or of the part that holds it.
template <typename TIn, bool PARTS>
__device__ __forceinline__ const TIn* src_row(const TIn* rows, const CsrArgs& a, int64_t s) {
  if constexpr (!PARTS) {
    return rows + s * a.D;
  } else {
    int f = 0;
#pragma unroll
    for (int k = 1; k < kMaxParts; ++k) f += (k < a.n_parts && s >= a.part_lo[k]) ? 1 : 0;
    const TIn* base = static_cast<const TIn*>(a.part_rows[0]);
    int64_t lo = 0;
#pragma unroll
    for (int k = 1; k < kMaxParts; ++k) {
      if (k == f) {
        base = static_cast<const TIn*>(a.part_rows[k]);
        lo = a.part_lo[k];
      }
    }
    return base + (s - lo) * a.D;
  }
}

__device__ __forceinline__ void cover_range(const CsrArgs& a, int64_t& lo, int64_t& hi) {
  lo = 0;
  hi = a.n_rows;
  if (a.cover) {
    lo = max(lo, load_index(a.cover, a.cover64, 0));
    hi = min(hi, load_index(a.cover, a.cover64, a.cover_S));
  }
}

// A whole wave works the list entries [e_begin, e_end) (uniform arguments, every lane calls):
// `src` and `coef` of 64 entries come from one coalesced load, a lane each, and reach the lanes
// that gather the rows through shuffles; lane group g of `groups` takes entries g, g + groups,
// ... with several row loads in flight. acc: this group's partial sum for columns
// c0 .. c0 + VEC (the caller folds the groups).
template <typename TIn, int VEC, bool PARTS>
__device__ __forceinline__ void wave_gather_range(const TIn* __restrict__ rows, const CsrArgs& a, int64_t c_lo,
                                                  int64_t c_hi, int32_t e_begin, int32_t e_end, int c0, bool col_ok,
                                                  int g, int groups, float (&acc)[VEC]) {
  constexpr int kFly = VEC >= 8 ? 4 : 8;  // row loads in flight per lane
  const int lane = threadIdx.x & (kWave - 1);
  for (int32_t cb = e_begin; cb < e_end; cb += kWave) {
    const int n_here = min(kWave, e_end - cb);
    int32_t s_mine = -1;
    float w_mine = 0.f;
    if (lane < n_here) {
      const int32_t sv = a.src[cb + lane];
      if (sv >= c_lo && sv < c_hi) {
        s_mine = sv;
        w_mine = a.coef ? load_coef(a.coef, a.coef_dt, cb + lane) : 1.0f;
      } else if (static_cast<int64_t>(sv) >= a.n_rows) {
        raise_device_error(a.err, RECIS_DEVERR_INDEX_RANGE);
      }
    }
    for (int q0 = 0; q0 < n_here; q0 += kFly * groups) {  // same trip count for the whole wave (shuffles inside)
      float v[kFly][VEC];
      float w[kFly];
#pragma unroll
      for (int k = 0; k < kFly; ++k) {
        const int e = q0 + g + k * groups;
        const int from = min(e, kWave - 1);
        int32_t id = __shfl(s_mine, from, kWave);
        w[k] = a.coef ? __shfl(w_mine, from, kWave) : 1.0f;
        if (e >= n_here || !col_ok) id = -1;
        if (id >= 0) {
          const TIn* row = src_row<TIn, PARTS>(rows, a, id);
          if (a.nt_in) {
            load_pack_stream<TIn, VEC>(row + c0, v[k]);
          } else {
            load_pack<TIn, VEC>(row + c0, v[k]);
          }
        } else {
          w[k] = 0.f;
#pragma unroll
          for (int j = 0; j < VEC; ++j) v[k][j] = 0.f;
        }
      }
#pragma unroll
      for (int k = 0; k < kFly; ++k) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) acc[j] = fmaf(v[k][j], w[k], acc[j]);
      }
    }
  }
}

constexpr int kCoopLen = 8;  // longer lists are shared among the lane groups of a wave

// One launch for all rows. The last cold_blocks workgroups: one group of LPR lanes per unique row
// with at most hot_len occurrences ("cold"); a wave that holds a row with more than kCoopLen
// occurrences works that row with all its lane groups striding over the list (a row of 200
// occurrences would otherwise be 50 dependent gathers of one group). The first workgroups
// walk the hot work items (row, chunk of kHotChunk occurrences): four waves share the chunk,
// fold their sums through LDS and store ONE partial row per item; csr_hot_finish_kernel adds up
// the partial rows of every hot row in chunk order. No atomics anywhere.
// SHUFFLE: long lists go through wave_gather_range (pays off when a wave has at most eight lane
// groups, i.e. rows of 128 bytes and more); otherwise every group loads its own entries.
template <typename TIn, typename TOut, int VEC, bool SHUFFLE, bool PARTS = false>
__global__ void __launch_bounds__(kBlock)
csr_rows_kernel(const TIn* __restrict__ rows, TOut* __restrict__ out, CsrArgs a) {
  extern __shared__ float s_part[];  // [waves][D], hot part only
  const int D = a.D;
  const int cl = threadIdx.x & ((1 << a.lpr_log2) - 1);
  const int lane = threadIdx.x & (kWave - 1);
  const int groups = kWave >> a.lpr_log2;  // lane groups of a wave
  const int g = lane >> a.lpr_log2;        // this lane's group in its wave
  int64_t c_lo, c_hi;
  cover_range(a, c_lo, c_hi);

  auto fetch = [&](int32_t k, int c0, float (&v)[VEC], float& w) {
    const int32_t s = a.src[k];
    w = a.coef ? load_coef(a.coef, a.coef_dt, k) : 1.0f;
    if (s < c_lo || s >= c_hi) {
      if (static_cast<int64_t>(s) >= a.n_rows) raise_device_error(a.err, RECIS_DEVERR_INDEX_RANGE);
#pragma unroll
      for (int j = 0; j < VEC; ++j) v[j] = 0.f;
      w = 0.f;
      return;
    }
    const TIn* row = src_row<TIn, PARTS>(rows, a, s);
    if (a.nt_in) {
      load_pack_stream<TIn, VEC>(row + c0, v);
    } else {
      load_pack<TIn, VEC>(row + c0, v);
    }
  };
  // acc += sum over list entries k = first, first + step, ... < last (4 gathers in flight)
  auto gather_sum = [&](int32_t first, int32_t last, int32_t step, int c0, float (&acc)[VEC]) {
    int32_t k = first;
    for (; k + 3 * step < last; k += 4 * step) {
      float v0[VEC], v1[VEC], v2[VEC], v3[VEC];
      float w0, w1, w2, w3;
      fetch(k, c0, v0, w0);
      fetch(k + step, c0, v1, w1);
      fetch(k + 2 * step, c0, v2, w2);
      fetch(k + 3 * step, c0, v3, w3);
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        acc[j] = fmaf(v0[j], w0, acc[j]);
        acc[j] = fmaf(v1[j], w1, acc[j]);
        acc[j] = fmaf(v2[j], w2, acc[j]);
        acc[j] = fmaf(v3[j], w3, acc[j]);
      }
    }
    for (; k < last; k += step) {
      float v0[VEC];
      float w0;
      fetch(k, c0, v0, w0);
#pragma unroll
      for (int j = 0; j < VEC; ++j) acc[j] = fmaf(v0[j], w0, acc[j]);
    }
  };
  // the wave's sum over the list entries [first, last) for columns c0.., the same in every group
  auto wave_sum = [&](int32_t first, int32_t last, int c0, bool col_ok, float (&acc)[VEC]) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) acc[j] = 0.f;
    if constexpr (SHUFFLE) {
      wave_gather_range<TIn, VEC, PARTS>(rows, a, c_lo, c_hi, first, last, c0, col_ok, g, groups, acc);
    } else {
      if (col_ok) gather_sum(first + g, last, groups, c0, acc);
    }
    for (int off = 1 << a.lpr_log2; off < kWave; off <<= 1) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) acc[j] += __shfl_xor(acc[j], off, kWave);
    }
  };

  const int64_t hot_blocks = static_cast<int64_t>(gridDim.x) - a.cold_blocks;
  if (static_cast<int64_t>(blockIdx.x) < hot_blocks) {
    // ---- hot work items (the first workgroups: the longest-running ones start first)
    int64_t n_items = a.counts[1];
    if (n_items > a.hot_cap) n_items = a.hot_cap;
    const int wave = threadIdx.x / kWave;
    constexpr int n_waves = kBlock / kWave;
    for (int64_t item = blockIdx.x; item < n_items; item += hot_blocks) {
      const int32_t u = a.hot_items[2 * item];
      const int32_t chunk = a.hot_items[2 * item + 1];
      const int32_t start = a.row_start[u] + chunk * kHotChunk;
      const int32_t end = min(a.row_start[u + 1], start + kHotChunk);
      const int32_t per_wave = (end - start + n_waves - 1) / n_waves;  // a contiguous share per wave
      const int32_t w_begin = min(end, start + wave * per_wave), w_end = min(end, w_begin + per_wave);
      for (int cbase = 0; cbase < D; cbase += VEC << a.lpr_log2) {  // uniform: shuffles inside
        const int c0 = cbase + cl * VEC;
        const bool col_ok = c0 < D;
        float acc[VEC];
        wave_sum(w_begin, w_end, c0, col_ok, acc);
        if (g == 0 && col_ok) {
#pragma unroll
          for (int j = 0; j < VEC; ++j) s_part[wave * D + c0 + j] = acc[j];
        }
      }
      __syncthreads();
      for (int d = threadIdx.x; d < D; d += kBlock) {
        float sum = 0.f;
        for (int w = 0; w < n_waves; ++w) sum += s_part[w * D + d];
        a.hot_part[item * D + d] = sum;
      }
      __syncthreads();
    }
    return;
  }

  // ---- cold rows
  const int rows_per_block = kBlock >> a.lpr_log2;
  const int64_t u = (static_cast<int64_t>(blockIdx.x) - hot_blocks) * rows_per_block + (threadIdx.x >> a.lpr_log2);
  const bool valid = u < a.U;
  const int32_t start = valid ? a.row_start[u] : 0;
  int32_t end = valid ? a.row_start[u + 1] : 0;
  const bool hot = end - start > a.hot_len;  // left to the work items and the finish kernel
  if (hot) end = start;
  auto finish = [&](int64_t row, int c0, float (&acc)[VEC]) {
    TOut* dst = out + row * D + c0;
    if (a.accumulate) {
      float old[VEC];
      load_pack<TOut, VEC>(dst, old);
#pragma unroll
      for (int j = 0; j < VEC; ++j) acc[j] += old[j];
    }
    store_pack<TOut, VEC>(dst, acc);
  };
  // short rows: every lane group works its own row
  const bool is_long = a.lpr_log2 < 6 && end - start > kCoopLen;  // with one group per wave there is nobody to share with
  if (valid && !is_long && !hot) {
    for (int c0 = cl * VEC; c0 < D; c0 += VEC << a.lpr_log2) {
      float acc[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) acc[j] = 0.f;
      gather_sum(start, end, 1, c0, acc);
      finish(u, c0, acc);
    }
  }
  // long rows of this wave, one after the other
  uint64_t todo = __ballot(is_long);
  while (todo) {
    const int owner = __ffsll(static_cast<unsigned long long>(todo)) - 1;  // first lane of the owning group
    todo &= ~(((uint64_t(1) << (1 << a.lpr_log2)) - 1) << owner);  // the group's lanes (fewer than 64 here)
    const int r = owner >> a.lpr_log2;
    const int32_t r_start = __shfl(start, owner, kWave), r_end = __shfl(end, owner, kWave);
    const int64_t row = u - g + r;  // rows of a wave are consecutive
    for (int cbase = 0; cbase < D; cbase += VEC << a.lpr_log2) {  // uniform: shuffles inside
      const int c0 = cbase + cl * VEC;
      const bool col_ok = c0 < D;
      float acc[VEC];
      wave_sum(r_start, r_end, c0, col_ok, acc);
      if (g == r && col_ok) finish(row, c0, acc);
    }
  }
}

// out[u] (+)= sum of the partial rows of hot row u, in chunk order. One lane group per work item
// with chunk 0 (the items of a row are consecutive).
template <typename TOut, int VEC>
__global__ void __launch_bounds__(kBlock)
csr_hot_finish_kernel(TOut* __restrict__ out, CsrArgs a) {
  int64_t n_items = a.counts[1];
  if (n_items > a.hot_cap) n_items = a.hot_cap;
  const int D = a.D;
  const int cl = threadIdx.x & ((1 << a.lpr_log2) - 1);
  const int64_t groups_total = static_cast<int64_t>(gridDim.x) * (kBlock >> a.lpr_log2);
  for (int64_t item = static_cast<int64_t>(blockIdx.x) * (kBlock >> a.lpr_log2) + (threadIdx.x >> a.lpr_log2);
       item < n_items; item += groups_total) {
    if (a.hot_items[2 * item + 1] != 0) continue;
    const int32_t u = a.hot_items[2 * item];
    const int32_t len = a.row_start[u + 1] - a.row_start[u];
    int64_t n_chunks = (len + kHotChunk - 1) / kHotChunk;
    if (item + n_chunks > n_items) n_chunks = n_items - item;  // items cut off by hot_cap (cannot happen with the documented hot_cap)
    for (int c0 = cl * VEC; c0 < D; c0 += VEC << a.lpr_log2) {
      float acc[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) acc[j] = 0.f;
      for (int64_t k = 0; k < n_chunks; ++k) {
        float v[VEC];
        load_pack<float, VEC>(a.hot_part + (item + k) * D + c0, v);
#pragma unroll
        for (int j = 0; j < VEC; ++j) acc[j] += v[j];
      }
      TOut* dst = out + static_cast<int64_t>(u) * D + c0;
      if (a.accumulate) {
        float old[VEC];
        load_pack<TOut, VEC>(dst, old);
#pragma unroll
        for (int j = 0; j < VEC; ++j) acc[j] += old[j];
      }
      store_pack<TOut, VEC>(dst, acc);
    }
  }
}

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
  int32_t hot_len;
  const int32_t* hot_items;
  const int64_t* counts;
  int64_t hot_cap;
  int64_t cold_blocks;
};

template <typename TIn, typename TOut, int VEC, bool BLK>
__global__ void __launch_bounds__(kBlock)
csr_expand_kernel(const TIn* __restrict__ rows, TOut* __restrict__ out, ExpArgs a) {
  const int D = a.D;
  const int cl = threadIdx.x & ((1 << a.lpr_log2) - 1);
  const int lane = threadIdx.x & (kWave - 1);
  const int groups = kWave >> a.lpr_log2;  // lane groups of a wave
  const int g = lane >> a.lpr_log2;        // this lane's group in its wave

  auto load_row = [&](int64_t u, int c0, float (&v)[VEC]) {
    const TIn* src = nullptr;
    if constexpr (BLK) {
      const int64_t ri = a.row_index[u];
      if (ri >= 0) {
        int64_t b = 0, r = ri;
        if (a.n_blocks > 1) {
          b = ri / a.block_rows;
          r = ri - b * a.block_rows;
        }
        if (b >= a.n_blocks || r >= a.block_rows)
          raise_device_error(a.err, RECIS_DEVERR_INDEX_RANGE);
        else
          src = static_cast<const TIn*>(a.blocks[b]) + r * D;
      }
    } else {
      src = rows + u * D;
    }
    if (src) {
      load_pack_stream<TIn, VEC>(src + c0, v);  // every row is read once here
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
        load_row(u, c0, v);
        store_list(start + gb, end, groups_per_block, c0, v);
      }
    }
    return;
  }

  // ---- cold rows
  const int rows_per_block = kBlock >> a.lpr_log2;
  const int64_t u = (static_cast<int64_t>(blockIdx.x) - hot_blocks) * rows_per_block + (threadIdx.x >> a.lpr_log2);
  const bool valid = u < a.U && u < a.counts[0];  // U may be the caller's upper bound: the plan's own count decides
  const int32_t start = valid ? a.row_start[u] : 0;
  int32_t end = valid ? a.row_start[u + 1] : 0;
  if (end - start > a.hot_len) end = start;  // written by the work items
  const bool is_long = a.lpr_log2 < 6 && end - start > kCoopLen;
  if (valid && !is_long && end > start) {
    for (int c0 = cl * VEC; c0 < D; c0 += VEC << a.lpr_log2) {
      float v[VEC];
      load_row(u, c0, v);
      store_list(start, end, 1, c0, v);
    }
  }
  // long rows of this wave, one after the other: the owner's row reaches every group by shuffles
  uint64_t todo = __ballot(is_long);
  while (todo) {
    const int owner = __ffsll(static_cast<unsigned long long>(todo)) - 1;
    todo &= ~(((uint64_t(1) << (1 << a.lpr_log2)) - 1) << owner);
    const int32_t r_start = __shfl(start, owner, kWave), r_end = __shfl(end, owner, kWave);
    const int64_t row = u - g + (owner >> a.lpr_log2);  // rows of a wave are consecutive
    for (int cbase = 0; cbase < D; cbase += VEC << a.lpr_log2) {  // uniform: shuffles inside
      const int c0 = cbase + cl * VEC;
      const bool col_ok = c0 < D;
      float mine[VEC], v[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) mine[j] = 0.f;
      if (lane >> a.lpr_log2 == owner >> a.lpr_log2 && col_ok) load_row(row, c0, mine);
#pragma unroll
      for (int j = 0; j < VEC; ++j) v[j] = __shfl(mine[j], owner + cl, kWave);
      if (col_ok) store_list(r_start + g, r_end, groups, c0, v);
    }
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

// Where the plan's scratch arrays lie in one buffer of `bytes` bytes, for n ids.
struct PlanLayout {
  PlanGeom g;
  int64_t nb;
  size_t o_tile, o_brec, o_res, o_occ, o_hist, o_off, o_nrec, o_small, bytes;
};

static PlanLayout plan_layout(int64_t n) {
  PlanLayout L;
  PlanGeom& g = L.g;
  g.n = n;
  g.tiles = static_cast<int>((n + kPlanBlock - 1) / kPlanBlock);
  g.tiles_per_wg = std::min(63, (g.tiles + kMaxRows - 1) / kMaxRows);  // 16-bit histogram counters
  g.rows = (g.tiles + g.tiles_per_wg - 1) / g.tiles_per_wg;
  // 512 to 1024 ids per bucket while the bucket count allows: a few hundred distinct ids for the
  // LDS table of a bucket
  int nb_log2 = 5;
  while ((int64_t(1) << (nb_log2 + 1)) <= kMaxBuckets && (int64_t(1) << (nb_log2 + 1)) * 512 <= n) ++nb_log2;
  g.nb_log2 = nb_log2;
  L.nb = int64_t(1) << nb_log2;
  const int64_t n_pad = static_cast<int64_t>(g.tiles) * kPlanBlock;
  // tile_rec[n_pad] (later: the unique ids of every bucket) | bucket_rec[n_pad] | result[n_pad] |
  // occ_rec[n] | hist[rows*nb] u16 | off[rows*nb] | tile_nrec[tiles] | 6 arrays of nb + 1
  size_t bytes = 0;
  auto take = [&](size_t b) {
    const size_t at = bytes;
    bytes += (b + 255) & ~size_t(255);
    return at;
  };
  L.o_tile = take(sizeof(Rec) * n_pad);
  L.o_brec = take(sizeof(Rec) * n_pad);
  L.o_res = take(sizeof(int2) * n_pad);
  L.o_occ = take(sizeof(uint32_t) * n_pad);
  L.o_hist = take(sizeof(uint16_t) * g.rows * L.nb);
  L.o_off = take(sizeof(int32_t) * g.rows * L.nb);
  L.o_nrec = take(sizeof(int32_t) * g.tiles);
  L.o_small = take(sizeof(int32_t) * 6 * (L.nb + 1));
  L.bytes = bytes;
  return L;
}

static int plan_check_args(const int64_t* ids, int64_t n, int64_t* unique_out, int32_t* inverse_out,
                           int32_t* row_start_out, int32_t* list_out, int32_t* hot_items_out, int64_t hot_cap,
                           int64_t* counts_out_dev) {
  RECIS_REQUIRE(n >= 0 && n < (int64_t(1) << 30), "n out of range: %lld", (long long)n);
  RECIS_REQUIRE(counts_out_dev && row_start_out, "counts_out_dev / row_start_out must not be NULL");
  RECIS_REQUIRE(hot_cap == 0 || (hot_items_out && hot_cap >= n / kHotLen + n / kHotChunk + 2),
                "hot_items_out must hold at least n/%d + n/%d + 2 items", kHotLen, kHotChunk);
  RECIS_REQUIRE(n == 0 || (ids && unique_out && inverse_out && list_out), "NULL argument");
  return RECIS_OK;
}

// The plan's launches for n > 0 over the scratch buffer `base` (L.bytes bytes). `staged`: pinned host
// word that receives the unique count as soon as it is final, or NULL.
static int plan_launch(const PlanLayout& L, char* base, const int64_t* ids, int64_t* unique_out,
                       int32_t* inverse_out, int32_t* row_start_out, int32_t* list_out, int32_t* pos_out,
                       int32_t* hot_items_out, int64_t hot_cap, int64_t* counts_out_dev, int64_t* staged,
                       hipEvent_t staged_event, int* err, hipStream_t stream) {
  const PlanGeom& g = L.g;
  const int64_t nb = L.nb, n = g.n;
  Rec* tile_rec = reinterpret_cast<Rec*>(base + L.o_tile);
  Rec* bucket_rec = reinterpret_cast<Rec*>(base + L.o_brec);
  int2* result = reinterpret_cast<int2*>(base + L.o_res);
  uint32_t* occ_rec = reinterpret_cast<uint32_t*>(base + L.o_occ);
  uint16_t* hist = reinterpret_cast<uint16_t*>(base + L.o_hist);
  int32_t* off = reinterpret_cast<int32_t*>(base + L.o_off);
  int32_t* tile_nrec = reinterpret_cast<int32_t*>(base + L.o_nrec);
  int32_t* bucket_total = reinterpret_cast<int32_t*>(base + L.o_small);
  int32_t* bucket_start = bucket_total + (nb + 1);
  int32_t* ucnt = bucket_start + (nb + 1);
  int32_t* ocnt = ucnt + (nb + 1);
  int32_t* ubase = ocnt + (nb + 1);
  int32_t* lbase = ubase + (nb + 1);
  URec* bucket_uniq = reinterpret_cast<URec*>(tile_rec);  // the tile records are dead after the scatter

  {
    RECIS_TIME_KERNEL("plan_tile_kernel", stream)
    plan_tile_kernel<<<dim3(g.rows), dim3(kPlanBlock), 0, stream>>>(ids, g, tile_rec, tile_nrec, occ_rec, hist,
                                                                   counts_out_dev);
    RECIS_LAUNCH_CHECK();
  }
  {
    RECIS_TIME_KERNEL("plan_colscan_kernel", stream)
    plan_colscan_kernel<<<dim3(nb / 32), dim3(1024), 0, stream>>>(hist, g, off, bucket_total);
    RECIS_LAUNCH_CHECK();
  }
  plan_scan_kernel<<<1, 1024, 0, stream>>>(bucket_total, bucket_start, nullptr, nullptr, static_cast<int>(nb),
                                           nullptr, nullptr, nullptr);
  RECIS_LAUNCH_CHECK();
  {
    RECIS_TIME_KERNEL("plan_scatter_kernel", stream)
    plan_scatter_kernel<<<dim3(g.rows), dim3(kPlanBlock), 0, stream>>>(tile_rec, tile_nrec, g, off, bucket_start,
                                                                      bucket_rec);
    RECIS_LAUNCH_CHECK();
  }
  {
    RECIS_TIME_KERNEL("plan_bucket_kernel", stream)
    plan_bucket_kernel<<<dim3(nb), dim3(kBucketBlock), 0, stream>>>(bucket_rec, bucket_start, g, result, bucket_uniq,
                                                                   ucnt, ocnt, err);
    RECIS_LAUNCH_CHECK();
  }
  // The count is final after this scan: the kernel stores it into pinned host memory as well (with
  // the soft-error bits raised so far), and the host waits for it only after the emit kernels are
  // queued, so that the GPU works while the host learns the size of the next launches.
  plan_scan_kernel<<<1, 1024, 0, stream>>>(ucnt, ubase, ocnt, lbase, static_cast<int>(nb), counts_out_dev, staged,
                                           err);
  RECIS_LAUNCH_CHECK();
  if (staged) RECIS_CHECK_HIP(hipEventRecord(staged_event, stream));
  {
    const int64_t tail_blocks = (n + 1 + kBlock * 16 - 1) / (kBlock * 16);
    const int64_t uniq_blocks = nb + tail_blocks, occ_blocks = (n + kBlock - 1) / kBlock;
    RECIS_TIME_KERNEL("plan_emit_kernel", stream)
    plan_emit_kernel<<<dim3(uniq_blocks + occ_blocks), dim3(kBlock), 0, stream>>>(
        uniq_blocks, ids, occ_rec, result, bucket_uniq, bucket_start, ubase, lbase, g, unique_out, inverse_out,
        row_start_out, list_out, pos_out, counts_out_dev, hot_items_out, hot_cap);
    RECIS_LAUNCH_CHECK();
  }
  return RECIS_OK;
}

int recis_unique_plan(const int64_t* ids, int64_t n, int64_t* unique_out, int32_t* inverse_out,
                      int32_t* row_start_out, int32_t* list_out, int32_t* pos_out, int32_t* hot_items_out,
                      int64_t hot_cap, int64_t* counts_out_dev, int64_t* unique_count_host, int flags, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (int rc = plan_check_args(ids, n, unique_out, inverse_out, row_start_out, list_out, hot_items_out, hot_cap,
                               counts_out_dev))
    return rc;
  int* err = device_error_word(current_device());
  RECIS_REQUIRE(err != nullptr, "could not reach the device error word");
  const bool stage = unique_count_host || (flags & RECIS_PLAN_STAGE_COUNT);
  int64_t* staged = nullptr;
  hipEvent_t staged_event = nullptr;
  if (stage) {
    if (int rc = get_count_staging(stream, &staged, &staged_event)) return rc;
  }
  if (n == 0) {
    plan_empty_kernel<<<1, 64, 0, stream>>>(counts_out_dev, row_start_out, staged, err);
    RECIS_LAUNCH_CHECK();
    if (stage) RECIS_CHECK_HIP(hipEventRecord(staged_event, stream));
    if (unique_count_host) *unique_count_host = 0;
    return RECIS_OK;
  }
  const PlanLayout L = plan_layout(n);
  void* ws = nullptr;
  if (int rc = get_workspace(stream, L.bytes, &ws)) return rc;
  if (int rc = plan_launch(L, static_cast<char*>(ws), ids, unique_out, inverse_out, row_start_out, list_out, pos_out,
                           hot_items_out, hot_cap, counts_out_dev, staged, staged_event, err, stream))
    return rc;
  if (unique_count_host) {
    RECIS_CHECK_HIP(hipEventSynchronize(staged_event));
    *unique_count_host = staged[0];
  }
  return RECIS_OK;
}

// The scratch of recis_unique_plan_noalloc: part of the library's code object on every device that
// loads it. Host code never uses this name as an address: the per-device address comes from
// hipGetSymbolAddress (below) and travels to the kernels as an argument.
constexpr size_t kStaticScratchBytes = size_t(RECIS_PLAN_NOALLOC_SCRATCH_MIB) << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
constexpr int kMaxScratchDevices = 64;
static std::mutex g_scratch_mu;
static char* g_scratch_ptr[kMaxScratchDevices];

int recis_unique_plan_noalloc(const int64_t* ids, int64_t n, int64_t* unique_out, int32_t* inverse_out,
                              int32_t* row_start_out, int32_t* list_out, int32_t* pos_out,
                              int32_t* hot_items_out, int64_t hot_cap, int64_t* counts_out_dev, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (int rc = plan_check_args(ids, n, unique_out, inverse_out, row_start_out, list_out, hot_items_out, hot_cap,
                               counts_out_dev))
    return rc;
  const int dev = current_device();
  RECIS_REQUIRE(dev >= 0 && dev < kMaxScratchDevices, "device %d out of range", dev);
  char* base = nullptr;
  {
    std::lock_guard<std::mutex> l(g_scratch_mu);
    if (g_scratch_ptr[dev] == nullptr) {  // first call on this device (it is the current one)
      void* p = nullptr;
      RECIS_CHECK_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
      g_scratch_ptr[dev] = static_cast<char*>(p);
    }
    base = g_scratch_ptr[dev];
  }
  int* err = device_error_word(dev);
  RECIS_REQUIRE(err != nullptr, "could not reach the device error word");
  if (n == 0) {
    plan_empty_kernel<<<1, 64, 0, stream>>>(counts_out_dev, row_start_out, nullptr, err);
    RECIS_LAUNCH_CHECK();
    return RECIS_OK;
  }
  RECIS_REQUIRE(n <= RECIS_PLAN_NOALLOC_MAX_IDS, "recis_unique_plan_noalloc takes at most %lld ids per call (got %lld); "
                "use recis_unique_plan for more", (long long)RECIS_PLAN_NOALLOC_MAX_IDS, (long long)n);
  const PlanLayout L = plan_layout(n);
  if (L.bytes > kStaticScratchBytes)
    return fail(RECIS_ERR_CAPACITY,
                "recis_unique_plan_noalloc: %lld ids need %zu bytes of scratch, the built-in buffer holds %zu "
                "(at most %lld ids per call; use recis_unique_plan for more)",
                (long long)n, L.bytes, kStaticScratchBytes, (long long)RECIS_PLAN_NOALLOC_MAX_IDS);
  // every scratch array is fully written by the kernel that produces it before any kernel reads it:
  // nothing of the previous call's contents is relied on, nothing needs clearing
  return plan_launch(L, base, ids, unique_out, inverse_out, row_start_out, list_out, pos_out, hot_items_out, hot_cap,
                     counts_out_dev, nullptr, nullptr, err, stream);
}

int recis_unique_plan_count(int64_t* unique_count_host, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(unique_count_host != nullptr, "unique_count_host must not be NULL");
  int64_t* staged = nullptr;
  hipEvent_t staged_event = nullptr;
  if (int rc = get_count_staging(stream, &staged, &staged_event)) return rc;
  RECIS_CHECK_HIP(hipEventSynchronize(staged_event));
  *unique_count_host = staged[0];
  return RECIS_OK;
}

int recis_hip_staged_device_errors(int* bits, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(bits != nullptr, "bits must not be NULL");
  int64_t* staged = nullptr;
  hipEvent_t staged_event = nullptr;
  if (int rc = get_count_staging(stream, &staged, &staged_event)) return rc;
  *bits = static_cast<int>(staged[1]);
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

static int csr_gather_reduce_impl(const void* rows, const void* const* part_rows, const int64_t* part_counts,
                                  int n_parts, int rows_dtype, int64_t n_rows, const int32_t* src, const void* coef,
                                  int coef_dtype, const int32_t* row_start, const int32_t* hot_items,
                                  int64_t hot_cap, const int64_t* counts_dev, void* out, int out_dtype, int64_t U,
                                  int64_t D, int accumulate, const void* cover_offsets, int cover_is64,
                                  int64_t cover_S, hipStream_t stream);

int recis_csr_gather_reduce(const void* rows, int rows_dtype, int64_t n_rows, const int32_t* src, const void* coef,
                            int coef_dtype, const int32_t* row_start, const int32_t* hot_items, int64_t hot_cap,
                            const int64_t* counts_dev, void* out, int out_dtype, int64_t U, int64_t D,
                            int accumulate, const void* cover_offsets, int cover_is64, int64_t cover_S,
                            void* stream_) {
  return csr_gather_reduce_impl(rows, nullptr, nullptr, 0, rows_dtype, n_rows, src, coef, coef_dtype, row_start,
                                hot_items, hot_cap, counts_dev, out, out_dtype, U, D, accumulate, cover_offsets,
                                cover_is64, cover_S, static_cast<hipStream_t>(stream_));
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
  return csr_gather_reduce_impl(nullptr, part_rows, part_counts, n_parts, rows_dtype, n_rows, src, nullptr, 0,
                                row_start, hot_items, hot_cap, counts_dev, out, RECIS_F32, U, D, accumulate, nullptr,
                                0, 0, static_cast<hipStream_t>(stream_));
}

static int csr_gather_reduce_impl(const void* rows, const void* const* part_rows, const int64_t* part_counts,
                                  int n_parts, int rows_dtype, int64_t n_rows, const int32_t* src, const void* coef,
                                  int coef_dtype, const int32_t* row_start, const int32_t* hot_items,
                                  int64_t hot_cap, const int64_t* counts_dev, void* out, int out_dtype, int64_t U,
                                  int64_t D, int accumulate, const void* cover_offsets, int cover_is64,
                                  int64_t cover_S, hipStream_t stream) {
  RECIS_REQUIRE(U >= 0 && n_rows >= 0, "negative size");
  RECIS_REQUIRE(D >= 1 && D <= 8192, "embedding dim %lld out of range", (long long)D);
  if (U == 0) return RECIS_OK;
  RECIS_REQUIRE(src && row_start && out && counts_dev, "NULL argument");
  RECIS_REQUIRE(n_parts > 0 || rows != nullptr || n_rows == 0, "rows must not be NULL");
  RECIS_REQUIRE(hot_cap == 0 || hot_items, "hot_items must not be NULL");
  const int in_sz = dtype_size(rows_dtype), out_sz = dtype_size(out_dtype);
  RECIS_REQUIRE(in_sz && out_sz, "invalid dtype");
  RECIS_REQUIRE(coef == nullptr || dtype_size(coef_dtype), "invalid coef dtype");
  uintptr_t align_of = reinterpret_cast<uintptr_t>(rows);
  for (int f = 0; f < n_parts; ++f) align_of |= reinterpret_cast<uintptr_t>(part_rows[f]);  // the coarsest alignment
  const int vb_in = pick_vec_bytes(D * in_sz, align_of);
  const int vb_out = pick_vec_bytes_max(D * out_sz, reinterpret_cast<uintptr_t>(out), 32);
  const int vec = std::max(1, std::min(vb_in / in_sz, vb_out / out_sz));
  CsrArgs a;
  a.row_start = row_start;
  a.src = src;
  a.coef = coef;
  a.coef_dt = coef_dtype;
  a.U = U;
  a.n_rows = n_rows;
  a.cover = cover_offsets;
  a.cover64 = cover_is64;
  a.cover_S = cover_S;
  a.D = static_cast<int>(D);
  a.lpr_log2 = std::min(6, ilog2_ceil((D + vec - 1) / vec));
  a.accumulate = accumulate;
  a.nt_in = n_rows * D * in_sz >= (int64_t(1) << 30);
  a.err = device_error_word(current_device());
  RECIS_REQUIRE(a.err != nullptr, "could not reach the device error word");
  const int rows_per_block = kBlock >> a.lpr_log2;
  a.cold_blocks = (U + rows_per_block - 1) / rows_per_block;
  a.hot_len = hot_cap > 0 ? kHotLen : INT_MAX;
  a.hot_items = hot_items;
  a.counts = counts_dev;
  a.hot_cap = hot_cap;
  a.hot_part = nullptr;
  a.n_parts = n_parts;
  a.part_lo[0] = 0;
  for (int f = 0; f < kMaxParts; ++f) {
    a.part_rows[f] = f < n_parts ? part_rows[f] : nullptr;
    a.part_lo[f + 1] = a.part_lo[f] + (f < n_parts ? part_counts[f] : 0);
  }
  int64_t hot_blocks = 0;
  if (hot_cap > 0) {
    void* ws = nullptr;
    if (int rc = get_workspace(stream, sizeof(float) * static_cast<size_t>(hot_cap) * static_cast<size_t>(D), &ws))
      return rc;
    a.hot_part = static_cast<float*>(ws);
    hot_blocks = std::min<int64_t>(hot_cap, 4096);
  }
  const size_t lds = sizeof(float) * (kBlock / kWave) * static_cast<size_t>(D);
  auto with_types = [&](auto tin, auto tout) {
    using TIn = decltype(tin);
    using TOut = decltype(tout);
    return dispatch_vec(vec, [&](auto vtag) {
      constexpr int VEC = decltype(vtag)::value;
      if constexpr (VEC * sizeof(TIn) > 16 || VEC * sizeof(TOut) > 32) {
        return fail(RECIS_ERR_ARG, "internal: vector too wide");
      } else {
        const TIn* rin = static_cast<const TIn*>(rows);
        TOut* o = static_cast<TOut*>(out);
        const bool shuffle = a.lpr_log2 >= 3;  // at most eight lane groups per wave
        {
          RECIS_TIME_KERNEL("csr_rows_kernel", stream)
          if (n_parts > 0) {
            if constexpr (sizeof(TOut) == 4) {  // parts go to fp32 rows only
              if (shuffle)
                csr_rows_kernel<TIn, TOut, VEC, true, true><<<dim3(a.cold_blocks + hot_blocks), dim3(kBlock), lds, stream>>>(rin, o, a);
              else
                csr_rows_kernel<TIn, TOut, VEC, false, true><<<dim3(a.cold_blocks + hot_blocks), dim3(kBlock), lds, stream>>>(rin, o, a);
            }
          } else if (shuffle)
            csr_rows_kernel<TIn, TOut, VEC, true><<<dim3(a.cold_blocks + hot_blocks), dim3(kBlock), lds, stream>>>(rin, o, a);
          else
            csr_rows_kernel<TIn, TOut, VEC, false><<<dim3(a.cold_blocks + hot_blocks), dim3(kBlock), lds, stream>>>(rin, o, a);
          RECIS_LAUNCH_CHECK();
        }
        if (hot_cap > 0) {
          const int64_t fin = std::min<int64_t>((hot_cap + rows_per_block - 1) / rows_per_block, 1024);
          csr_hot_finish_kernel<TOut, VEC><<<dim3(fin), dim3(kBlock), 0, stream>>>(o, a);
          RECIS_LAUNCH_CHECK();
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

int recis_csr_expand_rows(const void* rows, void* const* emb_blocks_dev, int64_t n_blocks, int64_t block_rows,
                          const int64_t* row_index, int rows_dtype, const void* weight, int weight_dtype,
                          const int32_t* row_start, const int32_t* dst, const int32_t* hot_items, int64_t hot_cap,
                          const int64_t* counts_dev, void* out, int out_dtype, int64_t U, int64_t n_out, int64_t D,
                          void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
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
  a.n_blocks = n_blocks;
  a.hot_len = hot_cap > 0 ? kHotLen : INT_MAX;
  a.hot_items = hot_items;
  a.counts = counts_dev;
  a.hot_cap = hot_cap;
  const int rows_per_block = kBlock >> a.lpr_log2;
  a.cold_blocks = (U + rows_per_block - 1) / rows_per_block;
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
        if (blk)
          csr_expand_kernel<TIn, TOut, VEC, true><<<grid, dim3(kBlock), 0, stream>>>(nullptr, static_cast<TOut*>(out), a);
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
