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
//   hist     ids per (tile, column) in an LDS histogram, a tile of ids per workgroup; a column is
//            a hash bucket (top bits of the mixed id) or, for the few ids that make up a sizeable
//            share of the batch, a column of their own (found by sampling, see find_heavy)
//   colscan  exclusive scan of every histogram column -> where each tile's ids of each column
//            go; column totals
//   scatter  (id, position) of every occurrence moves to its column; the columns are laid out
//            heavy ids first, then the fullest buckets, then the rest (see column_starts)
//   bucket   one workgroup per bucket, in the order of the layout: the bucket's ids are
//            deduplicated in an LDS hash table whose final state does not depend on the order of
//            insertion; the place of an id in the table is its rank among the bucket's unique
//            ids; occurrences are counted and placed into their id's list; the number of unique
//            ids of the earlier buckets comes from a decoupled look-back; every unique id is
//            written with its list start and, with an id map, found or inserted there
//   assign   rows for the keys that were new to the id map, in the order of the unique ids
//
// The batch may be one array or several that are tagged and concatenated by the reads themselves
// (IdJobs). Unique ids come out ordered by (place of their column in the layout, place in the
// bucket's table): a function of the input only. The order of the occurrences inside one id's list
// is not specified. The consumers of the plan (gather-reduce, expansion) live in csr*.hip.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <climits>
#include <mutex>
#include <atomic>
#include <type_traits>

#include "common.cuh"
#include "idmap_internal.cuh"

namespace recis_hip {
namespace {

constexpr int kTile = 10240;       // most ids per workgroup of the histogram / scatter kernels (more when n is huge)
constexpr int kTileMin = 2048;     // and fewest, when the batch is small
constexpr int kPartBlock = 1024;   // threads of those kernels
constexpr int kTilePer = kTile / kPartBlock;  // ids of a tile of at most kTile per thread
constexpr int kMaxRows = 1024;     // workgroups of those kernels == histogram rows
constexpr int kMinBuckets = 32;
constexpr int kMaxBuckets = 8192;   // the histogram of a workgroup lives in LDS
constexpr int kBucketIds = 2560;    // ids per bucket aimed at: an LDS table of 4096 home slots holds them all
constexpr int kTabHome = 4096;      // home slots of a bucket's LDS table
constexpr int kTabAll = kTabHome + 256;  // linear probing runs on past the last home slot and never wraps;
                                         // slot kTabAll - 1 is a guard that stays empty
constexpr int kSpecial = kTabAll;   // entry of the id that equals the empty marker
constexpr int kBucketBlock = 512;
constexpr int kPer = 9;             // consecutive table entries owned by a thread (9 * 512 > kTabAll)
constexpr int kRegs = 8;            // bucket records of a thread whose table entry stays in registers
constexpr int64_t kSetEmpty = -1;
constexpr int kHeavyMax = 64;       // ids that get a column of their own in the partition (see find_heavy)
constexpr int kHeavySamples = 2048; // ids sampled to find them
constexpr int kHeavyTab = 4096;     // LDS table of the sampling kernel
constexpr int kHeavySlots = 256;    // LDS table every partition workgroup looks ids up in
constexpr int kHotLen = RECIS_PLAN_HOT_LEN;  // rows with more occurrences than this are "hot"
constexpr int kHotChunk = RECIS_PLAN_HOT_CHUNK;  // occurrences per hot work item
static_assert(kPer * kBucketBlock > kTabAll, "every table entry needs an owner");

__device__ __forceinline__ uint64_t mix_id(int64_t key) { return mix_key(key); }

struct PlanGeom {
  int64_t n;
  int rows;     // workgroups of the histogram / scatter kernels == histogram rows
  int tile;     // ids per row (a multiple of kPartBlock)
  int nb_log2;  // buckets = 1 << nb_log2
};

__device__ __forceinline__ int bucket_of_mix(uint64_t mixed, int nb_log2) {
  return static_cast<int>(mixed >> (64 - nb_log2));
}
// Home entry of an id in its bucket's LDS table: the 12 bits below the bucket bits, so that the
// entries of a bucket lie in the order of the mixed id, like the buckets themselves.
__device__ __forceinline__ int home_of_mix(uint64_t mixed, int nb_log2) {
  return static_cast<int>(mixed >> (64 - nb_log2 - 12)) & (kTabHome - 1);
}

// The batch as the partition kernels read it: one array of ids, or up to kPlanJobs arrays laid end
// to end whose ids are tagged on the way in. The second form is ids_encode
// (csrc/ops/ids_encode_kernel.cu:16-20: id & (2^52 - 1) | table << 52) or a plain concatenation
// folded into the plan's own reads, so the encoded batch is never written and read back.
constexpr int kPlanJobs = 64;
struct IdJobs {
  int n_jobs;  // 0: one array
  int64_t mask;
  const int64_t* in[kPlanJobs];
  int64_t first[kPlanJobs + 1];  // place of the job's first id in the batch; first[n_jobs] = n
  int64_t tag[kPlanJobs];        // in place (shifted)
};
struct JobTable {  // the same in LDS: lanes index it
  const int64_t* in[kPlanJobs];
  int64_t first[kPlanJobs + 1];
  int64_t tag[kPlanJobs];
};
// Every thread of the workgroup calls; ends with a barrier. The kernels take IdJobs by value as
// their SECOND argument, after one pointer: the table is read here straight out of the kernel
// argument segment (ordinary memory), a lane per entry. Indexing the by-value argument with a
// lane's own index instead makes the compiler copy the whole table into every lane's scratch
// memory first, and a loop with uniform indices reads it one scalar load after the other (both
// measured: 6 and 13 us per kernel).
constexpr int kJobsArgOffset = 8;
template <bool JOBS>
__device__ __forceinline__ void load_jobs(const IdJobs& J, JobTable& t) {
  if constexpr (JOBS) {
    const IdJobs* in_memory = reinterpret_cast<const IdJobs*>(
        reinterpret_cast<uintptr_t>(__builtin_amdgcn_kernarg_segment_ptr()) + kJobsArgOffset);
    // the whole table, used or not: the loads go out without waiting for n_jobs
    const int k = threadIdx.x;
    if (k <= kPlanJobs) {
      t.first[k] = in_memory->first[k];
      if (k < kPlanJobs) {
        t.in[k] = in_memory->in[k];
        t.tag[k] = in_memory->tag[k];
      }
    }
    __syncthreads();
  }
}
// The id at place i of the batch. A reader keeps the job of its last read in registers (where its
// ids lie, its tag, where it ends): reads at ascending places, the usual case, cost one comparison
// more than a plain load; any other place costs a short search of the table.
template <bool JOBS>
struct IdReader {
  const int64_t* ids;  // one array: the batch; jobs: the current job's array moved so that place i is base[i]
  const JobTable* t;
  int n_jobs;
  int64_t mask;
  int j;
  int64_t begin, end, tag;  // of the current job
  __device__ __forceinline__ IdReader(const int64_t* ids_, const IdJobs& J, const JobTable& tab)
      : ids(ids_), t(&tab), n_jobs(J.n_jobs), mask(J.mask), j(-1), begin(0), end(0), tag(0) {}
  __device__ __forceinline__ void enter(int job) {
    j = job;
    begin = t->first[job];
    ids = t->in[job] - begin;
    end = t->first[job + 1];
    tag = t->tag[job];
  }
  // Whether the places a .. b all lie in the current job: then raw() reads them with no test in
  // between, so that a thread's loads stay in flight together.
  __device__ __forceinline__ bool covers(int64_t a, int64_t b) const { return !JOBS || (a >= begin && b < end); }
  __device__ __forceinline__ int64_t raw(int64_t i) const {
    if constexpr (!JOBS) {
      return ids[i];
    } else {
      return (ids[i] & mask) | tag;
    }
  }
  __device__ __forceinline__ void seek(int64_t i) {  // enters the job that holds place i
    int lo = 0, hi = n_jobs;                         // first[lo] <= i < first[hi]
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (t->first[mid] <= i)
        lo = mid;
      else
        hi = mid;
    }
    enter(lo);
    while (i >= end) enter(j + 1);  // the search may land on an empty job before the right one
  }
  __device__ __forceinline__ int64_t at(int64_t i) {  // i at or after the last read's place (after a seek)
    if constexpr (!JOBS) {
      return ids[i];
    } else {
      while (i >= end) enter(j + 1);  // empty jobs are stepped over
      return (ids[i] & mask) | tag;
    }
  }
  __device__ __forceinline__ int64_t at_any(int64_t i) {
    if constexpr (JOBS) {
      if (i >= end || i < begin) seek(i);
    }
    return at(i);
  }
};

// Heavy ids. An id that makes up a sizeable share of the batch (the head of a Zipf distribution, the
// few values of a low-cardinality feature) would put all its occurrences into one bucket and leave
// one workgroup with a hundred times the work of the others. Such ids are found beforehand by
// sampling and get a column of their own in the partition: their occurrences go straight into
// their list (no dedup needed: the column holds one id), and they become the first unique ids.
// kHeavySamples ids at a fixed stride are counted in an LDS table; an id counts as heavy when its
// estimated number of occurrences would fill more than a bucket and a half. The heavy ids come out
// ordered by (sample count descending, id ascending): a function of the input alone.
// Every workgroup of the histogram kernel runs this for itself (the samples are the same 16 KB for
// all of them, read out of the L2; a launch of one workgroup in front of the histogram cost more
// than all of them doing it side by side); the first one leaves the result in global memory for
// the kernels that follow.
struct HeavyScratch {  // LDS of find_heavy
  int64_t t_key[kHeavyTab];
  int32_t t_cnt[kHeavyTab];
  int64_t c_key[kHeavySamples / 8];
  int32_t c_cnt[kHeavySamples / 8];
  int32_t n_cand, minus1;
};
// out_ids [kHeavyMax] (LDS or global); returns their number (uniform). Every thread of a
// workgroup of kPartBlock threads calls; ends with a barrier.
template <bool JOBS>
__device__ __forceinline__ int find_heavy(IdReader<JOBS> rd, int64_t n, HeavyScratch& h, int64_t* out_ids) {
  const int tid = threadIdx.x;
  const int64_t stride = n / kHeavySamples;
  if (stride < 4) return 0;  // a batch this small is no burden for one workgroup per bucket (uniform)
  for (int e = tid; e < kHeavyTab; e += kPartBlock) {
    h.t_key[e] = kSetEmpty;
    h.t_cnt[e] = 0;
  }
  if (tid == 0) {
    h.n_cand = 0;
    h.minus1 = 0;
  }
  __syncthreads();
  constexpr int kMine = kHeavySamples / kPartBlock;
  int64_t k[kMine];
  if constexpr (JOBS) {  // where the samples lie first, then all loads in flight together
    const int64_t* at[kMine];
    int64_t tag[kMine];
#pragma unroll
    for (int x = 0; x < kMine; ++x) {
      const int64_t i = (static_cast<int64_t>(x) * kPartBlock + tid) * stride + stride / 2;
      rd.seek(i);
      at[x] = rd.ids + i;
      tag[x] = rd.tag;
    }
#pragma unroll
    for (int x = 0; x < kMine; ++x) k[x] = (*at[x] & rd.mask) | tag[x];
  } else {
#pragma unroll
    for (int x = 0; x < kMine; ++x) k[x] = rd.raw((static_cast<int64_t>(x) * kPartBlock + tid) * stride + stride / 2);
  }
#pragma unroll
  for (int x = 0; x < kMine; ++x) {
    if (k[x] == kSetEmpty) {  // the table's empty marker is a legal id: counted apart
      atomicAdd(&h.minus1, 1);
      continue;
    }
    int e = static_cast<int>(mix_id(k[x]) >> 40) & (kHeavyTab - 1);
    for (;;) {  // half empty at worst: always ends
      // (an atomic load, not a volatile one: a volatile access loses the LDS address space and
      // becomes a generic load, several times the latency of an LDS read)
      const int64_t c = __hip_atomic_load(&h.t_key[e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      if (c == k[x]) break;
      if (c == kSetEmpty) {
        const unsigned long long old = atomicCAS(reinterpret_cast<unsigned long long*>(&h.t_key[e]),
                                                 static_cast<unsigned long long>(kSetEmpty),
                                                 static_cast<unsigned long long>(k[x]));
        if (old == static_cast<unsigned long long>(kSetEmpty) || old == static_cast<unsigned long long>(k[x])) break;
        continue;  // somebody else's id landed there: look at it again
      }
      e = (e + 1) & (kHeavyTab - 1);
    }
    atomicAdd(&h.t_cnt[e], 1);
  }
  __syncthreads();
  // estimated occurrences = count * stride; heavy from one and a half buckets' worth, and never on
  // fewer than 8 samples (so at most kHeavySamples / 8 candidates)
  const int64_t want = (3 * kBucketIds / 2 + stride - 1) / stride;
  const int32_t thr = static_cast<int32_t>(want < 8 ? 8 : (want > kHeavySamples ? kHeavySamples + 1 : want));
  for (int e = tid; e <= kHeavyTab; e += kPartBlock) {
    const int32_t c = e < kHeavyTab ? h.t_cnt[e] : h.minus1;
    if (c >= thr) {
      const int at = atomicAdd(&h.n_cand, 1);
      h.c_key[at] = e < kHeavyTab ? h.t_key[e] : kSetEmpty;
      h.c_cnt[at] = c;
    }
  }
  __syncthreads();
  const int ncand = h.n_cand;
  for (int i = tid; i < ncand; i += kPartBlock) {  // rank by (count descending, id ascending): the first kHeavyMax stay
    int rank = 0;
    const int32_t ci = h.c_cnt[i];
    const uint64_t ki = static_cast<uint64_t>(h.c_key[i]);
    for (int j = 0; j < ncand; ++j) {
      const int32_t cj = h.c_cnt[j];
      rank += (cj > ci || (cj == ci && static_cast<uint64_t>(h.c_key[j]) < ki)) ? 1 : 0;
    }
    if (rank < kHeavyMax) out_ids[rank] = h.c_key[i];
  }
  __syncthreads();
  return ncand < kHeavyMax ? ncand : kHeavyMax;
}

// The heavy ids as an LDS table for the partition kernels: h_slot [kHeavySlots] holds the index of
// a heavy id or -1, h_key its id (at most a quarter full: most ids end their search on the first
// word they read). Every thread of the workgroup calls; ends with a barrier.
__device__ __forceinline__ int heavy_table(const int64_t* heavy_ids, int n_heavy, int32_t* h_slot, int64_t* h_key) {
  if (n_heavy == 0) return 0;  // uniform
  for (int e = threadIdx.x; e < kHeavySlots; e += blockDim.x) h_slot[e] = -1;
  __syncthreads();
  if (static_cast<int>(threadIdx.x) < n_heavy) {
    const int64_t key = heavy_ids[threadIdx.x];
    int e = static_cast<int>(mix_id(key) >> 24) & (kHeavySlots - 1);
    while (atomicCAS(&h_slot[e], -1, static_cast<int32_t>(threadIdx.x)) != -1) e = (e + 1) & (kHeavySlots - 1);
    h_key[e] = key;
  }
  __syncthreads();
  return n_heavy;
}
__device__ __forceinline__ int load_heavy(const int64_t* __restrict__ heavy_ids, const int32_t* __restrict__ heavy_n,
                                          int32_t* h_slot, int64_t* h_key) {
  return heavy_table(heavy_ids, *heavy_n, h_slot, h_key);
}
// Index of `key` among the heavy ids, or -1.
__device__ __forceinline__ int heavy_index(int64_t key, uint64_t mixed, const int32_t* h_slot, const int64_t* h_key) {
  int e = static_cast<int>(mixed >> 24) & (kHeavySlots - 1);
  for (;;) {
    const int32_t h = h_slot[e];
    if (h < 0) return -1;
    if (h_key[e] == key) return h;
    e = (e + 1) & (kHeavySlots - 1);
  }
}
// Column of an id in the partition: its own when it is heavy, else that of its bucket.
__device__ __forceinline__ int column_of(int64_t key, int nb_log2, int n_heavy, const int32_t* h_slot,
                                         const int64_t* h_key) {
  const uint64_t mixed = mix_id(key);
  if (n_heavy > 0) {
    const int h = heavy_index(key, mixed, h_slot, h_key);
    if (h >= 0) return h;
  }
  return kHeavyMax + bucket_of_mix(mixed, nb_log2);
}

// atomicAdd(&arr[e], 1) for every lane with `active`, each lane getting back a value that no other
// lane gets for the same entry. Ids of low-cardinality features repeat thousands of times in a
// bucket, and atomics of one wave on one LDS word are served one after the other (some 3 ns each:
// a bucket with a 6500-fold id spent 20 us there); so when many lanes of the wave name the entry
// of the first (or of the last) active lane, one of them adds their number and hands out the places.
__device__ __forceinline__ int32_t wave_add_one(int32_t* arr, int e, bool active) {
  int32_t result = 0;
  if (__ballot(active) == 0) return result;  // uniform
  const int lane = threadIdx.x & (kWave - 1);
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    const uint64_t todo = __ballot(active);
    if (todo == 0) break;
    const int leader = it == 0 ? __ffsll(static_cast<unsigned long long>(todo)) - 1 : 63 - __clzll(todo);
    const int e_l = __shfl(e, leader, kWave);
    const uint64_t same = __ballot(active && e == e_l);
    const int n_same = __popcll(same);
    if (n_same < 8) continue;
    int32_t base = 0;
    if (lane == leader) base = atomicAdd(&arr[e_l], n_same);
    base = __shfl(base, leader, kWave);
    if (active && e == e_l) {
      result = base + __popcll(same & ((uint64_t(1) << lane) - 1));
      active = false;
    }
  }
  if (active) result = atomicAdd(&arr[e], 1);
  return result;
}

// arr[e] += 1 for every lane with `active`, lanes that name the same entry adding up among themselves first
// when there are many of them (see wave_add_one, which also hands out the places).
__device__ __forceinline__ void wave_count_one(int32_t* arr, int e, bool active) {
  if (__ballot(active) == 0) return;  // uniform
  const int lane = threadIdx.x & (kWave - 1);
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    const uint64_t todo = __ballot(active);
    if (todo == 0) return;
    const int leader = it == 0 ? __ffsll(static_cast<unsigned long long>(todo)) - 1 : 63 - __clzll(todo);
    const int e_l = __shfl(e, leader, kWave);
    const uint64_t same = __ballot(active && e == e_l);
    if (__popcll(same) < 8) continue;
    if (lane == leader) atomicAdd(&arr[e_l], __popcll(same));
    if (e == e_l) active = false;
  }
  if (active) atomicAdd(&arr[e], 1);
}

// hist: the heavy ids (found here, see find_heavy; left in heavy_ids / heavy_n by the first
// workgroup), then ids per (row, column); columns: the heavy ids, then the buckets
template <bool JOBS>
__global__ void __launch_bounds__(kPartBlock)
plan_hist_kernel(const int64_t* __restrict__ ids, IdJobs jobs, PlanGeom g, int64_t* __restrict__ heavy_ids,
                 int32_t* __restrict__ heavy_n, int32_t* __restrict__ hist, int64_t* __restrict__ counts,
                 int32_t* __restrict__ sync) {
  __shared__ JobTable s_jobs;
  load_jobs<JOBS>(jobs, s_jobs);
  IdReader<JOBS> rd(ids, jobs, s_jobs);
  // the sampling's tables first, the histogram [kHeavyMax + nb] afterwards, in the same memory
  extern __shared__ __align__(16) unsigned char l_raw[];
  int32_t* l_hist = reinterpret_cast<int32_t*>(l_raw);
  __shared__ int32_t h_slot[kHeavySlots];
  __shared__ int64_t h_key[kHeavySlots];
  __shared__ int64_t h_ids[kHeavyMax];
  const int tid = threadIdx.x;
  const int nc = kHeavyMax + (1 << g.nb_log2);
  if (blockIdx.x == 0) {
    if (tid < 2) counts[tid] = 0;
    if (tid < 4) sync[tid] = 0;  // [1] finished workgroups of the bucket kernel, [2] of the row assignment, [3] new keys
  }
  // the first kTile ids of the tile (all of it unless the batch is huge) are requested now and
  // arrive while the heavy ids are looked for
  const int64_t lo = static_cast<int64_t>(blockIdx.x) * g.tile, hi = min(g.n, lo + g.tile);
  const int64_t hi_regs = min(hi, lo + kTile);
  int64_t k_first[kTilePer];
  {
    IdReader<JOBS> rt = rd;
    if (JOBS && lo < hi_regs) rt.seek(lo);
    if (lo < hi_regs && rt.covers(lo, hi_regs - 1)) {  // the whole stretch in one array (uniform)
#pragma unroll
      for (int x = 0; x < kTilePer; ++x) {
        const int64_t i = lo + tid + x * kPartBlock;
        k_first[x] = i < hi_regs ? rt.raw(i) : 0;
      }
    } else {
#pragma unroll
      for (int x = 0; x < kTilePer; ++x) {
        const int64_t i = lo + tid + x * kPartBlock;
        k_first[x] = i < hi_regs ? rt.at_any(i) : 0;
      }
    }
  }
  const int n_found = find_heavy<JOBS>(rd, g.n, *reinterpret_cast<HeavyScratch*>(l_raw), h_ids);
  if (blockIdx.x == 0) {
    if (tid < n_found) heavy_ids[tid] = h_ids[tid];
    if (tid == 0) *heavy_n = n_found;
  }
  for (int b = tid; b < nc; b += kPartBlock) l_hist[b] = 0;
  const int n_heavy = heavy_table(h_ids, n_found, h_slot, h_key);
  __syncthreads();
  auto count = [&](int64_t key, bool valid) {
    const int c = column_of(key, g.nb_log2, n_heavy, h_slot, h_key);
    const bool heavy = valid && c < kHeavyMax;
    if (n_heavy > 0) wave_count_one(l_hist, c, heavy);  // a heavy id is many lanes on one word
    if (valid && !heavy) atomicAdd(&l_hist[c], 1);
  };
#pragma unroll
  for (int x = 0; x < kTilePer; ++x) count(k_first[x], lo + tid + x * kPartBlock < hi_regs);
  if (JOBS && hi_regs + tid < hi) rd.seek(hi_regs + tid);
  for (int64_t i0 = hi_regs + tid; i0 < hi; i0 += 4 * kPartBlock) {  // four loads in flight
    int64_t k[4];
    if (rd.covers(i0, min(hi - 1, i0 + 3 * kPartBlock))) {
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        const int64_t i = i0 + x * kPartBlock;
        k[x] = i < hi ? rd.raw(i) : 0;
      }
    } else {  // the places straddle arrays
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        const int64_t i = i0 + x * kPartBlock;
        k[x] = i < hi ? rd.at_any(i) : 0;
      }
    }
#pragma unroll
    for (int x = 0; x < 4; ++x) count(k[x], i0 + x * kPartBlock < hi);
  }
  __syncthreads();
  int32_t* row = hist + static_cast<int64_t>(blockIdx.x) * nc;
  for (int b = tid; b < nc; b += kPartBlock) row[b] = l_hist[b];
}

// colscan: for every bucket, exclusive scan of its histogram column over the rows, in place, and
// the bucket's total. Workgroup = kColBuckets buckets x (1024 / kColBuckets) groups of rows.
constexpr int kColBuckets = 16;
constexpr int kColGroups = 1024 / kColBuckets;
__global__ void __launch_bounds__(1024)
plan_colscan_kernel(int32_t* __restrict__ hist, PlanGeom g, int32_t* __restrict__ bucket_total) {
  __shared__ int32_t part[kColGroups][kColBuckets + 1];
  const int nb = kHeavyMax + (1 << g.nb_log2);  // columns (a multiple of kColBuckets)
  const int t = threadIdx.x;
  const int bl = t % kColBuckets, rg = t / kColBuckets;
  const int b = blockIdx.x * kColBuckets + bl;
  const int per_rows = (g.rows + kColGroups - 1) / kColGroups;
  const int r_lo = min(g.rows, rg * per_rows), r_hi = min(g.rows, r_lo + per_rows);
  int32_t sum = 0;
  for (int r = r_lo; r < r_hi; ++r) sum += hist[static_cast<int64_t>(r) * nb + b];
  part[rg][bl] = sum;
  __syncthreads();
  int32_t run = 0;
  for (int q = 0; q < rg; ++q) run += part[q][bl];
  for (int r = r_lo; r < r_hi; ++r) {
    const int64_t at = static_cast<int64_t>(r) * nb + b;
    const int32_t c = hist[at];
    hist[at] = run;
    run += c;
  }
  if (rg == kColGroups - 1) bucket_total[b] = run;
}

// Exclusive scan of in[0 .. nb) into LDS (start[0 .. nb], start[nb] = the total) by the calling
// workgroup of kPartBlock threads: a thread sums its own stretch, the waves scan those sums with
// shuffles, one barrier joins the waves. `in` may be global or LDS memory (in == start is fine);
// `partial` is scratch of kPartBlock / kWave words. Ends with a barrier.
__device__ __forceinline__ void scan_counts(const int32_t* in, int nb, int32_t* start, int32_t* partial) {
  const int t = threadIdx.x, lane = t & (kWave - 1), wave = t / kWave;
  const int per = (nb + kPartBlock - 1) / kPartBlock;
  const int lo = min(nb, t * per), hi = min(nb, lo + per);
  int32_t sum = 0;
  for (int q = lo; q < hi; ++q) sum += in[q];
  int32_t incl = sum;
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    const int32_t y = __shfl_up(incl, o, kWave);
    if (lane >= o) incl += y;
  }
  if (lane == kWave - 1) partial[wave] = incl;
  __syncthreads();
  int32_t run = incl - sum, total = 0;
#pragma unroll
  for (int w = 0; w < kPartBlock / kWave; ++w) {
    const int32_t c = partial[w];
    if (w < wave) run += c;
    total += c;
  }
  for (int q = lo; q < hi; ++q) {
    const int32_t c = in[q];
    start[q] = run;
    run += c;
  }
  if (t == 0) start[nb] = total;
  __syncthreads();
}

// Where every column's entries start in the partitioned arrays (start[0 .. nc), start[nc] = n), by
// the calling workgroup of kPartBlock threads, from the column totals. The columns are NOT laid
// out in the order of their index: the heavy ids' columns come first (as always), then the buckets
// that hold more than one and a half times the average, then the others, each class in the order of
// the index. The bucket kernel takes the buckets in the order of this layout, one workgroup each,
// and the layout is the order of the unique ids; so the buckets that take longest (a bucket with
// three times the entries keeps its workgroup almost twice as long) are dispatched first and the
// short ones fill in behind them, instead of a long one starting last and the whole chip waiting
// for it. Still a function of the input alone. rank_start (global, may be NULL): written with the
// same starts indexed by the column's place in the layout ([nc + 1]), what the bucket kernel reads.
// `partial` is scratch of kPartBlock words. Ends with a barrier.
__device__ __forceinline__ void column_starts(const int32_t* __restrict__ total, int nc, int64_t n, int32_t* start,
                                              int32_t* partial, int32_t* __restrict__ rank_start) {
  unsigned long long* part64 =  // [2][waves], at the first 8-byte boundary of the scratch
      reinterpret_cast<unsigned long long*>((reinterpret_cast<uintptr_t>(partial) + 7) & ~static_cast<uintptr_t>(7));
  const int t = threadIdx.x, lane = t & (kWave - 1), wave = t / kWave;
  constexpr int n_waves = kPartBlock / kWave;
  const int per = (nc + kPartBlock - 1) / kPartBlock;
  const int lo = min(nc, t * per), hi = min(nc, lo + per);
  const int64_t fat_from = 3 * (n / (nc - kHeavyMax)) / 2 + 32;  // entries from which a bucket goes first
  auto is_first = [&](int c, int32_t cnt) { return c < kHeavyMax || cnt > fat_from; };
  // per class one word: entries << 14 | columns (n < 2^31 entries, fewer than 2^14 columns)
  unsigned long long sum[2] = {0, 0};
  for (int c = lo; c < hi; ++c) {
    const int32_t cnt = total[c];
    sum[is_first(c, cnt) ? 0 : 1] += (static_cast<unsigned long long>(cnt) << 14) | 1ull;
  }
  unsigned long long incl[2] = {sum[0], sum[1]};
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const unsigned long long y = __shfl_up(incl[k], o, kWave);
      if (lane >= o) incl[k] += y;
    }
  }
  if (lane == kWave - 1) {
    part64[wave] = incl[0];
    part64[n_waves + wave] = incl[1];
  }
  __syncthreads();
  unsigned long long run[2] = {incl[0] - sum[0], incl[1] - sum[1]}, all_first = 0;
#pragma unroll
  for (int w = 0; w < n_waves; ++w) {
    const unsigned long long c0 = part64[w], c1 = part64[n_waves + w];
    if (w < wave) {
      run[0] += c0;
      run[1] += c1;
    }
    all_first += c0;
  }
  run[1] += all_first;  // the second class lies behind all of the first
  for (int c = lo; c < hi; ++c) {
    const int32_t cnt = total[c];
    const int k = is_first(c, cnt) ? 0 : 1;
    const int32_t at = static_cast<int32_t>(run[k] >> 14);
    start[c] = at;
    if (rank_start) rank_start[run[k] & 0x3fff] = at;
    run[k] += (static_cast<unsigned long long>(cnt) << 14) | 1ull;
  }
  if (t == 0) {
    start[nc] = static_cast<int32_t>(n);
    if (rank_start) rank_start[nc] = static_cast<int32_t>(n);
  }
  __syncthreads();
}

// What the partition kernels need to put the occurrences of heavy ids straight into their lists.
struct HeavyArgs {
  const int64_t* ids;   // [kHeavyMax]
  const int32_t* n;     // [1]
  int32_t* list;        // the plan's list_out
  int32_t* inverse;     // may be NULL
  int32_t* pos_out;     // may be NULL
};

// scatter: (id, position) of every occurrence goes to its column: for a bucket into bkt_id / bkt_pos,
// for a heavy id the position goes into the plan's list at once (list space and bucket space are
// the same index space: a column's entries are its list entries). Every workgroup scans the column
// totals for itself (a thousand words), so no kernel stands between the column scan and this one;
// the first workgroup also leaves bucket_start [columns + 1] for the bucket kernel and clears that
// kernel's look-back words.
template <bool JOBS>
__global__ void __launch_bounds__(kPartBlock)
plan_scatter_kernel(const int64_t* __restrict__ ids, IdJobs jobs, PlanGeom g, HeavyArgs hv, const int32_t* __restrict__ off,
                    const int32_t* __restrict__ bucket_total, int32_t* __restrict__ bucket_start,
                    unsigned long long* __restrict__ agg, int64_t* __restrict__ bkt_id,
                    int32_t* __restrict__ bkt_pos) {
  extern __shared__ int32_t cursor[];  // [nc + 1], then kPartBlock words of scan scratch
  __shared__ int32_t h_slot[kHeavySlots];
  __shared__ int64_t h_key[kHeavySlots];
  __shared__ JobTable s_jobs;
  load_jobs<JOBS>(jobs, s_jobs);
  IdReader<JOBS> rd(ids, jobs, s_jobs);
  const int tid = threadIdx.x;
  const int nb = 1 << g.nb_log2, nc = kHeavyMax + nb;
  const int n_heavy = load_heavy(hv.ids, hv.n, h_slot, h_key);
  column_starts(bucket_total, nc, g.n, cursor, cursor + nc + 1, blockIdx.x == 0 ? bucket_start : nullptr);
  if (blockIdx.x == 0) {
    for (int b = tid; b < nb; b += kPartBlock) agg[b] = 0;
  }
  const int32_t* off_row = off + static_cast<int64_t>(blockIdx.x) * nc;
  __syncthreads();
  for (int b = tid; b < nc; b += kPartBlock) cursor[b] += off_row[b];
  __syncthreads();
  const int64_t lo = static_cast<int64_t>(blockIdx.x) * g.tile, hi = min(g.n, lo + g.tile);
  if (JOBS && lo + tid < hi) rd.seek(lo + tid);
  for (int64_t i0 = lo + tid; i0 < hi; i0 += 4 * kPartBlock) {
    int64_t k[4];
    if (rd.covers(i0, min(hi - 1, i0 + 3 * kPartBlock))) {
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        const int64_t i = i0 + x * kPartBlock;
        k[x] = i < hi ? rd.raw(i) : 0;
      }
    } else {  // the places straddle arrays
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        const int64_t i = i0 + x * kPartBlock;
        k[x] = i < hi ? rd.at_any(i) : 0;
      }
    }
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      const int64_t i = i0 + x * kPartBlock;
      const int c = column_of(k[x], g.nb_log2, n_heavy, h_slot, h_key);
      const bool heavy = i < hi && c < kHeavyMax;
      int32_t p = 0;
      if (n_heavy > 0) p = wave_add_one(cursor, c, heavy);
      if (i < hi && !heavy) p = atomicAdd(&cursor[c], 1);
      if (i >= hi) continue;
      if (c < kHeavyMax) {
        hv.list[p] = static_cast<int32_t>(i);
        if (hv.inverse) hv.inverse[i] = c;
        if (hv.pos_out) hv.pos_out[i] = p;
      } else {
        bkt_id[p] = k[x];
        bkt_pos[p] = static_cast<int32_t>(i);
      }
    }
  }
}

// scatter in runs, for tiles of at most kTile ids and few enough buckets that a tile sends several
// ids to each: a workgroup ranks its ids inside their buckets (LDS counters), orders them by bucket
// in LDS (id, place in the tile, column) and writes them out in that order, so that the ids a tile
// sends to one bucket leave together as one run of consecutive words instead of one scattered
// 8-byte and one scattered 4-byte store per id (scattered stores run at some 1e11 per second on
// this part whatever their size). The tile in LDS is 12 bytes per id, so a compute unit holds one
// workgroup (a second 1024-thread workgroup does not start beside the first on this part anyway);
// the host sizes the tiles so that a batch of up to cus * kTile ids is one round of workgroups.
// The tile's ids are requested first and arrive while the column starts are worked out; the
// write-out phase reads LDS only, so nothing waits for earlier stores (loads and stores share one
// counter on this part: with a load from global memory per id in that phase, every round of it
// waited for the stores of the round before, 11 us of a 25 us workgroup).
constexpr size_t scatter_runs_lds(int nc) {
  return sizeof(int32_t) * (2 * (nc + 1) + kPartBlock) + 8 + (sizeof(int64_t) + 2 * sizeof(uint16_t)) * kTile;
}
template <bool JOBS>
__global__ void __launch_bounds__(kPartBlock)
plan_scatter_runs_kernel(const int64_t* __restrict__ ids, IdJobs jobs, PlanGeom g, HeavyArgs hv,
                         const int32_t* __restrict__ off, const int32_t* __restrict__ bucket_total,
                         int32_t* __restrict__ bucket_start, unsigned long long* __restrict__ agg,
                         int64_t* __restrict__ bkt_id, int32_t* __restrict__ bkt_pos) {
  extern __shared__ int32_t lds[];
  __shared__ int32_t h_slot[kHeavySlots];
  __shared__ int64_t h_key[kHeavySlots];
  __shared__ JobTable s_jobs;
  load_jobs<JOBS>(jobs, s_jobs);
  IdReader<JOBS> rd(ids, jobs, s_jobs);
  const int tid = threadIdx.x;
  const int nb = 1 << g.nb_log2, nc = kHeavyMax + nb;
  int32_t* gbase = lds;               // [nc + 1] where the tile's ids of a column go
  int32_t* first = lds + nc + 1;      // [nc + 1] ids of the tile per column, then where they start in column order
  int32_t* partial = first + nc + 1;  // [kPartBlock] scan scratch
  int64_t* s_key = reinterpret_cast<int64_t*>((reinterpret_cast<uintptr_t>(partial + kPartBlock) + 7) &
                                              ~static_cast<uintptr_t>(7));  // [kTile] the tile's ids in column order
  uint16_t* s_at = reinterpret_cast<uint16_t*>(s_key + kTile);              // [kTile] their places in the tile
  uint16_t* s_col = s_at + kTile;                                           // [kTile] and their columns
  const int64_t lo = static_cast<int64_t>(blockIdx.x) * g.tile;
  const int n_here = static_cast<int>(min(g.n, lo + g.tile) - lo);
  int64_t k[kTilePer];
  if (JOBS && n_here > 0) rd.seek(lo);
  const bool one_job = n_here > 0 && rd.covers(lo, lo + n_here - 1);  // the whole tile in one array (uniform)
  if (one_job) {
#pragma unroll
    for (int x = 0; x < kTilePer; ++x) {  // all loads in flight
      const int i = tid + x * kPartBlock;
      k[x] = i < n_here ? rd.raw(lo + i) : 0;
    }
  } else {
#pragma unroll
    for (int x = 0; x < kTilePer; ++x) {
      const int i = tid + x * kPartBlock;
      k[x] = i < n_here ? rd.at_any(lo + i) : 0;
    }
  }
  for (int b = tid; b <= nc; b += kPartBlock) first[b] = 0;
  const int n_heavy = load_heavy(hv.ids, hv.n, h_slot, h_key);
  column_starts(bucket_total, nc, g.n, gbase, partial, blockIdx.x == 0 ? bucket_start : nullptr);
  if (blockIdx.x == 0) {
    for (int b = tid; b < nb; b += kPartBlock) agg[b] = 0;
  }
  const int32_t* off_row = off + static_cast<int64_t>(blockIdx.x) * nc;
  for (int b = tid; b < nc; b += kPartBlock) gbase[b] += off_row[b];  // column_starts ended with a barrier
  uint16_t rank[kTilePer], col[kTilePer];
#pragma unroll
  for (int x = 0; x < kTilePer; ++x) {
    const bool valid = tid + x * kPartBlock < n_here;
    col[x] = static_cast<uint16_t>(column_of(k[x], g.nb_log2, n_heavy, h_slot, h_key));
    const bool heavy = valid && col[x] < kHeavyMax;
    rank[x] = 0;
    if (n_heavy > 0) rank[x] = static_cast<uint16_t>(wave_add_one(first, col[x], heavy));
    if (valid && !heavy) rank[x] = static_cast<uint16_t>(atomicAdd(&first[col[x]], 1));
  }
  __syncthreads();
  scan_counts(first, nc, first, partial);  // counts -> starts in column order
#pragma unroll
  for (int x = 0; x < kTilePer; ++x) {
    const int i = tid + x * kPartBlock;
    if (i < n_here) {
      const int j = first[col[x]] + rank[x];
      s_key[j] = k[x];
      s_at[j] = static_cast<uint16_t>(i);
      s_col[j] = col[x];
    }
  }
  __syncthreads();
  for (int j = tid; j < n_here; j += kPartBlock) {
    const int b = s_col[j];
    const int32_t d = gbase[b] + (j - first[b]);
    const int32_t at = static_cast<int32_t>(lo) + s_at[j];
    if (b < kHeavyMax) {
      hv.list[d] = at;
      if (hv.inverse) hv.inverse[at] = b;
      if (hv.pos_out) hv.pos_out[at] = d;
    } else {
      bkt_id[d] = s_key[j];
      bkt_pos[d] = at;
    }
  }
}

// A new key of the fused find-or-insert: where it sits in the id map, which unique id it is.
struct alignas(16) NewRec {
  int64_t slot;
  int64_t u;
};

struct BucketArgs {
  const int64_t* bkt_id;
  const int32_t* bkt_pos;
  const int32_t* bucket_start;  // [kHeavyMax + nb + 1]: the columns of the heavy ids, then the buckets
  const int64_t* heavy_ids;     // [kHeavyMax]
  const int32_t* heavy_n;       // [1]
  PlanGeom g;
  unsigned long long* agg;  // [nb] look-back words: distinct ids per bucket
  int32_t* new_count;       // [1 + nb] keys new to the id map: among the heavy ids, then per bucket
  int32_t* sync;            // [1] = workgroups of the bucket kernel that are done, [2] = of the row assignment
  int64_t* unique_out;
  int32_t* inverse;    // may be NULL
  int32_t* row_start;
  int32_t* list;
  int32_t* pos_out;    // may be NULL
  int64_t* counts;
  int32_t* hot_items;
  int64_t hot_cap;
  volatile int64_t* staged;  // pinned host words (unique count, soft-error bits) or NULL
  int* err;
  uint32_t spin_limit;
  // fused find-or-insert in the id map
  Slot* table;
  uint64_t mask;
  int64_t* index_out;
  int64_t* state;
  volatile int64_t* mirror;
  int64_t seq;
  NewRec* new_list;  // [n] the new keys of a bucket, at the bucket's own entries
};

__device__ __forceinline__ bool in_round(uint64_t mixed, uint32_t rounds, uint32_t round) {
  return rounds == 1 || static_cast<uint32_t>((mixed >> 8) & 0xffffff) % rounds == round;
}

// Exclusive scan of a 64-bit value over the kBucketBlock threads of a workgroup (two counters
// packed in one word); `total` is the sum over all threads. Ends with a barrier.
__device__ __forceinline__ unsigned long long block_scan_u64(unsigned long long v, unsigned long long* s_wave,
                                                             unsigned long long& total) {
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  unsigned long long incl = v;
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    const unsigned long long y = __shfl_up(incl, o, kWave);
    if (lane >= o) incl += y;
  }
  __syncthreads();  // s_wave may still be read from the previous scan
  if (lane == kWave - 1) s_wave[wave] = incl;
  __syncthreads();
  unsigned long long before = incl - v, tot = 0;
#pragma unroll
  for (int w = 0; w < kBucketBlock / kWave; ++w) {
    const unsigned long long c = s_wave[w];
    if (w < wave) before += c;
    tot += c;
  }
  total = tot;
  return before;
}

constexpr unsigned long long kAggFlag = 1ull << 62, kPrefixFlag = 2ull << 62, kAggValue = (1ull << 62) - 1;

// Sum of the distinct-id counts of all buckets before bucket b, by the whole workgroup: thread t
// reads the look-back word of bucket hi - t (nearest first), so one round covers the 512 nearest
// predecessors; rounds go on until a word carries an inclusive prefix. Every predecessor has
// started (workgroups are dispatched in the order of their index) and publishes its word before it waits for anybody,
// so each word arrives after a bounded time; a wait that outlasts spin_limit polls raises the
// plan-overflow error bit and goes on with zero. A word carries its whole message (flag and value
// in one 64-bit atomic), so relaxed device-scope atomics are enough: nothing else has to become
// visible with it. (Release / acquire at device scope write back and invalidate the whole L2 of the
// XCD on this part: tens of microseconds per workgroup.) Every thread calls; ends with a barrier.
__device__ __forceinline__ int64_t look_back(unsigned long long* __restrict__ agg, int b, int n_heavy,
                                             uint32_t spin_limit, int* err,
                                             unsigned long long* s_look /* [kBucketBlock / kWave] */) {
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  int64_t sum = 0;
  for (int hi = b - 1;; hi -= kBucketBlock) {
    const int j = hi - static_cast<int>(threadIdx.x);
    // before the first bucket: the heavy ids, which are the first unique ids
    unsigned long long w = kPrefixFlag | static_cast<unsigned long long>(n_heavy);
    if (j >= 0) {
      uint32_t polls = 0;
      for (;;) {
        w = __hip_atomic_load(&agg[j], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if ((w >> 62) != 0) break;
        if (++polls > spin_limit) {
          raise_device_error(err, RECIS_DEVERR_PLAN_OVERFLOW);
          w = kPrefixFlag;  // goes on with zero
          break;
        }
        __builtin_amdgcn_s_sleep(2);
      }
    }
    const uint64_t is_prefix = __ballot((w >> 62) == 2);
    const int first = is_prefix ? __ffsll(static_cast<unsigned long long>(is_prefix)) - 1 : kWave;
    unsigned long long v = lane <= first ? (w & kAggValue) : 0;
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
    __syncthreads();  // s_look may still be read
    if (lane == 0) s_look[wave] = v | (is_prefix ? kPrefixFlag : 0ull);
    __syncthreads();
    bool done = false;
#pragma unroll
    for (int q = 0; q < kBucketBlock / kWave; ++q) {  // waves hold nearer buckets first
      if (done) continue;
      const unsigned long long x = s_look[q];
      sum += static_cast<int64_t>(x & kAggValue);
      done = (x >> 62) != 0;
    }
    if (done) break;
  }
  __syncthreads();
  return sum;
}

// One thread of a workgroup of the bucket kernel that is done calls this: the workgroup that
// finishes last sends the count and the soft-error bits to the host (pinned words: no copy kernel
// needed). Only then has every workgroup raised what it had to raise.
__device__ __forceinline__ void finish_ticket(const BucketArgs& a) {
  // this thread's earlier stores must have reached the L2 before its ticket does; a fence of
  // workgroup scope waits for exactly that (one of device scope would write back the whole L2)
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  if (atomicAdd(&a.sync[1], 1) == (1 << a.g.nb_log2)) {  // the buckets and the heavy ids' workgroup
    a.staged[1] = __hip_atomic_load(a.err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    a.staged[0] = __hip_atomic_load(&a.counts[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// The heavy ids' share of what the bucket kernel writes per unique id: heavy id h is unique id h, its
// list is its column (filled by the scatter kernel). One workgroup, a thread per heavy id.
template <bool PROBE>
__device__ __forceinline__ void heavy_rows(const BucketArgs& a, int n_heavy, unsigned long long* s_wave) {
  const int h = threadIdx.x;
  int32_t my_new = 0, my_empty = 0;
  int64_t row = -1;
  if (h < n_heavy) {
    const int64_t key = a.heavy_ids[h];
    const int32_t start = a.bucket_start[h], n_here = a.bucket_start[h + 1] - start;
    a.unique_out[h] = key;
    a.row_start[h] = start;
    if (a.hot_cap > 0 && n_here > kHotLen) {
      const int n_items = (n_here + kHotChunk - 1) / kHotChunk;
      const int64_t base = static_cast<int64_t>(atomicAdd(reinterpret_cast<unsigned long long*>(&a.counts[1]),
                                                          static_cast<unsigned long long>(n_items)));
      for (int c = 0; c < n_items; ++c) {
        if (base + c < a.hot_cap) {
          a.hot_items[2 * (base + c)] = h;
          a.hot_items[2 * (base + c) + 1] = c;
        }
      }
    }
    if constexpr (PROBE) {
      if (key == kEmpty || key == kTomb) {
        raise_device_error(a.err, RECIS_DEVERR_INDEX_RANGE);  // the map's reserved keys
      } else {
        const uint64_t home = home_slot(key, a.mask);
        const longlong2 hint = *reinterpret_cast<const longlong2*>(&a.table[home]);
        int64_t value = -1, slot = -1;
        bool took_empty = false;
        switch (probe_or_claim(a.table, a.mask, key, home, hint, -2, &value, &slot, &took_empty)) {
          case kProbeFound:
            row = value;
            break;
          case kProbeClaimed:
            row = -(slot + 2);
            my_new = 1;
            my_empty = took_empty ? 1 : 0;
            break;
          default:
            raise_device_error(a.err, RECIS_DEVERR_TABLE_FULL);
            break;
        }
      }
      a.index_out[h] = row;
    }
  }
  if constexpr (PROBE) {  // new keys among them, in the order of the unique ids, at the first column's entries
    unsigned long long new_total;
    const unsigned long long new_before = block_scan_u64(
        (static_cast<unsigned long long>(my_empty) << 32) | static_cast<unsigned long long>(my_new), s_wave, new_total);
    if (threadIdx.x == 0) {
      if ((new_total >> 32) != 0) atomicAdd(reinterpret_cast<unsigned long long*>(&a.state[ST_OCC]), new_total >> 32);
      a.new_count[0] = static_cast<int32_t>(new_total & 0xffffffffull);
      if (new_total & 0xffffffffull) atomicAdd(&a.sync[3], static_cast<int32_t>(new_total & 0xffffffffull));
    }
    if (my_new) {
      NewRec nr;
      nr.u = h;
      nr.slot = -(row + 2);
      a.new_list[a.bucket_start[0] + static_cast<int32_t>(new_before & 0xffffffffull)] = nr;
    }
  }
  __syncthreads();
  if (threadIdx.x == 0 && a.staged) finish_ticket(a);
}

// bucket: one workgroup per bucket, in the order of the workgroup index. The bucket's ids are
// deduplicated in an LDS hash table with linear probing that never wraps. Insertion is the
// phase-concurrent, history-independent kind: of two ids that want the same entry the one with the
// smaller unsigned value stays and the other moves on, so the table ends up the same whatever the
// order of the insertions, and the position of an id in the table is a function of the input
// alone. That position orders the unique ids: one scan over the table gives every id its rank and
// the start of its list. The number of distinct ids of all earlier buckets comes from a decoupled
// look-back over one word per bucket. With PROBE, every distinct id is looked up in the id map
// from here (find or claim); ids the map did not hold are listed per bucket, in the order of the
// unique ids, for plan_assign_new_kernel to give them rows.
// A bucket with more distinct ids than the table takes is worked in `rounds` hash-partitioned
// rounds (first a dry run over all rounds to find a round count that fits).
template <bool PROBE>
__global__ void __launch_bounds__(kBucketBlock, 4)
plan_bucket_kernel(BucketArgs a) {
  __shared__ int64_t l_key[kTabAll + 1];
  __shared__ int32_t l_cnt[kTabAll + 1];  // occurrences of the entry; after ranking: its next free list position
  __shared__ int32_t l_u[kTabAll + 1];    // rank of the entry among the distinct ids of the round
  __shared__ uint16_t l_ent[kTabAll + 1]; // the entry of every rank
  __shared__ unsigned long long s_wave[kBucketBlock / kWave];
  __shared__ int s_overflow;
  __shared__ int s_claimed;  // entries of the table that the current build has taken
  const int tid = threadIdx.x;
  const int nb_log2 = a.g.nb_log2;
  // Buckets are taken in the order of the workgroup index. The look-back below waits for the
  // workgroups of lower index; those have been dispatched before this one (the dispatcher walks
  // the grid in order), so they run and publish without waiting for anything later. A ticket from
  // a global counter would say the same, but a thousand atomics on one word are served one after
  // the other (25 ns each on this part: the last workgroup would start 25 us late).
  const int b = blockIdx.x;
  const int n_heavy = *a.heavy_n;
  if (b == (1 << nb_log2)) {  // the workgroup after the last bucket's: the heavy ids
    heavy_rows<PROBE>(a, n_heavy, s_wave);
    return;
  }
  const int32_t r_lo = a.bucket_start[kHeavyMax + b], r_hi = a.bucket_start[kHeavyMax + b + 1];
  for (int e = tid; e <= kTabAll; e += kBucketBlock) {
    l_key[e] = kSetEmpty;
    l_cnt[e] = 0;
  }
  if (tid == 0) {
    s_overflow = 0;
    s_claimed = 0;
  }
  __syncthreads();
  int e_reg[kRegs];  // table entry of the thread's first kRegs records (-2: none / not of this round)
  int32_t pos_reg[kRegs];
#pragma unroll
  for (int x = 0; x < kRegs; ++x) {  // an empty bucket never enters the loops that set them
    e_reg[x] = -2;
    pos_reg[x] = 0;
  }

  // enters `key` into the table; false when the table cannot take it. Every distinct id takes
  // exactly one empty entry, whoever ends up there: `claimed` counts the entries this thread took.
  int claimed = 0;
  auto insert = [&](int64_t key, uint64_t mixed) -> bool {
    if (key == kSetEmpty) {
      if (atomicExch(reinterpret_cast<unsigned long long*>(&l_key[kSpecial]), 0ull) ==
          static_cast<unsigned long long>(kSetEmpty))
        ++claimed;
      return true;
    }
    unsigned long long v = static_cast<unsigned long long>(key);
    int e = home_of_mix(mixed, nb_log2);
    for (;;) {
      const unsigned long long c = static_cast<unsigned long long>(  // (atomic, not volatile: see find_heavy)
          __hip_atomic_load(&l_key[e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP));
      if (c == v) return true;
      if (c < v) {  // the id there keeps its place (the empty marker is the largest value)
        if (++e >= kTabAll - 1) return false;  // the guard entry stays empty
        continue;
      }
      if (atomicCAS(reinterpret_cast<unsigned long long*>(&l_key[e]), c, v) != c) continue;  // it changed: look again
      if (c == static_cast<unsigned long long>(kSetEmpty)) {
        ++claimed;
        return true;
      }
      v = c;  // the id that sat here moves on
      if (++e >= kTabAll - 1) return false;
    }
  };
  auto find_from = [&](int64_t key, int e) -> int {  // e = the id's home entry
    if (key == kSetEmpty) return kSpecial;
    for (;;) {
      const int64_t k = l_key[e];
      if (k == key) return e;
      if (k == kSetEmpty || ++e >= kTabAll - 1) return -1;
    }
  };
  // the table of one round (cleared by the caller): every id of the round entered (pass 1), its
  // occurrences counted (pass 2). The bucket's records are taken kRegs per thread at a time, all
  // loads of a turn in flight together; for the first turn the table entry stays in e_reg.
  // `announce`: publish the number of distinct ids for the later buckets as soon as it is known
  // (after the first pass; the ranking and the lists of this bucket are still to come)
  auto build = [&](uint32_t rounds, uint32_t round, bool announce) {
    bool ok = true;
    claimed = 0;
    for (int32_t q0 = r_lo; q0 < r_hi; q0 += kRegs * kBucketBlock) {
      int64_t k[kRegs];
#pragma unroll
      for (int x = 0; x < kRegs; ++x) {
        const int32_t q = q0 + tid + x * kBucketBlock;
        k[x] = q < r_hi ? a.bkt_id[q] : 0;
        if (q0 == r_lo) pos_reg[x] = q < r_hi ? a.bkt_pos[q] : 0;
      }
#pragma unroll
      for (int x = 0; x < kRegs; ++x) {
        int mark = -2;  // not of this round
        if (q0 + tid + x * kBucketBlock < r_hi) {
          const uint64_t mixed = mix_id(k[x]);
          if (in_round(mixed, rounds, round)) {
            mark = -3 - home_of_mix(mixed, nb_log2);  // pass 2 starts its search there
            ok = insert(k[x], mixed) && ok;
          }
        }
        if (q0 == r_lo) e_reg[x] = mark;
      }
    }
    if (!ok) s_overflow = 1;
    if (announce) {
#pragma unroll
      for (int o = kWave / 2; o > 0; o >>= 1) claimed += __shfl_xor(claimed, o, kWave);
      if ((tid & (kWave - 1)) == 0 && claimed) atomicAdd(&s_claimed, claimed);
    }
    __syncthreads();
    if (s_overflow) return;
    if (announce && tid == 0)
      __hip_atomic_store(&a.agg[b], kAggFlag | static_cast<unsigned long long>(s_claimed), __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
    for (int32_t q0 = r_lo; q0 < r_hi; q0 += kRegs * kBucketBlock) {
      const bool first_turn = q0 == r_lo;
      int64_t k[kRegs];
#pragma unroll
      for (int x = 0; x < kRegs; ++x) {
        const int32_t q = q0 + tid + x * kBucketBlock;
        k[x] = q < r_hi ? a.bkt_id[q] : 0;  // the first turn reads what it has just read: a cache hit
      }
#pragma unroll
      for (int x = 0; x < kRegs; ++x) {
        int e = -2;
        if (q0 + tid + x * kBucketBlock < r_hi) {
          if (first_turn) {
            if (e_reg[x] <= -3) e = find_from(k[x], -3 - e_reg[x]);
          } else {
            const uint64_t mixed = mix_id(k[x]);
            if (in_round(mixed, rounds, round)) e = find_from(k[x], home_of_mix(mixed, nb_log2));
          }
        }
        if (first_turn) e_reg[x] = e;
        wave_add_one(l_cnt, e, e >= 0);
      }
    }
    __syncthreads();
  };
  auto clear = [&]() {
    __syncthreads();
    for (int e = tid; e <= kTabAll; e += kBucketBlock) {
      l_key[e] = kSetEmpty;
      l_cnt[e] = 0;
    }
    if (tid == 0) s_overflow = 0;
    __syncthreads();
  };

  uint32_t rounds = 1;
  build(1, 0, true);
  while (s_overflow) {  // dry runs: double the rounds until every round fits
    if (rounds >= (1u << 16)) {
      if (tid == 0) raise_device_error(a.err, RECIS_DEVERR_PLAN_OVERFLOW);
      break;  // entries that found no room are dropped (flagged)
    }
    rounds *= 2;
    bool fits = true;
    for (uint32_t r = 0; r < rounds && fits; ++r) {
      clear();
      build(rounds, r, false);
      fits = !s_overflow;
    }
    if (fits) {
      clear();
      build(rounds, 0, false);
      break;
    }
  }

  int64_t u_base = 0;  // distinct ids of all earlier buckets
  // the rare case: learn the base first, publish the total after the last round
  if (rounds > 1) u_base = look_back(a.agg, b, n_heavy, a.spin_limit, a.err, s_wave);
  const int32_t l_base = r_lo;  // the bucket's occurrences are its list entries
  int32_t u_done = 0, l_done = 0, new_done = 0;
  const int s_lo = tid * kPer;
  // The inverse holds unique indices, so with it the base must be known before the occurrences are
  // placed. Without it the placing (bucket-local) comes first and the look-back after: by then the
  // earlier buckets have published, and nobody waits.
  const bool base_first = a.inverse != nullptr;
  constexpr int kBatch = 2;  // unique ids of a thread whose id-map probes are in flight together

  for (uint32_t round = 0; round < rounds; ++round) {
    if (round > 0) {
      clear();
      build(rounds, round, false);
    }
    // ---- rank the entries this thread owns: position in the table = order of the unique ids
    int32_t n_ent, n_occ;
    {
      int32_t cnt[kPer];
      unsigned long long mine = 0;
#pragma unroll
      for (int x = 0; x < kPer; ++x) {
        const int e = s_lo + x;
        const bool occ = e <= kTabAll && l_key[e] != kSetEmpty;
        cnt[x] = occ ? l_cnt[e] : -1;  // -1: not occupied
        if (occ) mine += (static_cast<unsigned long long>(cnt[x]) << 32) | 1ull;
      }
      unsigned long long total;
      unsigned long long run = block_scan_u64(mine, s_wave, total);
      n_ent = static_cast<int32_t>(total & 0xffffffffull);
      n_occ = static_cast<int32_t>(total >> 32);
      // (with one round the later buckets know n_ent already: build announced it)
#pragma unroll
      for (int x = 0; x < kPer; ++x) {
        if (cnt[x] < 0) continue;
        const int32_t rank = static_cast<int32_t>(run & 0xffffffffull);
        l_u[s_lo + x] = rank;
        l_ent[rank] = static_cast<uint16_t>(s_lo + x);
        l_cnt[s_lo + x] = static_cast<int32_t>(run >> 32);  // the start of its list; only its owner has read the count
        run += (static_cast<unsigned long long>(cnt[x]) << 32) | 1ull;
      }
    }
    __syncthreads();

    // ---- the unique ids are shared out by rank, a stretch of consecutive ranks per thread; the
    // probes of the id map for the first kBatch of them start now and land while the lists are made
    const int per = (n_ent + kBucketBlock - 1) / kBucketBlock;
    const int rk_lo = min(n_ent, tid * per), rk_hi = min(n_ent, rk_lo + per);
    longlong2 hint[kBatch];  // all that stays in registers meanwhile: the home slots as they were read
    auto key_of_rank = [&](int r, int* e) -> int64_t {
      *e = l_ent[r];
      return *e == kSpecial ? kSetEmpty : l_key[*e];
    };
    auto fetch = [&](int r_first) {
#pragma unroll
      for (int y = 0; y < kBatch; ++y) {
        hint[y] = make_longlong2(0, 0);
        if constexpr (PROBE) {
          if (r_first + y < rk_hi) {
            int e;
            const int64_t key = key_of_rank(r_first + y, &e);
            if (key != kEmpty && key != kTomb)
              hint[y] = *reinterpret_cast<const longlong2*>(&a.table[home_slot(key, a.mask)]);
          }
        }
      }
    };
    fetch(rk_lo);

    // ---- where this bucket's unique ids start
    auto learn_base = [&]() {
      u_base = look_back(a.agg, b, n_heavy, a.spin_limit, a.err, s_wave);
      if (tid == 0)
        __hip_atomic_store(&a.agg[b], kPrefixFlag | static_cast<unsigned long long>(u_base + n_ent), __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    };
    if (rounds == 1 && base_first) learn_base();

    // ---- per occurrence: its place in the list of its id, its unique index
    auto place = [&](int e, int32_t pos) {  // every lane of the wave calls; e < 0: nothing to place
      const int32_t at = wave_add_one(l_cnt, e, e >= 0);
      if (e < 0) return;
      const int32_t lp = l_base + l_done + at;
      if (lp < r_lo || lp >= r_hi || static_cast<uint32_t>(pos) >= static_cast<uint64_t>(a.g.n)) {
        raise_device_error(a.err, RECIS_DEVERR_PLAN_OVERFLOW);  // cannot happen; never store out of bounds
        return;
      }
      a.list[lp] = pos;
      if (a.pos_out) a.pos_out[pos] = lp;
      if (a.inverse) a.inverse[pos] = static_cast<int32_t>(u_base + u_done + l_u[e]);
    };
#pragma unroll
    for (int x = 0; x < kRegs; ++x) place(e_reg[x], pos_reg[x]);
    for (int32_t q0 = r_lo + kRegs * kBucketBlock; q0 < r_hi; q0 += kRegs * kBucketBlock) {
      int64_t k[kRegs];
      int32_t pos[kRegs];
#pragma unroll
      for (int x = 0; x < kRegs; ++x) {
        const int32_t q = q0 + tid + x * kBucketBlock;
        k[x] = q < r_hi ? a.bkt_id[q] : 0;
        pos[x] = q < r_hi ? a.bkt_pos[q] : 0;
      }
#pragma unroll
      for (int x = 0; x < kRegs; ++x) {
        int e = -1;
        if (q0 + tid + x * kBucketBlock < r_hi) {
          const uint64_t mixed = mix_id(k[x]);
          if (in_round(mixed, rounds, round)) e = find_from(k[x], home_of_mix(mixed, nb_log2));
        }
        place(e, pos[x]);
      }
    }
    __syncthreads();  // every entry's l_cnt now holds the END of its list
    if (rounds == 1 && !base_first) learn_base();

    // ---- per unique id: the id, the start of its list, hot work items, its row in the id map
    int32_t my_new = 0, my_empty = 0;
    for (int rb = rk_lo; rb < rk_hi; rb += kBatch) {
      if (rb != rk_lo) fetch(rb);
#pragma unroll
      for (int y = 0; y < kBatch; ++y) {
        const int r = rb + y;
        if (r >= rk_hi) continue;
        int e;
        const int64_t key = key_of_rank(r, &e);
        const int64_t u = u_base + u_done + r;
        if (u < 0 || u >= a.g.n) {
          raise_device_error(a.err, RECIS_DEVERR_PLAN_OVERFLOW);  // cannot happen; never store out of bounds
          continue;
        }
        const int32_t start = r == 0 ? 0 : l_cnt[l_ent[r - 1]], n_here = l_cnt[e] - start;
        a.unique_out[u] = key;
        a.row_start[u] = l_base + l_done + start;
        if (a.hot_cap > 0 && n_here > kHotLen) {
          const int n_items = (n_here + kHotChunk - 1) / kHotChunk;
          const int64_t base = static_cast<int64_t>(atomicAdd(reinterpret_cast<unsigned long long*>(&a.counts[1]),
                                                              static_cast<unsigned long long>(n_items)));
          for (int c = 0; c < n_items; ++c) {
            if (base + c < a.hot_cap) {
              a.hot_items[2 * (base + c)] = static_cast<int32_t>(u);
              a.hot_items[2 * (base + c) + 1] = c;
            }
          }
        }
        if constexpr (PROBE) {
          int64_t row = -1;  // what index_out gets; a claimed slot travels as -(slot + 2) until rows are assigned
          if (key == kEmpty || key == kTomb) {
            raise_device_error(a.err, RECIS_DEVERR_INDEX_RANGE);  // the map's reserved keys
          } else {
            int64_t value = -1, slot = -1;
            bool took_empty = false;
            switch (probe_or_claim(a.table, a.mask, key, home_slot(key, a.mask), hint[y], -2, &value, &slot, &took_empty)) {
              case kProbeFound:
                row = value;
                break;
              case kProbeClaimed:
                row = -(slot + 2);
                ++my_new;
                my_empty += took_empty ? 1 : 0;
                break;
              default:  // no slot left, or the key is being inserted by a concurrent call (not allowed)
                raise_device_error(a.err, RECIS_DEVERR_TABLE_FULL);
                break;
            }
          }
          a.index_out[u] = row;
        }
      }
    }
    // ---- new keys: listed per bucket in the order of the unique ids, for the row assignment
    int32_t n_new = 0;
    if constexpr (PROBE) {
      unsigned long long new_total;
      const unsigned long long new_before = block_scan_u64(
          (static_cast<unsigned long long>(my_empty) << 32) | static_cast<unsigned long long>(my_new), s_wave,
          new_total);
      n_new = static_cast<int32_t>(new_total & 0xffffffffull);
      if (tid == 0 && (new_total >> 32) != 0)
        atomicAdd(reinterpret_cast<unsigned long long*>(&a.state[ST_OCC]), new_total >> 32);
      if (my_new > 0) {
        int32_t at = l_base + new_done + static_cast<int32_t>(new_before & 0xffffffffull);
        for (int r = rk_lo; r < rk_hi; ++r) {
          NewRec nr;
          nr.u = u_base + u_done + r;
          if (nr.u < 0 || nr.u >= a.g.n) continue;  // flagged above
          const int64_t row = a.index_out[nr.u];    // written by this thread above
          if (row >= -1) continue;
          nr.slot = -(row + 2);
          if (at >= r_hi) continue;  // cannot happen: a bucket has no more new keys than records
          a.new_list[at++] = nr;
        }
      }
    }
    u_done += n_ent;
    l_done += n_occ;
    new_done += n_new;
  }

  __syncthreads();
  if (tid == 0) {
    if (rounds > 1)
      __hip_atomic_store(&a.agg[b], kPrefixFlag | static_cast<unsigned long long>(u_base + u_done), __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
    if constexpr (PROBE) {
      a.new_count[1 + b] = new_done;
      if (new_done) atomicAdd(&a.sync[3], new_done);  // lets the row assignment leave at once when there are none
    }
    if (b == (1 << nb_log2) - 1) {  // the last bucket knows the total
      const int64_t U = u_base + u_done;
      __hip_atomic_store(&a.counts[0], U, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      a.row_start[U] = static_cast<int32_t>(a.g.n);
    }
    // (the barrier above this block orders the raises of this workgroup's threads before the ticket)
    if (a.staged) finish_ticket(a);
  }
}

// Rows of the keys the fused find-or-insert added to the id map, in the order of the unique ids
// (IdAllocator::GenIds, csrc/embedding/id_allocator.cc:17-26): every workgroup scans the per-bucket
// counts of new keys for itself, takes a share of the buckets and gives the k-th new key of bucket
// b the rank (new keys of earlier buckets) + k. The workgroup that finishes last (all others have
// read the allocator words by then) does the allocator's bookkeeping and publishes it to the host.
__global__ void __launch_bounds__(kPartBlock)
plan_assign_new_kernel(Slot* __restrict__ table, const NewRec* __restrict__ new_list,
                       const int32_t* __restrict__ bucket_start, const int32_t* __restrict__ new_count, int nb,
                       int64_t* __restrict__ state, volatile int64_t* mirror, int64_t seq,
                       const int64_t* __restrict__ free_list, int64_t* __restrict__ index_out,
                       int32_t* __restrict__ sync) {
  // nb here = 1 + buckets: the new keys among the heavy ids, then those of every bucket
  extern __shared__ int32_t first_new[];  // [nb + 1], then kPartBlock words of scan scratch
  // a batch of known keys only (the steady state of a table that is not growing): nothing to scan
  const bool any_new = __hip_atomic_load(&sync[3], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0;  // uniform
  if (any_new) scan_counts(new_count, nb, first_new, first_new + nb + 1);
  const int64_t n_new = any_new ? first_new[nb] : 0;
  const int64_t old_cur = state[ST_CUR], old_free = state[ST_FREE];
  for (int b = blockIdx.x; b < nb && n_new > 0; b += gridDim.x) {
    const int32_t cnt = new_count[b];
    const NewRec* mine = new_list + (b == 0 ? bucket_start[0] : bucket_start[kHeavyMax + b - 1]);
    for (int k = threadIdx.x; k < cnt; k += kPartBlock) {
      const NewRec r = mine[k];
      const int64_t row = row_of_new_key(first_new[b] + k, n_new, old_cur, old_free, free_list);
      st_relaxed(&table[r.slot].val, row);
      index_out[r.u] = row;
    }
  }
  __syncthreads();
  if (threadIdx.x == 0 && atomicAdd(&sync[2], 1) == static_cast<int>(gridDim.x) - 1) {
    commit_new_keys(state, n_new);
    publish(state, mirror, seq);
  }
}

// inverse / pos from the lists, for plans that were made without them: list entry k belongs to the
// unique id u with row_start[u] <= k < row_start[u + 1] (binary search; the arrays are cache
// resident right after the plan).
__global__ void __launch_bounds__(kBlock)
plan_inverse_from_lists_kernel(const int32_t* __restrict__ row_start, const int32_t* __restrict__ list,
                               const int64_t* __restrict__ counts, int64_t n, int32_t* __restrict__ inverse,
                               int32_t* __restrict__ pos_out) {
  const int64_t k = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (k >= n) return;
  int64_t lo = 0, hi = counts[0];  // row_start[lo] <= k < row_start[hi]
  while (hi - lo > 1) {
    const int64_t mid = (lo + hi) >> 1;
    if (row_start[mid] <= k)
      lo = mid;
    else
      hi = mid;
  }
  const int32_t i = list[k];
  if (static_cast<uint32_t>(i) >= static_cast<uint64_t>(n)) return;
  if (inverse) inverse[i] = static_cast<int32_t>(lo);
  if (pos_out) pos_out[i] = static_cast<int32_t>(k);
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

}  // namespace
}  // namespace recis_hip

using namespace recis_hip;

extern "C" {

// Where the plan's scratch arrays lie in one buffer of `bytes` bytes, for n ids.
struct PlanLayout {
  PlanGeom g;
  int64_t nb;
  size_t o_hist, o_total, o_start, o_agg, o_newc, o_sync, o_heavy, o_id, o_pos, o_new, bytes;
};

static int compute_units() {  // of the current device; asked once per device
  static std::atomic<int> cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  int v = cached[dev].load(std::memory_order_relaxed);
  if (v == 0) {
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0) v = 256;
    cached[dev].store(v, std::memory_order_relaxed);
  }
  return v;
}

static PlanLayout plan_layout(int64_t n, bool with_lookup) {
  PlanLayout L;
  PlanGeom& g = L.g;
  g.n = n;
  // One workgroup per compute unit is what runs at a time (see plan_scatter_runs_kernel), so the
  // rows are as many as the device has units while that keeps a tile between kTileMin and kTile
  // ids: a batch of up to cus * kTile ids is one round of workgroups, none left over for a
  // second round on a few units.
  const int64_t cus = compute_units();
  int64_t rows = (n + kTile - 1) / kTile;
  if (rows <= cus) rows = std::max<int64_t>(1, std::min<int64_t>(cus, n / kTileMin));
  rows = std::min<int64_t>(rows, kMaxRows);
  g.tile = static_cast<int>(((n + rows - 1) / rows + kPartBlock - 1) / kPartBlock * kPartBlock);
  g.rows = static_cast<int>((n + g.tile - 1) / g.tile);
  int nb_log2 = 5;
  while ((int64_t(1) << nb_log2) < kMaxBuckets && (int64_t(1) << nb_log2) * kBucketIds < n) ++nb_log2;
  g.nb_log2 = nb_log2;
  L.nb = int64_t(1) << nb_log2;
  // hist[rows * columns] (counts, then offsets, in place) | bucket_total[columns] | bucket_start[columns + 1] |
  // agg[nb] look-back words | new_count[1 + nb] | sync[4] | heavy ids | bkt_id[n] | bkt_pos[n] |
  // new_list[n] (fused lookup only)
  size_t bytes = 0;
  auto take = [&](size_t b) {
    const size_t at = bytes;
    bytes += (b + 255) & ~size_t(255);
    return at;
  };
  const int64_t nc = kHeavyMax + L.nb;  // columns of the partition: the heavy ids, then the buckets
  L.o_hist = take(sizeof(int32_t) * g.rows * nc);
  L.o_total = take(sizeof(int32_t) * nc);
  L.o_start = take(sizeof(int32_t) * (nc + 1));
  L.o_agg = take(sizeof(unsigned long long) * L.nb);
  L.o_newc = take(sizeof(int32_t) * (L.nb + 1));
  L.o_sync = take(sizeof(int32_t) * 4);
  L.o_heavy = take(sizeof(int64_t) * kHeavyMax + sizeof(int32_t));  // heavy_ids[kHeavyMax], heavy_n
  L.o_id = take(sizeof(int64_t) * n);
  L.o_pos = take(sizeof(int32_t) * n);
  L.o_new = with_lookup ? take(sizeof(NewRec) * n) : bytes;
  L.bytes = bytes;
  return L;
}

static int plan_check_args(const int64_t* ids, int64_t n, int64_t* unique_out, int32_t* row_start_out,
                           int32_t* list_out, int32_t* hot_items_out, int64_t hot_cap, int64_t* counts_out_dev) {
  RECIS_REQUIRE(n >= 0 && n < (int64_t(1) << 30), "n out of range: %lld", (long long)n);
  RECIS_REQUIRE(counts_out_dev && row_start_out, "counts_out_dev / row_start_out must not be NULL");
  RECIS_REQUIRE(hot_cap == 0 || (hot_items_out && hot_cap >= n / kHotLen + n / kHotChunk + 2),
                "hot_items_out must hold at least n/%d + n/%d + 2 items", kHotLen, kHotChunk);
  RECIS_REQUIRE(n == 0 || (ids && unique_out && list_out), "NULL argument");
  return RECIS_OK;
}

// Polls of one look-back word before a workgroup gives up (a word is due within microseconds; the
// limit only bounds a wait that can never end, e.g. after a failed launch of an earlier kernel).
static std::atomic<uint32_t> g_spin_limit{RECIS_PLAN_SPIN_LIMIT_DEFAULT};

// The plan's launches for n > 0 over the scratch buffer `base` (L.bytes bytes). `staged`: pinned host
// words that receive the unique count (and the soft-error bits) as soon as they are final, or NULL.
// With a map, every unique id is looked up (find or insert) from inside the bucket kernel and
// index_out receives its row.
static int plan_launch(const PlanLayout& L, char* base, const int64_t* ids, const IdJobs* jobs_in, int64_t* unique_out,
                       int32_t* inverse_out, int32_t* row_start_out, int32_t* list_out, int32_t* pos_out,
                       int32_t* hot_items_out, int64_t hot_cap, int64_t* counts_out_dev, int64_t* staged,
                       hipEvent_t staged_event, int* err, recis_idmap* map, int64_t map_seq, int64_t* index_out,
                       hipStream_t stream) {
  const PlanGeom& g = L.g;
  const int64_t nb = L.nb;
  int32_t* hist = reinterpret_cast<int32_t*>(base + L.o_hist);
  int32_t* bucket_total = reinterpret_cast<int32_t*>(base + L.o_total);
  int32_t* bucket_start = reinterpret_cast<int32_t*>(base + L.o_start);
  unsigned long long* agg = reinterpret_cast<unsigned long long*>(base + L.o_agg);
  int32_t* sync = reinterpret_cast<int32_t*>(base + L.o_sync);
  int64_t* bkt_id = reinterpret_cast<int64_t*>(base + L.o_id);
  int32_t* bkt_pos = reinterpret_cast<int32_t*>(base + L.o_pos);
  const int64_t nc = kHeavyMax + nb;
  const size_t lds = sizeof(int32_t) * static_cast<size_t>(nc);
  int64_t* heavy_ids = reinterpret_cast<int64_t*>(base + L.o_heavy);
  int32_t* heavy_n = reinterpret_cast<int32_t*>(heavy_ids + kHeavyMax);
  HeavyArgs hv;
  hv.ids = heavy_ids;
  hv.n = heavy_n;
  hv.list = list_out;
  hv.inverse = inverse_out;
  hv.pos_out = pos_out;
  const bool by_jobs = jobs_in != nullptr;
  IdJobs jobs;  // the kernels take it by value
  if (by_jobs)
    jobs = *jobs_in;
  else
    jobs.n_jobs = 0;
  {
    const size_t hist_lds = std::max(lds, sizeof(HeavyScratch));
    RECIS_TIME_KERNEL("plan_hist_kernel", stream)
    if (by_jobs)
      plan_hist_kernel<true><<<dim3(g.rows), dim3(kPartBlock), hist_lds, stream>>>(ids, jobs, g, heavy_ids, heavy_n, hist,
                                                                                  counts_out_dev, sync);
    else
      plan_hist_kernel<false><<<dim3(g.rows), dim3(kPartBlock), hist_lds, stream>>>(ids, jobs, g, heavy_ids, heavy_n,
                                                                                   hist, counts_out_dev, sync);
    RECIS_LAUNCH_CHECK();
  }
  {
    RECIS_TIME_KERNEL("plan_colscan_kernel", stream)
    plan_colscan_kernel<<<dim3(nc / kColBuckets), dim3(1024), 0, stream>>>(hist, g, bucket_total);
    RECIS_LAUNCH_CHECK();
  }
  {
    const dim3 grid(g.rows), block(kPartBlock);
    RECIS_TIME_KERNEL("plan_scatter_kernel", stream)
    if (g.tile <= kTile && g.tile >= 4 * nb) {  // a tile sends four ids or more to a bucket: worth ordering them
      const size_t runs_lds = scatter_runs_lds(nc);
      static std::atomic<bool> lds_allowed_on[64];  // more than the 64 KB a kernel may take unasked; per device
      int dev = 0;
      RECIS_CHECK_HIP(hipGetDevice(&dev));
      std::atomic<bool>& lds_allowed = lds_allowed_on[dev & 63];
      if (!lds_allowed.load(std::memory_order_acquire)) {
        RECIS_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&plan_scatter_runs_kernel<true>),
                                            hipFuncAttributeMaxDynamicSharedMemorySize,
                                            static_cast<int>(scatter_runs_lds(kHeavyMax + kTile / 4))));
        RECIS_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&plan_scatter_runs_kernel<false>),
                                            hipFuncAttributeMaxDynamicSharedMemorySize,
                                            static_cast<int>(scatter_runs_lds(kHeavyMax + kTile / 4))));
        lds_allowed.store(true, std::memory_order_release);
      }
      if (by_jobs)
        plan_scatter_runs_kernel<true><<<grid, block, runs_lds, stream>>>(ids, jobs, g, hv, hist, bucket_total,
                                                                         bucket_start, agg, bkt_id, bkt_pos);
      else
        plan_scatter_runs_kernel<false><<<grid, block, runs_lds, stream>>>(ids, jobs, g, hv, hist, bucket_total,
                                                                          bucket_start, agg, bkt_id, bkt_pos);
    } else {
      const size_t plain_lds = lds + sizeof(int32_t) * (kPartBlock + 1);
      if (by_jobs)
        plan_scatter_kernel<true><<<grid, block, plain_lds, stream>>>(ids, jobs, g, hv, hist, bucket_total, bucket_start,
                                                                     agg, bkt_id, bkt_pos);
      else
        plan_scatter_kernel<false><<<grid, block, plain_lds, stream>>>(ids, jobs, g, hv, hist, bucket_total, bucket_start,
                                                                      agg, bkt_id, bkt_pos);
    }
    RECIS_LAUNCH_CHECK();
  }
  BucketArgs a;
  a.bkt_id = bkt_id;
  a.bkt_pos = bkt_pos;
  a.bucket_start = bucket_start;
  a.heavy_ids = heavy_ids;
  a.heavy_n = heavy_n;
  a.g = g;
  a.agg = agg;
  a.new_count = reinterpret_cast<int32_t*>(base + L.o_newc);
  a.sync = sync;
  a.unique_out = unique_out;
  a.inverse = inverse_out;
  a.row_start = row_start_out;
  a.list = list_out;
  a.pos_out = pos_out;
  a.counts = counts_out_dev;
  a.hot_items = hot_items_out;
  a.hot_cap = hot_cap;
  a.staged = staged;
  a.err = err;
  a.spin_limit = g_spin_limit.load(std::memory_order_relaxed);
  a.table = nullptr;
  a.mask = 0;
  a.index_out = index_out;
  a.state = nullptr;
  a.mirror = nullptr;
  a.seq = map_seq;
  a.new_list = reinterpret_cast<NewRec*>(base + L.o_new);
  if (map) {
    a.table = map->table;
    a.mask = static_cast<uint64_t>(map->capacity - 1);
    a.state = map->state;
    a.mirror = map->mirror;
    {
      RECIS_TIME_KERNEL("plan_bucket_kernel", stream)
      plan_bucket_kernel<true><<<dim3(nb + 1), dim3(kBucketBlock), 0, stream>>>(a);
      RECIS_LAUNCH_CHECK();
    }
    plan_assign_new_kernel<<<dim3(std::max<int64_t>(nb / 4, 1)), dim3(kPartBlock),
                             sizeof(int32_t) * (nb + 2 + kPartBlock + 1), stream>>>(
        map->table, a.new_list, bucket_start, a.new_count, static_cast<int>(nb + 1), map->state, map->mirror, map_seq,
        map->free_list, index_out, sync);
    RECIS_LAUNCH_CHECK();
  } else {
    RECIS_TIME_KERNEL("plan_bucket_kernel", stream)
    plan_bucket_kernel<false><<<dim3(nb + 1), dim3(kBucketBlock), 0, stream>>>(a);
    RECIS_LAUNCH_CHECK();
  }
  if (staged) RECIS_CHECK_HIP(hipEventRecord(staged_event, stream));
  return RECIS_OK;
}

static int plan_entry(recis_idmap* map, const int64_t* ids, int64_t n, int64_t* unique_out, int32_t* inverse_out,
                      int32_t* row_start_out, int32_t* list_out, int32_t* pos_out, int32_t* hot_items_out,
                      int64_t hot_cap, int64_t* counts_out_dev, int64_t* index_out, int64_t* unique_count_host,
                      int flags, hipStream_t stream, const IdJobs* jobs = nullptr) {
  // with jobs, `ids` is unused (the kernels read the jobs' arrays); any non-NULL value passes the checks
  if (int rc = plan_check_args(jobs ? reinterpret_cast<const int64_t*>(jobs) : ids, n, unique_out, row_start_out,
                               list_out, hot_items_out, hot_cap, counts_out_dev))
    return rc;
  RECIS_REQUIRE(map == nullptr || n == 0 || index_out != nullptr, "index_out must not be NULL");
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
  int64_t seq = 0;
  if (map) {
    if (int rc = idmap_begin_call(map, n, stream, &seq)) return rc;
  }
  const PlanLayout L = plan_layout(n, map != nullptr);
  void* ws = nullptr;
  if (int rc = get_workspace(stream, L.bytes, &ws)) return rc;
  if (int rc = plan_launch(L, static_cast<char*>(ws), ids, jobs, unique_out, inverse_out, row_start_out, list_out, pos_out,
                           hot_items_out, hot_cap, counts_out_dev, staged, staged_event, err, map, seq, index_out,
                           stream))
    return rc;
  if (map) idmap_end_call(map, seq, n);
  if (unique_count_host) {
    RECIS_CHECK_HIP(hipEventSynchronize(staged_event));
    *unique_count_host = staged[0];
  }
  return RECIS_OK;
}

int recis_unique_plan(const int64_t* ids, int64_t n, int64_t* unique_out, int32_t* inverse_out,
                      int32_t* row_start_out, int32_t* list_out, int32_t* pos_out, int32_t* hot_items_out,
                      int64_t hot_cap, int64_t* counts_out_dev, int64_t* unique_count_host, int flags, void* stream_) {
  return plan_entry(nullptr, ids, n, unique_out, inverse_out, row_start_out, list_out, pos_out, hot_items_out, hot_cap,
                    counts_out_dev, nullptr, unique_count_host, flags, static_cast<hipStream_t>(stream_));
}

int recis_unique_plan_lookup(recis_idmap* map, const int64_t* ids, int64_t n, int64_t* unique_out,
                             int32_t* inverse_out, int32_t* row_start_out, int32_t* list_out, int32_t* pos_out,
                             int32_t* hot_items_out, int64_t hot_cap, int64_t* counts_out_dev, int64_t* index_out,
                             int64_t* unique_count_host, int flags, void* stream_) {
  RECIS_REQUIRE(map != nullptr, "id map is NULL");
  return plan_entry(map, ids, n, unique_out, inverse_out, row_start_out, list_out, pos_out, hot_items_out, hot_cap,
                    counts_out_dev, index_out, unique_count_host, flags, static_cast<hipStream_t>(stream_));
}

int recis_unique_plan_jobs(recis_idmap* map, const int64_t* const* ids_ptrs, const int64_t* sizes,
                           const int64_t* table_ids, int64_t n_jobs, int64_t* unique_out, int32_t* inverse_out,
                           int32_t* row_start_out, int32_t* list_out, int32_t* pos_out, int32_t* hot_items_out,
                           int64_t hot_cap, int64_t* counts_out_dev, int64_t* index_out, int64_t* unique_count_host,
                           int flags, void* stream_) {
  RECIS_REQUIRE(n_jobs >= 1 && n_jobs <= kPlanJobs, "1 to %d arrays of ids (got %lld)", kPlanJobs, (long long)n_jobs);
  RECIS_REQUIRE(ids_ptrs && sizes, "NULL argument");
  IdJobs jobs;
  jobs.n_jobs = static_cast<int>(n_jobs);
  jobs.mask = table_ids ? (int64_t(1) << 52) - 1 : ~int64_t(0);
  int64_t n = 0;
  for (int k = 0; k < kPlanJobs; ++k) {
    jobs.in[k] = nullptr;
    jobs.tag[k] = 0;
    jobs.first[k] = n;
    if (k >= n_jobs) continue;
    RECIS_REQUIRE(sizes[k] >= 0 && (sizes[k] == 0 || ids_ptrs[k]), "bad array %d", k);
    if (table_ids) {
      RECIS_REQUIRE(table_ids[k] >= 0 && table_ids[k] < 4096, "table id %lld out of 12 bits", (long long)table_ids[k]);
      jobs.tag[k] = static_cast<int64_t>(static_cast<uint64_t>(table_ids[k]) << 52);
    }
    jobs.in[k] = ids_ptrs[k];
    n += sizes[k];
  }
  jobs.first[kPlanJobs] = n;
  for (int k = static_cast<int>(n_jobs); k <= kPlanJobs; ++k) jobs.first[k] = n;
  return plan_entry(map, nullptr, n, unique_out, inverse_out, row_start_out, list_out, pos_out, hot_items_out, hot_cap,
                    counts_out_dev, index_out, unique_count_host, flags, static_cast<hipStream_t>(stream_), &jobs);
}

int recis_plan_inverse_from_lists(const int32_t* row_start, const int32_t* list, const int64_t* counts_dev, int64_t n,
                                  int32_t* inverse_out, int32_t* pos_out, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(n >= 0, "negative size");
  if (n == 0 || (!inverse_out && !pos_out)) return RECIS_OK;
  RECIS_REQUIRE(row_start && list && counts_dev, "NULL argument");
  plan_inverse_from_lists_kernel<<<dim3((n + kBlock - 1) / kBlock), dim3(kBlock), 0, stream>>>(
      row_start, list, counts_dev, n, inverse_out, pos_out);
  RECIS_LAUNCH_CHECK();
  return RECIS_OK;
}

int recis_plan_set_spin_limit(int64_t polls) {
  RECIS_REQUIRE(polls >= 1 && polls <= (int64_t(1) << 31) - 1, "polls out of range");
  g_spin_limit.store(static_cast<uint32_t>(polls), std::memory_order_relaxed);
  return RECIS_OK;
}

int recis_plan_get_spin_limit(int64_t* polls) {
  RECIS_REQUIRE(polls != nullptr, "polls must not be NULL");
  *polls = g_spin_limit.load(std::memory_order_relaxed);
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
  if (int rc = plan_check_args(ids, n, unique_out, row_start_out, list_out, hot_items_out, hot_cap, counts_out_dev))
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
  const PlanLayout L = plan_layout(n, false);
  if (L.bytes > kStaticScratchBytes)
    return fail(RECIS_ERR_CAPACITY,
                "recis_unique_plan_noalloc: %lld ids need %zu bytes of scratch, the built-in buffer holds %zu "
                "(at most %lld ids per call; use recis_unique_plan for more)",
                (long long)n, L.bytes, kStaticScratchBytes, (long long)RECIS_PLAN_NOALLOC_MAX_IDS);
  // What must start at zero (the two counters in `sync`, the look-back words) is cleared by the
  // plan's own first two kernels; every other scratch array is fully written by the kernel that
  // produces it before any kernel reads it: nothing of the previous call's contents is relied on.
  return plan_launch(L, base, ids, nullptr, unique_out, inverse_out, row_start_out, list_out, pos_out, hot_items_out, hot_cap,
                     counts_out_dev, nullptr, nullptr, err, nullptr, 0, nullptr, stream);
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

}  // extern "C"
