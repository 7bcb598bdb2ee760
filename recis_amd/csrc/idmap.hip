// IDMap for gfx950: 64-bit key -> row index, with the row-index allocator folded in.
//
// Stands in for GpuIdMap + cuco::dynamic_map + IdAllocator
// (csrc/embedding/gpu_id_map.cu:19-121, csrc/embedding/id_allocator.cc:17-64,
// csrc/ops/hashtable_ops_kernel.cu:32-173). Design:
//   * ONE flat open-addressing table of 16-byte slots {key, row}, power-of-two
//     capacity, linear probing, load factor <= 1/2; claims are a 64-bit
//     atomicCAS on the key word (empty = -1, tombstone = -2, as in the reference)
//   * allocator state (high-water mark, free count) and the free list live in
//     device memory, so a find-or-insert needs no host round trip: four
//     back-to-back launches (probe+claim, scan, assign, resolve) replace the
//     reference's find / cumsum / .item() / GenIds+sync / compact / scatter /
//     insert+sync-per-submap sequence
//   * row indices are assigned exactly as IdAllocator::GenIds does: missing keys
//     are ranked in input order; rank i of n takes free_list[free - n + i] when
//     that index is >= 0, else the fresh index cur - (free - n + i + 1). A missing
//     key that occurs more than once in a call is ranked at whichever occurrence
//     wins the claim, so only duplicate-free calls have a reproducible assignment
//   * erase leaves tombstones, later inserts reuse them; the table is rebuilt
//     (sized up) only when live + tombstones would pass the load limit
#include <hip/hip_runtime.h>

#include <algorithm>
#include <deque>
#include <utility>

#include "common.cuh"
#include "idmap_internal.cuh"

namespace recis_hip {
namespace {

// Number of ids of a call whose count is still on the device: the first *n_dev of n_max.
__device__ __forceinline__ int64_t counted(int64_t n_max, const int64_t* n_dev) {
  if (n_dev == nullptr) return n_max;
  const int64_t n = *n_dev;
  return n < 0 ? 0 : (n < n_max ? n : n_max);
}

__global__ void publish_kernel(const int64_t* state, volatile int64_t* mirror, int64_t seq) {
  publish(state, mirror, seq);
}

__global__ void __launch_bounds__(kBlock) fill_slots_kernel(Slot* t, int64_t n) {
  int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
  for (; i < n; i += stride) {
    t[i].key = kEmpty;
    t[i].val = kValUnset;
  }
}

__global__ void zero_words_kernel(int64_t* p, int n) {
  if (threadIdx.x < n) p[threadIdx.x] = 0;
}

// Block-wide sum of a 0/1 flag; returns the total in every thread and the
// exclusive rank of this thread among the set flags.
__device__ __forceinline__ void block_rank(bool flag, int& rank, int& total) {
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

// Pass 1 of find-or-insert. slotpos[i]: -1 = resolved (out[i] written),
// >= 0 = this thread claimed that slot (a new key), <= -2 = the key is being
// inserted by another thread of this call, slot = -(slotpos + 2).
__global__ void __launch_bounds__(kBlock)
find_or_claim_kernel(Slot* __restrict__ table, uint64_t mask, const int64_t* __restrict__ ids,
                     int64_t n, const int64_t* __restrict__ n_dev, int64_t* __restrict__ out,
                     int64_t* __restrict__ slotpos, int32_t* __restrict__ block_counts,
                     int64_t* __restrict__ state, int64_t seq, int* err) {
  n = counted(n, n_dev);
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  bool is_new = false;
  bool took_empty = false;
  if (i < n) {
    const int64_t key = ids[i];
    int64_t sp = -1;
    if (key == kEmpty || key == kTomb) {
      raise_device_error(err, RECIS_DEVERR_INDEX_RANGE);
      out[i] = -1;
    } else {
      const uint64_t h = home_slot(key, mask);
      const longlong2 hint = *reinterpret_cast<const longlong2*>(&table[h]);
      int64_t value = -1, slot = -1;
      switch (probe_or_claim(table, mask, key, h, hint, -(i + 2) /* pending, owner = occurrence i */, &value, &slot,
                             &took_empty)) {
        case kProbeFound:
          out[i] = value;
          break;
        case kProbeClaimed:
          sp = slot;
          is_new = true;
          break;
        case kProbePending:
          sp = -(slot + 2);
          st_relaxed(&state[ST_DUPS], seq);  // "this call has duplicates": every writer stores the same word
          break;
        case kProbeFull:
          raise_device_error(err, RECIS_DEVERR_TABLE_FULL);
          out[i] = -1;
          break;
      }
    }
    slotpos[i] = sp;
  }
  int rank, total;
  block_rank(is_new, rank, total);
  int rank_e, total_e;
  block_rank(took_empty, rank_e, total_e);
  if (threadIdx.x == 0) {
    block_counts[blockIdx.x] = total;
    if (total_e)
      atomicAdd(reinterpret_cast<unsigned long long*>(&state[ST_OCC]),
                static_cast<unsigned long long>(total_e));
  }
}

// Pass 2: exclusive scan of the per-block counts (single workgroup) and the
// allocator bookkeeping of IdAllocator::GenIds (id_allocator.cc:17-26).
__global__ void __launch_bounds__(1024)
scan_commit_kernel(int32_t* __restrict__ block_counts, int64_t nb, int64_t n, const int64_t* __restrict__ n_dev,
                   int64_t* __restrict__ state, volatile int64_t* mirror, int64_t seq) {
  nb = min(nb, (counted(n, n_dev) + kBlock - 1) / kBlock);  // later blocks hold nothing (and zero counts)
  __shared__ int64_t partial[1024];
  const int t = threadIdx.x;
  const int64_t per = (nb + 1023) / 1024;
  const int64_t lo = std::min<int64_t>(t * per, nb), hi = std::min<int64_t>(lo + per, nb);
  int64_t sum = 0;
  for (int64_t b = lo; b < hi; ++b) sum += block_counts[b];
  partial[t] = sum;
  __syncthreads();
  // Hillis-Steele inclusive scan over the 1024 partials
  for (int off = 1; off < 1024; off <<= 1) {
    int64_t add = t >= off ? partial[t - off] : 0;
    __syncthreads();
    partial[t] += add;
    __syncthreads();
  }
  int64_t run = t ? partial[t - 1] : 0;
  for (int64_t b = lo; b < hi; ++b) {
    int32_t c = block_counts[b];
    block_counts[b] = static_cast<int32_t>(run);  // per-call counts fit 31 bits
    run += c;
  }
  if (t == 1023) {
    commit_new_keys(state, partial[1023]);
    publish(state, mirror, seq);
  }
}

// Pass 3: give every claimed slot its row index (IdGeneratorFunctor,
// hashtable_ops.cc:15-27) in input order.
__global__ void __launch_bounds__(kBlock)
assign_rows_kernel(Slot* __restrict__ table, const int64_t* __restrict__ slotpos, int64_t n,
                   const int64_t* __restrict__ n_dev, const int32_t* __restrict__ block_prefix,
                   const int64_t* __restrict__ state, const int64_t* __restrict__ free_list,
                   int64_t* __restrict__ out) {
  n = counted(n, n_dev);
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  const int64_t sp = i < n ? slotpos[i] : -1;
  const bool is_new = sp >= 0;
  int rank, total;
  block_rank(is_new, rank, total);
  if (!is_new) return;
  const int64_t row = row_of_new_key(block_prefix[blockIdx.x] + rank, state[ST_NNEW], state[ST_OLD_CUR],
                                     state[ST_OLD_FREE], free_list);
  st_relaxed(&table[sp].val, row);
  out[i] = row;
}

// Pass 4: occurrences whose key was claimed by another occurrence of the same call.
__global__ void __launch_bounds__(kBlock)
resolve_dups_kernel(const Slot* __restrict__ table, const int64_t* __restrict__ slotpos, int64_t n,
                    const int64_t* __restrict__ n_dev, const int64_t* __restrict__ state, int64_t seq,
                    int64_t* __restrict__ out) {
  if (state[ST_DUPS] != seq) return;  // the calls of a map are numbered 1, 2, ...: no reset between them
  n = counted(n, n_dev);
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (i >= n) return;
  const int64_t sp = slotpos[i];
  if (sp <= -2) out[i] = table[-(sp + 2)].val;
}

__global__ void __launch_bounds__(kBlock)
find_kernel(const Slot* __restrict__ table, uint64_t mask, const int64_t* __restrict__ ids,
            int64_t n, int64_t* __restrict__ out) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (i >= n) return;
  const int64_t key = ids[i];
  int64_t res = -1;
  if (key != kEmpty && key != kTomb) {
    uint64_t p = home_slot(key, mask);
    for (uint64_t probes = 0; probes <= mask; ++probes) {
      const int64_t k = table[p].key;
      if (k == key) {
        res = table[p].val;
        break;
      }
      if (k == kEmpty) break;
      p = (p + 1) & mask;
    }
  }
  out[i] = res;
}

// DeleteIds (gpu_id_map.cu:84-96): tombstone the keys, append `index` to the
// free list in the order given (IdFreeFunctor, hashtable_ops.cc:39-58).
__global__ void __launch_bounds__(kBlock)
erase_kernel(Slot* __restrict__ table, uint64_t mask, const int64_t* __restrict__ ids,
             const int64_t* __restrict__ index, int64_t n, int64_t* __restrict__ free_list,
             int64_t* __restrict__ state) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  bool found = false;
  if (i < n) {
    const int64_t key = ids[i];
    if (key != kEmpty && key != kTomb) {
      uint64_t p = home_slot(key, mask);
      for (uint64_t probes = 0; probes <= mask; ++probes) {
        const int64_t k = ld_relaxed(&table[p].key);
        if (k == key) {
          // a key listed twice is erased once: only the CAS winner counts it
          const int64_t old = static_cast<int64_t>(atomicCAS(
              reinterpret_cast<unsigned long long*>(&table[p].key),
              static_cast<unsigned long long>(key), static_cast<unsigned long long>(kTomb)));
          if (old == key) {
            st_relaxed(&table[p].val, kValUnset);
            found = true;
          }
          break;
        }
        if (k == kEmpty) break;
        p = (p + 1) & mask;
      }
    }
    free_list[state[ST_FREE] + i] = index[i];
  }
  int rank, total;
  block_rank(found, rank, total);
  if (threadIdx.x == 0 && total)
    atomicAdd(reinterpret_cast<unsigned long long*>(&state[ST_TMP]),
              static_cast<unsigned long long>(total));
}

// Eviction sweep in one pass over the table: every live slot reads the stamp of its row and,
// when the stamp is older than the threshold, leaves the table (tombstone), hands its row to the
// free list and reports (key, row) so that the caller can re-initialise the row.
// The places in the output come from ONE counter, and atomics on one word are served one after the
// other (some 12 - 25 ns each on this part): with an atomic per 256 slots a sweep over a table of
// 2^29 slots spent 25 ms on two million of them and a tenth of that on the table. So a workgroup
// takes kEvictPer * 256 slots per round and one atomic per round: a thread first only notes which
// of its slots leave (a bit each), the counts are scanned over the workgroup, and the slots that
// leave are read again (the lines were fetched a moment ago) when their places are known.
constexpr int kEvictPer = 32;
__global__ void __launch_bounds__(kBlock)
evict_older_kernel(Slot* __restrict__ table, int64_t capacity, const void* const* __restrict__ stamp_blocks,
                   int64_t n_blocks, int64_t block_rows, int stamp64, int64_t threshold,
                   int64_t* __restrict__ ids_out, int64_t* __restrict__ index_out, int64_t max_out,
                   int64_t* __restrict__ free_list, int64_t* __restrict__ state, int* err) {
  __shared__ int wave_counts[kBlock / kWave];
  __shared__ int64_t s_base;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int64_t per_round = static_cast<int64_t>(kBlock) * kEvictPer;
  const int64_t free_at = state[ST_FREE];  // advanced by the commit kernel, after this one
  for (int64_t r0 = static_cast<int64_t>(blockIdx.x) * per_round; r0 < capacity;
       r0 += static_cast<int64_t>(gridDim.x) * per_round) {  // uniform in the workgroup (barriers inside)
    uint32_t leaves = 0;
    for (int x0 = 0; x0 < kEvictPer; x0 += 8) {  // eight slots in flight, then their stamps
      longlong2 kv[8];
#pragma unroll
      for (int x = 0; x < 8; ++x) {
        const int64_t i = r0 + static_cast<int64_t>(x0 + x) * kBlock + threadIdx.x;
        kv[x] = i < capacity ? *reinterpret_cast<const longlong2*>(&table[i]) : make_longlong2(kEmpty, 0);
      }
#pragma unroll
      for (int x = 0; x < 8; ++x) {
        const int64_t k = kv[x].x, v = kv[x].y;
        if (k != kEmpty && k != kTomb && v >= 0) {
          const int64_t b = v / block_rows, r = v - b * block_rows;
          if (b < n_blocks) {
            const int64_t stamp = stamp64 ? static_cast<const int64_t*>(stamp_blocks[b])[r]
                                          : static_cast<int64_t>(static_cast<const int32_t*>(stamp_blocks[b])[r]);
            if (stamp < threshold) leaves |= 1u << (x0 + x);
          } else {
            raise_device_error(err, RECIS_DEVERR_INDEX_RANGE);
          }
        }
      }
    }
    // exclusive scan of the threads' counts over the workgroup
    const int mine = __popc(leaves);
    int incl = mine;
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
      const int y = __shfl_up(incl, o, kWave);
      if (lane >= o) incl += y;
    }
    if (lane == kWave - 1) wave_counts[wave] = incl;
    __syncthreads();
    int before = incl - mine, total = 0;
#pragma unroll
    for (int w = 0; w < kBlock / kWave; ++w) {
      if (w < wave) before += wave_counts[w];
      total += wave_counts[w];
    }
    if (threadIdx.x == 0 && total)
      s_base = static_cast<int64_t>(atomicAdd(reinterpret_cast<unsigned long long*>(&state[ST_TMP]),
                                              static_cast<unsigned long long>(total)));
    __syncthreads();
    if (total) {
      int64_t pos = s_base + before;
      while (leaves) {
        const int x = __ffs(leaves) - 1;
        leaves &= leaves - 1;
        const int64_t i = r0 + static_cast<int64_t>(x) * kBlock + threadIdx.x;
        if (pos < max_out) {  // beyond the caller's buffers the key stays (counted, reported by the host)
          const longlong2 kv = *reinterpret_cast<const longlong2*>(&table[i]);
          ids_out[pos] = kv.x;
          index_out[pos] = kv.y;
          free_list[free_at + pos] = kv.y;
          table[i].key = kTomb;
          table[i].val = kValUnset;
        }
        ++pos;
      }
    }
    __syncthreads();  // wave_counts and s_base are reused by the next round
  }
}

__global__ void evict_commit_kernel(int64_t* state, int64_t max_out) {
  const int64_t n = state[ST_TMP] < max_out ? state[ST_TMP] : max_out;
  state[ST_FREE] += n;
  state[ST_LIVE] -= n;
}

__global__ void erase_commit_kernel(int64_t* state, int64_t n) {
  state[ST_FREE] += n;
  state[ST_LIVE] -= state[ST_TMP];
  state[ST_TMP] = 0;
}

// retrieve_all: every live (key, row) pair, in no particular order.
__global__ void __launch_bounds__(kBlock)
snapshot_kernel(const Slot* __restrict__ table, int64_t capacity, int64_t* __restrict__ ids_out,
                int64_t* __restrict__ index_out, int64_t max_out, int64_t* __restrict__ state) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  bool live = false;
  int64_t k = 0, v = 0;
  if (i < capacity) {
    k = table[i].key;
    v = table[i].val;
    live = k != kEmpty && k != kTomb && v >= 0;
  }
  int rank, total;
  block_rank(live, rank, total);
  __shared__ int64_t base;
  if (threadIdx.x == 0)
    base = total ? static_cast<int64_t>(atomicAdd(reinterpret_cast<unsigned long long*>(&state[ST_TMP]),
                                                  static_cast<unsigned long long>(total)))
                 : 0;
  __syncthreads();
  if (live) {
    const int64_t pos = base + rank;
    if (pos < max_out) {
      ids_out[pos] = k;
      index_out[pos] = v;
    }
  }
}

// Re-insert all live entries of an old table into a new, empty one.
__global__ void __launch_bounds__(kBlock)
rehash_kernel(const Slot* __restrict__ old_table, int64_t old_capacity, Slot* __restrict__ table,
              uint64_t mask) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (i >= old_capacity) return;
  const int64_t key = old_table[i].key;
  const int64_t val = old_table[i].val;
  if (key == kEmpty || key == kTomb || val < 0) return;
  uint64_t p = home_slot(key, mask);
  for (uint64_t probes = 0; probes <= mask; ++probes) {
    const int64_t old = static_cast<int64_t>(atomicCAS(
        reinterpret_cast<unsigned long long*>(&table[p].key),
        static_cast<unsigned long long>(kEmpty), static_cast<unsigned long long>(key)));
    if (old == kEmpty) {
      table[p].val = val;
      return;
    }
    p = (p + 1) & mask;
  }
}

// ---- standalone allocator ops (csrc/ops/hashtable_ops_kernel.cu:32-173)
__global__ void __launch_bounds__(kBlock)
generate_ids_kernel(int64_t n, const int64_t* const* __restrict__ free_blocks, int64_t free_count,
                    int64_t cur_count, int64_t free_block_size, int64_t* __restrict__ out) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (i >= n) return;
  const int64_t free_index = free_count - n + i;
  out[i] = free_index >= 0 ? free_blocks[free_index / free_block_size][free_index % free_block_size]
                           : cur_count - (free_index + 1);
}

__global__ void __launch_bounds__(kBlock)
free_ids_kernel(const int64_t* __restrict__ ids, int64_t n, int64_t* const* __restrict__ free_blocks,
                int64_t free_count, int64_t free_block_size) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (i >= n) return;
  const int64_t free_index = free_count + i;
  free_blocks[free_index / free_block_size][free_index % free_block_size] = ids[i];
}

__global__ void __launch_bounds__(kBlock)
mask_key_index_kernel(const int64_t* __restrict__ keys, const uint8_t* __restrict__ mask,
                      const int64_t* __restrict__ cumsum, int64_t n, int64_t out_size,
                      int64_t* __restrict__ out_keys, int64_t* __restrict__ out_index, int* err) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (i >= n || !mask[i]) return;
  const int64_t pos = cumsum[i] - 1;
  if (static_cast<uint64_t>(pos) >= static_cast<uint64_t>(out_size)) {
    raise_device_error(err, RECIS_DEVERR_INDEX_RANGE);
    return;
  }
  out_keys[pos] = keys[i];
  out_index[pos] = i;
}

__global__ void __launch_bounds__(kBlock)
scatter_ids_kernel(int64_t* __restrict__ out_ids, int64_t out_size, const int64_t* __restrict__ in_ids,
                   const int64_t* __restrict__ mask_index, int64_t n, int* err) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (i >= n) return;
  const int64_t pos = mask_index[i];
  if (static_cast<uint64_t>(pos) >= static_cast<uint64_t>(out_size)) {
    raise_device_error(err, RECIS_DEVERR_INDEX_RANGE);
    return;
  }
  out_ids[pos] = in_ids[i];
}

inline int64_t blocks_for(int64_t n) { return (n + kBlock - 1) / kBlock; }

int64_t capacity_for(int64_t keys) {
  int64_t cap = 1024;
  while (cap < keys * 2) cap <<= 1;
  return cap;
}

}  // namespace
}  // namespace recis_hip

using namespace recis_hip;

namespace {

int alloc_table(recis_idmap* m, int64_t capacity, hipStream_t stream, Slot** out) {
  Slot* t = nullptr;
  RECIS_CHECK_HIP(hipMalloc(reinterpret_cast<void**>(&t), sizeof(Slot) * static_cast<size_t>(capacity)));
  int64_t grid = std::min<int64_t>(blocks_for(capacity), 256 * 64);
  fill_slots_kernel<<<dim3(grid), dim3(kBlock), 0, stream>>>(t, capacity);
  RECIS_LAUNCH_CHECK();
  *out = t;
  (void)m;
  return RECIS_OK;
}

void mirror_set(recis_idmap* m, const int64_t* words);

int sync_stats(recis_idmap* m, hipStream_t stream, int64_t* words) {
  RECIS_CHECK_HIP(hipMemcpyAsync(words, m->state, sizeof(int64_t) * ST_WORDS, hipMemcpyDeviceToHost, stream));
  RECIS_CHECK_HIP(hipStreamSynchronize(stream));
  m->occ_ub = words[ST_OCC];
  m->free_ub = words[ST_FREE];
  mirror_set(m, words);
  return RECIS_OK;
}

// Upper bounds of occupied slots and of the allocator's high-water mark from the mirror, without
// waiting: what the last landed publication says plus every id of the calls issued after it.
void mirror_bounds(recis_idmap* m, int64_t* occ_ub, int64_t* cur_ub) {
  int64_t seq, occ, cur;
  do {
    seq = m->mirror[MR_SEQ];
    __atomic_thread_fence(__ATOMIC_ACQUIRE);
    occ = m->mirror[MR_OCC];
    cur = m->mirror[MR_CUR];
    __atomic_thread_fence(__ATOMIC_ACQUIRE);
  } while (seq != m->mirror[MR_SEQ]);
  while (!m->in_flight.empty() && m->in_flight.front().first <= seq) m->in_flight.pop_front();
  int64_t pending = 0;
  for (const auto& c : m->in_flight) pending += c.second;
  if (occ_ub) *occ_ub = occ + pending;
  if (cur_ub) *cur_ub = cur + pending;
}

// After the stream has been drained and `words` read back: the mirror is exact.
void mirror_set(recis_idmap* m, const int64_t* words) {
  m->mirror[MR_CUR] = words[ST_CUR];
  m->mirror[MR_FREE] = words[ST_FREE];
  m->mirror[MR_LIVE] = words[ST_LIVE];
  m->mirror[MR_OCC] = words[ST_OCC];
  m->mirror[MR_SEQ] = m->seq_issued;
  m->in_flight.clear();
}

int rebuild(recis_idmap* m, int64_t new_capacity, hipStream_t stream) {
  Slot* nt = nullptr;
  if (int rc = alloc_table(m, new_capacity, stream, &nt)) return rc;
  rehash_kernel<<<dim3(blocks_for(m->capacity)), dim3(kBlock), 0, stream>>>(
      m->table, m->capacity, nt, static_cast<uint64_t>(new_capacity - 1));
  RECIS_LAUNCH_CHECK();
  int64_t words[ST_WORDS];
  if (int rc = sync_stats(m, stream, words)) return rc;
  // tombstones are gone: occupied == live
  RECIS_CHECK_HIP(hipMemcpyAsync(m->state + ST_OCC, &words[ST_LIVE], sizeof(int64_t),
                                 hipMemcpyHostToDevice, stream));
  RECIS_CHECK_HIP(hipStreamSynchronize(stream));
  RECIS_CHECK_HIP(hipFree(m->table));
  m->table = nt;
  m->capacity = new_capacity;
  m->occ_ub = words[ST_LIVE];
  m->mirror[MR_OCC] = words[ST_LIVE];
  return RECIS_OK;
}

// Make room for up to `incoming` more claimed slots.
int ensure_table_room(recis_idmap* m, int64_t incoming, hipStream_t stream) {
  mirror_bounds(m, &m->occ_ub, nullptr);
  if ((m->occ_ub + incoming) * 2 <= m->capacity) return RECIS_OK;
  int64_t words[ST_WORDS];
  if (int rc = sync_stats(m, stream, words)) return rc;
  if ((m->occ_ub + incoming) * 2 <= m->capacity) return RECIS_OK;
  const int64_t live = words[ST_LIVE];
  return rebuild(m, capacity_for(live + incoming + (live + incoming) / 2), stream);
}

int ensure_free_room(recis_idmap* m, int64_t incoming, hipStream_t stream) {
  if (m->free_ub + incoming <= m->free_cap) return RECIS_OK;
  int64_t words[ST_WORDS];
  if (int rc = sync_stats(m, stream, words)) return rc;
  if (m->free_ub + incoming <= m->free_cap) return RECIS_OK;
  int64_t cap = std::max<int64_t>(m->free_cap * 2, 10240);
  while (cap < m->free_ub + incoming) cap *= 2;
  int64_t* nf = nullptr;
  RECIS_CHECK_HIP(hipMalloc(reinterpret_cast<void**>(&nf), sizeof(int64_t) * static_cast<size_t>(cap)));
  if (m->free_ub > 0)
    RECIS_CHECK_HIP(hipMemcpyAsync(nf, m->free_list, sizeof(int64_t) * static_cast<size_t>(m->free_ub),
                                   hipMemcpyDeviceToDevice, stream));
  RECIS_CHECK_HIP(hipStreamSynchronize(stream));
  if (m->free_list) RECIS_CHECK_HIP(hipFree(m->free_list));
  m->free_list = nf;
  m->free_cap = cap;
  return RECIS_OK;
}

}  // namespace

namespace recis_hip {
int idmap_begin_call(recis_idmap* m, int64_t incoming, hipStream_t stream, int64_t* seq) {
  if (int rc = ensure_table_room(m, incoming, stream)) return rc;
  *seq = ++m->seq_issued;
  return RECIS_OK;
}
void idmap_end_call(recis_idmap* m, int64_t seq, int64_t incoming) { m->in_flight.emplace_back(seq, incoming); }
}  // namespace recis_hip

extern "C" {

int recis_idmap_create(int64_t reserve_keys, recis_idmap** out) {
  RECIS_REQUIRE(out != nullptr, "out must not be NULL");
  RECIS_REQUIRE(reserve_keys >= 0, "reserve_keys must be >= 0");
  recis_idmap* m = new recis_idmap();
  m->device = current_device();
  m->err = device_error_word(m->device);
  if (!m->err) {
    delete m;
    return fail(RECIS_ERR_HIP, "could not reach the device error word");
  }
  // The reference starts at 640000 slots (gpu_id_map.h:12); we start at the
  // next power of two unless the caller reserves more.
  m->capacity = capacity_for(std::max<int64_t>(reserve_keys, 320000));
  int rc = alloc_table(m, m->capacity, nullptr, &m->table);
  if (rc == RECIS_OK && hipMalloc(reinterpret_cast<void**>(&m->state), sizeof(int64_t) * ST_WORDS) != hipSuccess)
    rc = fail(RECIS_ERR_HIP, "hipMalloc of the allocator state failed");
  if (rc == RECIS_OK) {
    zero_words_kernel<<<1, 64>>>(m->state, ST_WORDS);
    if (hipStreamSynchronize(nullptr) != hipSuccess) rc = fail(RECIS_ERR_HIP, "id-map initialisation failed");
  }
  if (rc == RECIS_OK) {
    void* mp = nullptr;
    if (hipHostMalloc(&mp, sizeof(int64_t) * MR_WORDS, hipHostMallocDefault) != hipSuccess) {
      rc = fail(RECIS_ERR_HIP, "hipHostMalloc of the allocator mirror failed");
    } else {
      m->mirror = static_cast<volatile int64_t*>(mp);
      for (int w = 0; w < MR_WORDS; ++w) m->mirror[w] = 0;
    }
  }
  if (rc == RECIS_OK) rc = ensure_free_room(m, 10240, nullptr);
  if (rc != RECIS_OK) {
    if (m->mirror) (void)hipHostFree(const_cast<int64_t*>(m->mirror));
    if (m->table) (void)hipFree(m->table);
    if (m->state) (void)hipFree(m->state);
    delete m;
    return rc;
  }
  *out = m;
  return RECIS_OK;
}

int recis_idmap_destroy(recis_idmap* m) {
  if (!m) return RECIS_OK;
  (void)hipDeviceSynchronize();
  if (m->table) (void)hipFree(m->table);
  if (m->state) (void)hipFree(m->state);
  if (m->free_list) (void)hipFree(m->free_list);
  if (m->mirror) (void)hipHostFree(const_cast<int64_t*>(m->mirror));
  delete m;
  return RECIS_OK;
}

static int lookup_impl(recis_idmap* m, const int64_t* ids, int64_t n, const int64_t* n_dev, int64_t* index_out,
                       hipStream_t stream) {
  RECIS_REQUIRE(m != nullptr, "id map is NULL");
  RECIS_REQUIRE(n >= 0 && n < (int64_t(1) << 31), "n out of range: %lld", (long long)n);
  if (n == 0) return RECIS_OK;
  RECIS_REQUIRE(ids != nullptr && index_out != nullptr, "ids/index_out must not be NULL");
  if (int rc = ensure_table_room(m, n, stream)) return rc;
  const int64_t nb = blocks_for(n);
  void* ws = nullptr;
  const size_t ws_bytes = sizeof(int64_t) * static_cast<size_t>(n) + sizeof(int32_t) * static_cast<size_t>(nb);
  if (int rc = get_workspace(stream, ws_bytes, &ws)) return rc;
  int64_t* slotpos = static_cast<int64_t*>(ws);
  int32_t* block_counts = reinterpret_cast<int32_t*>(slotpos + n);
  const uint64_t mask = static_cast<uint64_t>(m->capacity - 1);
  const int64_t seq = ++m->seq_issued;

  RECIS_TIME_KERNEL("find_or_claim_kernel", stream)
  find_or_claim_kernel<<<dim3(nb), dim3(kBlock), 0, stream>>>(m->table, mask, ids, n, n_dev, index_out, slotpos,
                                                             block_counts, m->state, seq, m->err);
  RECIS_LAUNCH_CHECK();
  scan_commit_kernel<<<1, 1024, 0, stream>>>(block_counts, nb, n, n_dev, m->state, m->mirror, seq);
  RECIS_LAUNCH_CHECK();
  assign_rows_kernel<<<dim3(nb), dim3(kBlock), 0, stream>>>(m->table, slotpos, n, n_dev, block_counts, m->state,
                                                           m->free_list, index_out);
  RECIS_LAUNCH_CHECK();
  resolve_dups_kernel<<<dim3(nb), dim3(kBlock), 0, stream>>>(m->table, slotpos, n, n_dev, m->state, seq, index_out);
  RECIS_LAUNCH_CHECK();
  m->in_flight.emplace_back(seq, n);
  return RECIS_OK;
}

int recis_idmap_lookup(recis_idmap* m, const int64_t* ids, int64_t n, int64_t* index_out,
                       void* stream_) {
  return lookup_impl(m, ids, n, nullptr, index_out, static_cast<hipStream_t>(stream_));
}

int recis_idmap_lookup_counted(recis_idmap* m, const int64_t* ids, int64_t n_max, const int64_t* n_dev,
                               int64_t* index_out, void* stream_) {
  RECIS_REQUIRE(n_dev != nullptr, "n_dev must not be NULL");
  return lookup_impl(m, ids, n_max, n_dev, index_out, static_cast<hipStream_t>(stream_));
}

int recis_idmap_settle_count(recis_idmap* m, int64_t n_true) {
  RECIS_REQUIRE(m != nullptr && n_true >= 0, "bad arguments");
  if (!m->in_flight.empty() && m->in_flight.back().first == m->seq_issued && m->in_flight.back().second > n_true)
    m->in_flight.back().second = n_true;
  return RECIS_OK;
}

int recis_idmap_last_call(recis_idmap* m, int64_t* seq) {
  RECIS_REQUIRE(m != nullptr && seq != nullptr, "bad arguments");
  *seq = m->seq_issued;
  return RECIS_OK;
}

int recis_idmap_settle_call(recis_idmap* m, int64_t seq, int64_t n_true) {
  RECIS_REQUIRE(m != nullptr && n_true >= 0, "bad arguments");
  for (auto& c : m->in_flight) {
    if (c.first == seq) {
      if (c.second > n_true) c.second = n_true;
      break;
    }
  }
  return RECIS_OK;  // a call whose publication has landed is not in the list any more: nothing to settle
}

int recis_idmap_bounds(recis_idmap* m, int64_t* id_num_ub, int64_t* occupied_ub) {
  RECIS_REQUIRE(m != nullptr, "id map is NULL");
  mirror_bounds(m, occupied_ub, id_num_ub);
  return RECIS_OK;
}

int recis_idmap_lookup_readonly(recis_idmap* m, const int64_t* ids, int64_t n, int64_t* index_out,
                                void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(m != nullptr, "id map is NULL");
  RECIS_REQUIRE(n >= 0, "n out of range: %lld", (long long)n);
  if (n == 0) return RECIS_OK;
  RECIS_REQUIRE(ids != nullptr && index_out != nullptr, "ids/index_out must not be NULL");
  find_kernel<<<dim3(blocks_for(n)), dim3(kBlock), 0, stream>>>(
      m->table, static_cast<uint64_t>(m->capacity - 1), ids, n, index_out);
  RECIS_LAUNCH_CHECK();
  return RECIS_OK;
}

int recis_idmap_erase(recis_idmap* m, const int64_t* ids, const int64_t* index, int64_t n,
                      void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(m != nullptr, "id map is NULL");
  RECIS_REQUIRE(n >= 0, "n out of range: %lld", (long long)n);
  if (n == 0) return RECIS_OK;
  RECIS_REQUIRE(ids != nullptr && index != nullptr, "ids/index must not be NULL");
  if (int rc = ensure_free_room(m, n, stream)) return rc;
  erase_kernel<<<dim3(blocks_for(n)), dim3(kBlock), 0, stream>>>(
      m->table, static_cast<uint64_t>(m->capacity - 1), ids, index, n, m->free_list, m->state);
  RECIS_LAUNCH_CHECK();
  erase_commit_kernel<<<1, 1, 0, stream>>>(m->state, n);
  RECIS_LAUNCH_CHECK();
  m->free_ub += n;
  return RECIS_OK;
}

int recis_idmap_stats(recis_idmap* m, int64_t* live, int64_t* id_num, int64_t* free_size,
                      int64_t* capacity, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(m != nullptr, "id map is NULL");
  int64_t words[ST_WORDS];
  if (int rc = sync_stats(m, stream, words)) return rc;
  if (live) *live = words[ST_LIVE];
  if (id_num) *id_num = words[ST_CUR];
  if (free_size) *free_size = words[ST_FREE];
  if (capacity) *capacity = m->capacity;
  return RECIS_OK;
}

int recis_idmap_snapshot(recis_idmap* m, int64_t* ids_out, int64_t* index_out, int64_t max_out,
                         int64_t* count, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(m != nullptr && count != nullptr, "id map / count is NULL");
  RECIS_REQUIRE(max_out >= 0 && (max_out == 0 || (ids_out && index_out)), "bad output buffers");
  snapshot_kernel<<<dim3(blocks_for(m->capacity)), dim3(kBlock), 0, stream>>>(
      m->table, m->capacity, ids_out, index_out, max_out, m->state);
  RECIS_LAUNCH_CHECK();
  int64_t words[ST_WORDS];
  if (int rc = sync_stats(m, stream, words)) return rc;
  *count = words[ST_TMP];
  zero_words_kernel<<<1, 64, 0, stream>>>(m->state + ST_TMP, 1);
  RECIS_LAUNCH_CHECK();
  return RECIS_OK;
}

int recis_idmap_evict_older(recis_idmap* m, const void* const* stamp_blocks_dev, int64_t n_blocks,
                            int64_t block_rows, int stamp_is64, int64_t threshold, int64_t* ids_out,
                            int64_t* index_out, int64_t max_out, int64_t* count, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(m != nullptr && count != nullptr, "id map / count is NULL");
  RECIS_REQUIRE(stamp_blocks_dev != nullptr && n_blocks >= 0 && block_rows > 0, "bad stamp blocks");
  RECIS_REQUIRE(max_out >= 0 && (max_out == 0 || (ids_out && index_out)), "bad output buffers");
  *count = 0;
  if (max_out == 0) return RECIS_OK;
  int* err = device_error_word(current_device());
  RECIS_REQUIRE(err != nullptr, "could not reach the device error word");
  if (int rc = ensure_free_room(m, max_out, stream)) return rc;
  const int64_t rounds = (m->capacity + static_cast<int64_t>(kBlock) * kEvictPer - 1) / (static_cast<int64_t>(kBlock) * kEvictPer);
  evict_older_kernel<<<dim3(static_cast<unsigned>(std::min<int64_t>(rounds, 256 * 16))), dim3(kBlock), 0, stream>>>(
      m->table, m->capacity, stamp_blocks_dev, n_blocks, block_rows, stamp_is64, threshold, ids_out, index_out,
      max_out, m->free_list, m->state, err);
  RECIS_LAUNCH_CHECK();
  evict_commit_kernel<<<1, 1, 0, stream>>>(m->state, max_out);
  RECIS_LAUNCH_CHECK();
  int64_t words[ST_WORDS];
  if (int rc = sync_stats(m, stream, words)) return rc;
  *count = std::min<int64_t>(words[ST_TMP], max_out);
  m->free_ub += *count;
  zero_words_kernel<<<1, 64, 0, stream>>>(m->state + ST_TMP, 1);
  RECIS_LAUNCH_CHECK();
  return RECIS_OK;
}

int recis_idmap_clear(recis_idmap* m, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(m != nullptr, "id map is NULL");
  int64_t grid = std::min<int64_t>(blocks_for(m->capacity), 256 * 64);
  fill_slots_kernel<<<dim3(grid), dim3(kBlock), 0, stream>>>(m->table, m->capacity);
  RECIS_LAUNCH_CHECK();
  zero_words_kernel<<<1, 64, 0, stream>>>(m->state, ST_WORDS);
  RECIS_LAUNCH_CHECK();
  const int64_t seq = ++m->seq_issued;
  publish_kernel<<<1, 1, 0, stream>>>(m->state, m->mirror, seq);
  RECIS_LAUNCH_CHECK();
  m->in_flight.emplace_back(seq, 0);
  m->free_ub = 0;
  return RECIS_OK;
}

int recis_idmap_reserve(recis_idmap* m, int64_t n_keys, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(m != nullptr, "id map is NULL");
  const int64_t want = capacity_for(n_keys);
  if (want <= m->capacity) return RECIS_OK;
  return rebuild(m, want, stream);
}

int recis_generate_ids(int64_t n, const int64_t* const* free_blocks_dev, int64_t free_count,
                       int64_t cur_count, int64_t free_block_size, int64_t* out, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(n >= 0 && free_block_size > 0, "bad sizes");
  if (n == 0) return RECIS_OK;
  RECIS_REQUIRE(out != nullptr && (free_blocks_dev != nullptr || free_count == 0), "NULL argument");
  generate_ids_kernel<<<dim3(blocks_for(n)), dim3(kBlock), 0, stream>>>(n, free_blocks_dev, free_count,
                                                                       cur_count, free_block_size, out);
  RECIS_LAUNCH_CHECK();
  return RECIS_OK;
}

int recis_free_ids(const int64_t* ids, int64_t n, int64_t* const* free_blocks_dev, int64_t free_count,
                   int64_t free_block_size, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(n >= 0 && free_block_size > 0, "bad sizes");
  if (n == 0) return RECIS_OK;
  RECIS_REQUIRE(ids != nullptr && free_blocks_dev != nullptr, "NULL argument");
  free_ids_kernel<<<dim3(blocks_for(n)), dim3(kBlock), 0, stream>>>(ids, n, free_blocks_dev, free_count,
                                                                   free_block_size);
  RECIS_LAUNCH_CHECK();
  return RECIS_OK;
}

int recis_mask_key_index(const int64_t* keys, const uint8_t* mask, const int64_t* cumsum, int64_t n,
                         int64_t out_size, int64_t* out_keys, int64_t* out_index, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(n >= 0 && out_size >= 0, "bad sizes");
  if (n == 0 || out_size == 0) return RECIS_OK;
  RECIS_REQUIRE(keys && mask && cumsum && out_keys && out_index, "NULL argument");
  int* err = device_error_word(current_device());
  mask_key_index_kernel<<<dim3(blocks_for(n)), dim3(kBlock), 0, stream>>>(keys, mask, cumsum, n, out_size,
                                                                         out_keys, out_index, err);
  RECIS_LAUNCH_CHECK();
  return RECIS_OK;
}

int recis_scatter_ids_with_mask(int64_t* out_ids, int64_t out_size, const int64_t* in_ids,
                                const int64_t* mask_index, int64_t n, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  RECIS_REQUIRE(n >= 0 && out_size >= 0, "bad sizes");
  if (n == 0 || out_size == 0) return RECIS_OK;
  RECIS_REQUIRE(out_ids && in_ids && mask_index, "NULL argument");
  int* err = device_error_word(current_device());
  scatter_ids_kernel<<<dim3(blocks_for(n)), dim3(kBlock), 0, stream>>>(out_ids, out_size, in_ids,
                                                                      mask_index, n, err);
  RECIS_LAUNCH_CHECK();
  return RECIS_OK;
}

}  // extern "C"
