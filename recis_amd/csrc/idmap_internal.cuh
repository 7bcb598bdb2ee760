// Internals of the id map shared by idmap.hip (the map's own entry points) and plan.hip (the
// batch plan that probes the map from inside its bucket kernel): slot layout, allocator words,
// the probe.
#pragma once
#include <hip/hip_runtime.h>

#include <deque>
#include <utility>

#include "common.cuh"

namespace recis_hip {

struct alignas(16) Slot {
  int64_t key;
  int64_t val;
};

constexpr int64_t kEmpty = -1;
constexpr int64_t kTomb = -2;
constexpr int64_t kValUnset = -1;

// allocator words in device memory
enum { ST_CUR = 0, ST_FREE, ST_LIVE, ST_OCC, ST_NNEW, ST_OLD_CUR, ST_OLD_FREE, ST_TMP, ST_DUPS, ST_WORDS };
// the words the host wants to know without waiting for the stream: written by the last kernel of
// every call that changes them into pinned host memory, stamped with the call's sequence number
// (written last, after a system-scope fence)
enum { MR_SEQ = 0, MR_CUR, MR_FREE, MR_LIVE, MR_OCC, MR_WORDS };

__device__ __forceinline__ uint64_t mix_key(int64_t key) {
  uint64_t x = static_cast<uint64_t>(key);
  x ^= x >> 33;
  x *= 0xff51afd7ed558ccdULL;
  x ^= x >> 33;
  x *= 0xc4ceb9fe1a85ec53ULL;
  x ^= x >> 33;
  return x;
}

// First slot probed for a key: the TOP bits of the mixed key. Batches come out of the batch
// plan ordered by the top bits of the same mix, so their probes walk the table front to back.
__device__ __forceinline__ uint64_t home_slot_of_mix(uint64_t mixed, uint64_t mask) {
  return mixed >> __builtin_clzll(mask);  // mask = capacity - 1, capacity a power of two >= 2
}
__device__ __forceinline__ uint64_t home_slot(int64_t key, uint64_t mask) {
  return home_slot_of_mix(mix_key(key), mask);
}

__device__ __forceinline__ void publish(const int64_t* state, volatile int64_t* mirror, int64_t seq) {
  mirror[MR_CUR] = state[ST_CUR];
  mirror[MR_FREE] = state[ST_FREE];
  mirror[MR_LIVE] = state[ST_LIVE];
  mirror[MR_OCC] = state[ST_OCC];
  __threadfence_system();
  mirror[MR_SEQ] = seq;
}

__device__ __forceinline__ int64_t ld_relaxed(const int64_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_relaxed(int64_t* p, int64_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// What one probe of find-or-insert found.
enum ProbeResult { kProbeFound = 0, kProbeClaimed = 1, kProbePending = 2, kProbeFull = 3 };

// Find `key` or claim a slot for it. `hint` is a plain 16-byte load of the key's home slot that the
// caller has issued already (L1-cacheable, may be stale). Two things a hint shows cannot change
// while the calling kernel runs: a key with an assigned row, and a slot held by another key.
//   kProbeFound:   *value = the key's row
//   kProbeClaimed: this thread claimed slot *slot for the key (its value now holds `pending`,
//                  a negative number); *took_empty says whether an empty slot (not a tombstone) was used
//   kProbePending: the key is being inserted by another thread of this call, in slot *slot
//   kProbeFull:    the probe sequence found no slot
__device__ __forceinline__ ProbeResult probe_or_claim(Slot* __restrict__ table, uint64_t mask, int64_t key,
                                                       uint64_t home, longlong2 hint, int64_t pending,
                                                       int64_t* value, int64_t* slot, bool* took_empty) {
  uint64_t p = home;
  int64_t first_tomb = -1;
  uint64_t probes = 0;
  bool have_hint = true;
  for (;;) {
    if (!have_hint) hint = *reinterpret_cast<const longlong2*>(&table[p]);
    have_hint = false;
    if (hint.x == key && hint.y >= 0) {
      *value = hint.y;
      return kProbeFound;
    }
    if (hint.x != key && hint.x != kEmpty && hint.x != kTomb) {
      p = (p + 1) & mask;
      if (++probes > mask) return kProbeFull;
      continue;
    }
    const int64_t k = ld_relaxed(&table[p].key);
    if (k == key) {
      const int64_t v = ld_relaxed(&table[p].val);
      if (v >= 0) {
        *value = v;
        return kProbeFound;
      }
      *slot = static_cast<int64_t>(p);
      return kProbePending;
    }
    if (k == kEmpty) {
      const bool use_tomb = first_tomb >= 0;
      const int64_t target = use_tomb ? first_tomb : static_cast<int64_t>(p);
      const int64_t expect = use_tomb ? kTomb : kEmpty;
      const int64_t old = static_cast<int64_t>(atomicCAS(reinterpret_cast<unsigned long long*>(&table[target].key),
                                                         static_cast<unsigned long long>(expect),
                                                         static_cast<unsigned long long>(key)));
      if (old == expect) {
        st_relaxed(&table[target].val, pending);
        *slot = target;
        *took_empty = !use_tomb;
        return kProbeClaimed;
      }
      // somebody else took that slot: start over, keys never vanish meanwhile
      p = home;
      first_tomb = -1;
      probes = 0;
      continue;
    }
    if (k == kTomb && first_tomb < 0) first_tomb = static_cast<int64_t>(p);
    p = (p + 1) & mask;
    if (++probes > mask) return kProbeFull;
  }
}

// Row of the rank-th of n_new missing keys of a call (IdGeneratorFunctor, csrc/ops/hashtable_ops.cc:15-27):
// the tail of the free list first, then fresh indices counting down from the new high-water mark.
__device__ __forceinline__ int64_t row_of_new_key(int64_t rank, int64_t n_new, int64_t old_cur, int64_t old_free,
                                                  const int64_t* __restrict__ free_list) {
  const int64_t free_index = old_free - n_new + rank;
  return free_index >= 0 ? free_list[free_index] : old_cur - (free_index + 1);
}

// The allocator bookkeeping of IdAllocator::GenIds (id_allocator.cc:17-26) for a call that found
// `total` missing keys. One thread; publish() the words to the host mirror once every kernel that
// adds to ST_OCC has finished.
__device__ __forceinline__ void commit_new_keys(int64_t* state, int64_t total) {
  const int64_t cur = state[ST_CUR], fr = state[ST_FREE];
  state[ST_OLD_CUR] = cur;
  state[ST_OLD_FREE] = fr;
  state[ST_NNEW] = total;
  const int64_t fresh = fr >= total ? 0 : total - fr;
  state[ST_CUR] = cur + fresh;
  state[ST_FREE] = fr >= total ? fr - total : 0;
  state[ST_LIVE] += total;
  __threadfence();
}

}  // namespace recis_hip

struct recis_idmap {
  int device = 0;
  int64_t capacity = 0;
  recis_hip::Slot* table = nullptr;
  int64_t* state = nullptr;      // device, ST_WORDS int64
  int64_t* free_list = nullptr;  // device
  int64_t free_cap = 0;
  // host-side upper bounds, refreshed by sync_stats()
  int64_t occ_ub = 0;   // non-empty slots (live + tombstones)
  int64_t free_ub = 0;  // entries in the free list
  int* err = nullptr;
  // pinned host mirror of the allocator words + the calls whose publication has not landed yet
  volatile int64_t* mirror = nullptr;
  int64_t seq_issued = 0;
  std::deque<std::pair<int64_t, int64_t>> in_flight;  // (sequence number, ids of the call)
};

namespace recis_hip {
// Host side of a find-or-insert call of up to `incoming` ids: makes room in the slot table (may
// rebuild it, waiting for the stream), numbers the call. Pair with idmap_end_call once the
// kernels are queued.
int idmap_begin_call(recis_idmap* m, int64_t incoming, hipStream_t stream, int64_t* seq);
void idmap_end_call(recis_idmap* m, int64_t seq, int64_t incoming);
}  // namespace recis_hip
