/*
 * recis_oracle.c - TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A plain-C, CPU restatement of the algorithms on RecIS's sparse-embedding hot
 * path, used only as the checker in tests/, in __graft_entry__.smoke() and as
 * the timed CPU baseline in bench.py. Nothing in recis_amd/ may call it.
 *
 * Each function cites the reference file:line (relative to the alibaba/RecIS
 * tree) whose behaviour it restates. Where the reference has no CPU code for an
 * op (the CUDA-only pooling and hash kernels) the kernel's arithmetic is
 * restated element by element in a sequential loop.
 *
 * Parity status: every function here is pinned by a reference known-answer
 * vector, a closed form / library routine, or a brute-force model in
 * tests/test_oracle_*.py, except those marked "parity unpinned" below:
 *   (none so far)
 * and tests/test_oracle_ref_ops.py compares the table, allocator, row-block,
 * optimizer, tagging, partition and feature functions bit for bit with the
 * reference's own CPU operators where oracle/_ref/ref_ops has been built.
 * Additions with no reference counterpart (MAX combiner, Adagrad row update)
 * are pinned by torch / textbook closed forms instead.
 *
 * Loops the reference runs under at::parallel_for carry an OpenMP pragma; with
 * OMP_NUM_THREADS=1 (the default used by the tests) everything is sequential
 * and deterministic.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORACLE_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------------- *
 * Pooling, ragged mode.
 * Restates segment_reduce_forward_kernel / segment_reduce_backward_kernel,
 * csrc/ops/embedding_segment_reduce_kernel.cu:23-75 and :79-120:
 *   w = weight[idx] (1 without weights); MEAN: w = w / length (in float);
 *   forward:  SUM/MEAN out[s] += emb[rev[idx]] * w ; TILE out[idx] = emb[rev[idx]] * w
 *   backward: g[rev[idx]] += grad[s or idx] * w
 * Accumulation is sequential in float (the reference's atomic order is
 * unspecified). mode: 0 sum, 1 mean, 2 tile. offsets has S+1 entries.
 * ------------------------------------------------------------------------- */
ORACLE_API void oracle_segment_reduce_forward(const float* emb, const float* weight,
                                              const int64_t* rev, const int64_t* offsets,
                                              float* out, int64_t B, int64_t U, int64_t S,
                                              int64_t D, int mode) {
  int64_t out_rows = (mode == 2) ? B : S;
  memset(out, 0, sizeof(float) * (size_t)(out_rows * D));
  for (int64_t s = 0; s < S; ++s) {
    int64_t start = offsets[s], end = offsets[s + 1];
    int64_t length = end - start;
    for (int64_t idx = start; idx < end; ++idx) {
      int64_t raw = rev ? rev[idx] : idx;
      float w = weight ? weight[idx] : 1.0f;
      if (mode == 1) w = w / (float)length;
      const float* src = emb + raw * D;
      if (mode == 2) {
        for (int64_t d = 0; d < D; ++d) out[idx * D + d] = src[d] * w;
      } else {
        for (int64_t d = 0; d < D; ++d) out[s * D + d] += src[d] * w;
      }
    }
  }
  (void)U;
}

ORACLE_API void oracle_segment_reduce_backward(const float* grad, const float* weight,
                                               const int64_t* rev, const int64_t* offsets,
                                               float* grad_unique, int64_t B, int64_t U,
                                               int64_t S, int64_t D, int mode) {
  memset(grad_unique, 0, sizeof(float) * (size_t)(U * D));
  for (int64_t s = 0; s < S; ++s) {
    int64_t start = offsets[s], end = offsets[s + 1];
    int64_t length = end - start;
    for (int64_t idx = start; idx < end; ++idx) {
      int64_t raw = rev ? rev[idx] : idx;
      float w = weight ? weight[idx] : 1.0f;
      if (mode == 1) w /= (float)length;
      const float* g = (mode == 2) ? grad + idx * D : grad + s * D;
      for (int64_t d = 0; d < D; ++d) grad_unique[raw * D + d] += g[d] * w;
    }
  }
  (void)B;
}

/* Same forward with double accumulators: used by tests to bound the rounding
 * error of any fp32 summation order. Also returns sum |w * x| per output. */
ORACLE_API void oracle_segment_reduce_forward_f64(const float* emb, const float* weight,
                                                  const int64_t* rev, const int64_t* offsets,
                                                  double* out, double* out_abs, int64_t S,
                                                  int64_t D, int mean) {
  for (int64_t s = 0; s < S; ++s) {
    int64_t start = offsets[s], end = offsets[s + 1];
    for (int64_t d = 0; d < D; ++d) out[s * D + d] = out_abs[s * D + d] = 0.0;
    for (int64_t idx = start; idx < end; ++idx) {
      int64_t raw = rev ? rev[idx] : idx;
      double w = weight ? (double)weight[idx] : 1.0;
      if (mean) w /= (double)(end - start);
      for (int64_t d = 0; d < D; ++d) {
        double t = (double)emb[raw * D + d] * w;
        out[s * D + d] += t;
        out_abs[s * D + d] += fabs(t);
      }
    }
  }
}

/* MAX combiner (no reference counterpart): element-wise maximum over the
 * segment's rows, first occurrence wins ties, NaN propagates, empty segment
 * gives 0 and argmax -1. argmax holds the absolute occurrence index. */
ORACLE_API void oracle_segment_max_forward(const float* emb, const int64_t* rev,
                                           const int64_t* offsets, float* out,
                                           int32_t* argmax, int64_t S, int64_t D) {
  for (int64_t s = 0; s < S; ++s) {
    int64_t start = offsets[s], end = offsets[s + 1];
    for (int64_t d = 0; d < D; ++d) {
      float best = 0.0f;
      int32_t arg = -1;
      for (int64_t idx = start; idx < end; ++idx) {
        int64_t raw = rev ? rev[idx] : idx;
        float v = emb[raw * D + d];
        if (arg < 0 || v > best || (v != v && best == best)) {
          best = v;
          arg = (int32_t)idx;
        }
      }
      out[s * D + d] = best;
      argmax[s * D + d] = arg;
    }
  }
}

ORACLE_API void oracle_segment_max_backward(const float* grad, const int32_t* argmax,
                                            const int64_t* rev, float* grad_unique,
                                            int64_t U, int64_t S, int64_t D) {
  memset(grad_unique, 0, sizeof(float) * (size_t)(U * D));
  for (int64_t e = 0; e < S * D; ++e) {
    int32_t r = argmax[e];
    if (r < 0) continue;
    int64_t raw = rev ? rev[r] : r;
    grad_unique[raw * D + e % D] += grad[e];
  }
}

/* merge_offsets, csrc/ops/embedding_segment_reduce_kernel.cu:357-391:
 * tensor i contributes its first n_i - 1 entries (all n_i for the last one),
 * each shifted by prefix_i = sum_{j<i} max_value[j]. */
ORACLE_API int64_t oracle_merge_offsets(const int64_t* const* offsets, const int64_t* sizes,
                                        const int64_t* max_value, int64_t n, int64_t* out) {
  int64_t pos = 0, prefix = 0;
  for (int64_t i = 0; i < n; ++i) {
    int64_t take = (i < n - 1) ? sizes[i] - 1 : sizes[i];
    for (int64_t k = 0; k < take; ++k) out[pos++] = offsets[i][k] + prefix;
    prefix += max_value[i];
  }
  return pos;
}

/* gen_segment_indices_by_offset, embedding_segment_reduce_kernel.cu:395-423 */
ORACLE_API void oracle_gen_segment_indices(const int64_t* offsets, int64_t S, int64_t* out) {
  for (int64_t i = 1; i <= S; ++i)
    for (int64_t j = offsets[i - 1]; j < offsets[i]; ++j) out[j] = i - 1;
}

/* ------------------------------------------------------------------------- *
 * Pooling, sparse mode.
 * segment_sum_kernel, csrc/ops/segment_ops_kernel.cu:133-165:
 *   out[seg[i]] += data[indices[i]] * w[i]   (w = weight[0] broadcast if !use_weight)
 * segment_weight_sum_kernel / segment_weight_norm_kernel, :74-108:
 *   sum[seg] += w_i for 0 <= seg < num_segments; norm_i = w_i / sum[seg_i];
 *   an out-of-range segment id keeps the raw weight.
 * ------------------------------------------------------------------------- */
ORACLE_API void oracle_segment_sum(const float* data, const float* weight, int use_weight,
                                   const int64_t* indices, const int64_t* seg_ids,
                                   float* out, int64_t n, int64_t num_segments, int64_t D) {
  memset(out, 0, sizeof(float) * (size_t)(num_segments * D));
  for (int64_t i = 0; i < n; ++i) {
    float w = weight[use_weight ? i : 0];
    const float* src = data + indices[i] * D;
    float* dst = out + seg_ids[i] * D;
    for (int64_t d = 0; d < D; ++d) dst[d] += src[d] * w;
  }
}

ORACLE_API void oracle_segment_mean_weight(const float* weight, int use_weight,
                                           const int64_t* seg_ids, float* weight_sum,
                                           float* weight_norm, int64_t n,
                                           int64_t num_segments) {
  for (int64_t s = 0; s < num_segments; ++s) weight_sum[s] = 0.0f;
  for (int64_t i = 0; i < n; ++i) {
    int64_t s = seg_ids[i];
    if (s < 0 || s >= num_segments) continue;
    weight_sum[s] += weight[use_weight ? i : 0];
  }
  for (int64_t i = 0; i < n; ++i) {
    int64_t s = seg_ids[i];
    float w = weight[use_weight ? i : 0];
    weight_norm[i] = (s < 0 || s >= num_segments) ? w : w / weight_sum[s];
  }
}

/* ------------------------------------------------------------------------- *
 * Unpooled padded gather.
 * ragged_tile / ragged_tile_back, csrc/ops/ragged_tile_kernel.cu:26-60,93-131,
 * 214-280: features are concatenated; feature f has batch[f] samples whose
 * offsets occupy offset[obase_f .. obase_f + batch[f]] (obase_f = sum of
 * earlier batch sizes, the per-feature offsets having been merged so that each
 * boundary is shared); sample b of feature f fills seq[f] output rows starting
 * at row (sum_{g<f} batch[g]*seq[g]) + b*seq[f]: row t is table[value[start+t]]
 * for t < min(len, seq[f]), zero otherwise. Weights play no part.
 * ------------------------------------------------------------------------- */
ORACLE_API void oracle_ragged_tile(const int64_t* batch, const int64_t* seq, int64_t nfeat,
                                   const int64_t* value, const int64_t* offset,
                                   const float* table, float* out, int64_t D) {
  int64_t obase = 0, rbase = 0;
  for (int64_t f = 0; f < nfeat; ++f) {
    for (int64_t b = 0; b < batch[f]; ++b) {
      int64_t start = offset[obase + b], len = offset[obase + b + 1] - start;
      float* dst = out + (rbase + b * seq[f]) * D;
      for (int64_t t = 0; t < seq[f]; ++t) {
        if (t < len)
          memcpy(dst + t * D, table + value[start + t] * D, sizeof(float) * (size_t)D);
        else
          memset(dst + t * D, 0, sizeof(float) * (size_t)D);
      }
    }
    obase += batch[f];
    rbase += batch[f] * seq[f];
  }
}

ORACLE_API void oracle_ragged_tile_back(const int64_t* batch, const int64_t* seq,
                                        int64_t nfeat, const int64_t* value,
                                        const int64_t* offset, const float* dy,
                                        float* d_table, int64_t table_rows, int64_t D) {
  memset(d_table, 0, sizeof(float) * (size_t)(table_rows * D));
  int64_t obase = 0, rbase = 0;
  for (int64_t f = 0; f < nfeat; ++f) {
    for (int64_t b = 0; b < batch[f]; ++b) {
      int64_t start = offset[obase + b], len = offset[obase + b + 1] - start;
      int64_t rows = len < seq[f] ? len : seq[f];
      const float* src = dy + (rbase + b * seq[f]) * D;
      for (int64_t t = 0; t < rows; ++t) {
        float* dst = d_table + value[start + t] * D;
        for (int64_t d = 0; d < D; ++d) dst[d] += src[t * D + d];
      }
    }
    obase += batch[f];
    rbase += batch[f] * seq[f];
  }
}

/* ------------------------------------------------------------------------- *
 * Row-index allocator.
 * IdGeneratorFunctor / IdFreeFunctor, csrc/ops/hashtable_ops.cc:5-58, and
 * IdAllocator::GenIds / FreeIds, csrc/embedding/id_allocator.cc:17-34:
 *   for i in [0, n): free_index = free_count - n + i
 *     free_index >= 0 -> recycled id free_list[free_index]
 *     else            -> fresh id cur_count - (free_index + 1)   (descending)
 *   afterwards cur += max(0, n - free), free = max(0, free - n);
 *   FreeIds appends ids at free_list[free_count ...].
 * The free list is kept here as one flat growable array; the reference's
 * 10240-entry blocks only chunk that same array.
 * ------------------------------------------------------------------------- */
ORACLE_API void oracle_generate_ids(int64_t n, const int64_t* free_list, int64_t free_count,
                                    int64_t cur_count, int64_t* out) {
  for (int64_t i = 0; i < n; ++i) {
    int64_t free_index = free_count - n + i;
    out[i] = (free_index >= 0) ? free_list[free_index] : cur_count - (free_index + 1);
  }
}

typedef struct {
  int64_t cur_size;
  int64_t free_size;
  int64_t* free_list;
  int64_t free_cap;
} OracleAllocator;

static void alloc_gen(OracleAllocator* a, int64_t n, int64_t* out) {
  oracle_generate_ids(n, a->free_list, a->free_size, a->cur_size, out);
  int64_t fresh = (a->free_size >= n) ? 0 : n - a->free_size;
  a->cur_size += fresh;
  a->free_size = (a->free_size - n > 0) ? a->free_size - n : 0;
}

static void alloc_free(OracleAllocator* a, const int64_t* ids, int64_t n) {
  if (a->free_size + n > a->free_cap) {
    int64_t cap = a->free_cap ? a->free_cap : 1024;
    while (cap < a->free_size + n) cap *= 2;
    a->free_list = (int64_t*)realloc(a->free_list, sizeof(int64_t) * (size_t)cap);
    a->free_cap = cap;
  }
  memcpy(a->free_list + a->free_size, ids, sizeof(int64_t) * (size_t)n);
  a->free_size += n;
}

/* mask_key_index / scatter_ids_with_mask, csrc/ops/hashtable_ops.cc:150-214 */
ORACLE_API void oracle_mask_key_index(const int64_t* keys, const uint8_t* mask,
                                      const int64_t* cumsum, int64_t n, int64_t* out_keys,
                                      int64_t* out_index) {
  for (int64_t i = 0; i < n; ++i) {
    if (mask[i]) {
      out_keys[cumsum[i] - 1] = keys[i];
      out_index[cumsum[i] - 1] = i;
    }
  }
}

ORACLE_API void oracle_scatter_ids_with_mask(int64_t* out_ids, const int64_t* in_ids,
                                             const int64_t* mask_index, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out_ids[mask_index[i]] = in_ids[i];
}

/* ------------------------------------------------------------------------- *
 * Key -> row map.
 * CpuIdMap, csrc/embedding/cpu_id_map.cc:73-174: Lookup finds every id; ids not
 * present are collected in input order (one thread), get indices from
 * GenIds(n_missing) and are inserted one by one; `insert` does not overwrite,
 * so a key repeated inside one call takes the index of its first insertion
 * while later indices of that batch are leaked. LookupReadOnly returns -1 for
 * a missing key. DeleteIds erases the keys and frees `index` as given.
 * The container here is a linear-probing table; the reference uses
 * ska::flat_hash_map, whose iteration order is not part of the contract.
 * ------------------------------------------------------------------------- */
typedef struct {
  int64_t* keys;
  int64_t* vals;
  uint8_t* state; /* 0 empty, 1 full, 2 tombstone */
  int64_t cap;    /* power of two */
  int64_t size;
  int64_t used; /* full + tombstones */
  OracleAllocator alloc;
} OracleIdMap;

static uint64_t mix64(uint64_t x) {
  x ^= x >> 33;
  x *= 0xff51afd7ed558ccdULL;
  x ^= x >> 33;
  x *= 0xc4ceb9fe1a85ec53ULL;
  x ^= x >> 33;
  return x;
}

static void idmap_alloc_table(OracleIdMap* m, int64_t cap) {
  m->keys = (int64_t*)malloc(sizeof(int64_t) * (size_t)cap);
  m->vals = (int64_t*)malloc(sizeof(int64_t) * (size_t)cap);
  m->state = (uint8_t*)calloc((size_t)cap, 1);
  m->cap = cap;
  m->size = 0;
  m->used = 0;
}

ORACLE_API OracleIdMap* oracle_idmap_create(int64_t reserve) {
  OracleIdMap* m = (OracleIdMap*)calloc(1, sizeof(OracleIdMap));
  int64_t cap = 1024;
  while (cap < reserve * 2) cap *= 2;
  idmap_alloc_table(m, cap);
  return m;
}

ORACLE_API void oracle_idmap_destroy(OracleIdMap* m) {
  if (!m) return;
  free(m->keys);
  free(m->vals);
  free(m->state);
  free(m->alloc.free_list);
  free(m);
}

static int64_t idmap_find_slot(const OracleIdMap* m, int64_t key) {
  uint64_t mask = (uint64_t)m->cap - 1;
  uint64_t p = mix64((uint64_t)key) & mask;
  while (m->state[p] != 0) {
    if (m->state[p] == 1 && m->keys[p] == key) return (int64_t)p;
    p = (p + 1) & mask;
  }
  return -1;
}

static void idmap_put_new(OracleIdMap* m, int64_t key, int64_t val);

static void idmap_grow(OracleIdMap* m) {
  OracleIdMap old = *m;
  int64_t cap = old.cap;
  if (old.size * 4 >= old.cap) cap *= 2; /* else only purge tombstones */
  idmap_alloc_table(m, cap);
  for (int64_t i = 0; i < old.cap; ++i)
    if (old.state[i] == 1) idmap_put_new(m, old.keys[i], old.vals[i]);
  free(old.keys);
  free(old.vals);
  free(old.state);
}

static void idmap_put_new(OracleIdMap* m, int64_t key, int64_t val) {
  if ((m->used + 1) * 2 > m->cap) idmap_grow(m);
  uint64_t mask = (uint64_t)m->cap - 1;
  uint64_t p = mix64((uint64_t)key) & mask;
  while (m->state[p] == 1) p = (p + 1) & mask;
  if (m->state[p] == 0) m->used++;
  m->state[p] = 1;
  m->keys[p] = key;
  m->vals[p] = val;
  m->size++;
}

ORACLE_API void oracle_idmap_lookup(OracleIdMap* m, const int64_t* ids, int64_t n,
                                    int64_t* out) {
  int64_t* miss_pos = (int64_t*)malloc(sizeof(int64_t) * (size_t)(n > 0 ? n : 1));
  int64_t n_miss = 0;
  /* sequential: the order of the misses must be the input order */
  for (int64_t i = 0; i < n; ++i) {
    int64_t slot = idmap_find_slot(m, ids[i]);
    if (slot >= 0)
      out[i] = m->vals[slot];
    else
      miss_pos[n_miss++] = i;
  }
  int64_t* new_index = (int64_t*)malloc(sizeof(int64_t) * (size_t)(n_miss > 0 ? n_miss : 1));
  alloc_gen(&m->alloc, n_miss, new_index);
  for (int64_t k = 0; k < n_miss; ++k) {
    int64_t i = miss_pos[k];
    int64_t slot = idmap_find_slot(m, ids[i]);
    if (slot >= 0) { /* repeated key in this call: keep the first insertion */
      out[i] = m->vals[slot];
    } else {
      idmap_put_new(m, ids[i], new_index[k]);
      out[i] = new_index[k];
    }
  }
  free(miss_pos);
  free(new_index);
}

ORACLE_API void oracle_idmap_lookup_readonly(const OracleIdMap* m, const int64_t* ids,
                                             int64_t n, int64_t* out) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    int64_t slot = idmap_find_slot(m, ids[i]);
    out[i] = slot >= 0 ? m->vals[slot] : -1;
  }
}

ORACLE_API void oracle_idmap_delete(OracleIdMap* m, const int64_t* ids, const int64_t* index,
                                    int64_t n) {
  if (n == 0) return;
  for (int64_t i = 0; i < n; ++i) {
    int64_t slot = idmap_find_slot(m, ids[i]);
    if (slot >= 0) {
      m->state[slot] = 2;
      m->size--;
    }
  }
  alloc_free(&m->alloc, index, n);
}

ORACLE_API int64_t oracle_idmap_size(const OracleIdMap* m) { return m->size; }
/* IdMap::GetIdNum = allocator high-water mark, csrc/embedding/id_map.h:29 */
ORACLE_API int64_t oracle_idmap_id_num(const OracleIdMap* m) { return m->alloc.cur_size; }
ORACLE_API int64_t oracle_idmap_free_size(const OracleIdMap* m) { return m->alloc.free_size; }

ORACLE_API int64_t oracle_idmap_snapshot(const OracleIdMap* m, int64_t* ids, int64_t* index) {
  int64_t k = 0;
  for (int64_t i = 0; i < m->cap; ++i) {
    if (m->state[i] == 1) {
      ids[k] = m->keys[i];
      index[k] = m->vals[i];
      ++k;
    }
  }
  return k;
}

ORACLE_API void oracle_idmap_clear(OracleIdMap* m) {
  memset(m->state, 0, (size_t)m->cap);
  m->size = m->used = 0;
  m->alloc.cur_size = 0;
  m->alloc.free_size = 0;
}

/* ------------------------------------------------------------------------- *
 * Row storage in blocks.
 * csrc/ops/block_ops.cc:7-52 (gather), :31-98 (block gather, read-only zero
 * fill for the default key), :100-133 (insert, 1-row broadcast), :135-165
 * (masked insert), :223-260 (filter: slot value < threshold).
 * `blocks` is an array of pointers to [block_size, D] arrays; esize = element
 * size in bytes (rows are moved with memcpy, as in the reference).
 * ------------------------------------------------------------------------- */
ORACLE_API void oracle_gather(const int64_t* ids, int64_t n, const void* emb, void* out,
                              int64_t D, int64_t esize) {
  size_t row = (size_t)(D * esize);
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i)
    memcpy((char*)out + (size_t)i * row, (const char*)emb + (size_t)ids[i] * row, row);
}

ORACLE_API void oracle_block_gather(const int64_t* ids, int64_t n, void* const* blocks,
                                    int64_t block_size, int64_t default_key, int readonly,
                                    void* out, int64_t D, int64_t esize) {
  size_t row = (size_t)(D * esize);
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    int64_t src = ids[i];
    if (readonly && src == default_key) {
      memset((char*)out + (size_t)i * row, 0, row);
      continue;
    }
    memcpy((char*)out + (size_t)i * row,
           (const char*)blocks[src / block_size] + (size_t)(src % block_size) * row, row);
  }
}

ORACLE_API void oracle_block_insert(const int64_t* ids, int64_t n, const void* emb,
                                    int broadcast, const uint8_t* mask, void* const* blocks,
                                    int64_t block_size, int64_t D, int64_t esize) {
  size_t row = (size_t)(D * esize);
  /* sequential: with duplicate ids the last writer must win deterministically */
  for (int64_t i = 0; i < n; ++i) {
    if (mask && !mask[i]) continue;
    int64_t dst = ids[i];
    memcpy((char*)blocks[dst / block_size] + (size_t)(dst % block_size) * row,
           (const char*)emb + (broadcast ? 0 : (size_t)i * row), row);
  }
}

ORACLE_API void oracle_block_filter(const int64_t* ids, int64_t n, void* const* blocks,
                                    int64_t block_size, int64_t threshold, int slot_is64,
                                    uint8_t* mask_out) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    int64_t idx = ids[i];
    int64_t v = slot_is64 ? ((const int64_t*)blocks[idx / block_size])[idx % block_size]
                          : (int64_t)((const int32_t*)blocks[idx / block_size])[idx % block_size];
    mask_out[i] = v < threshold;
  }
}

/* ------------------------------------------------------------------------- *
 * Sparse optimizers.
 * cal_alpha_cpu_kernel + BlocksApplyAdamwTFFunctor,
 * csrc/ops/block_apply_adamw_op.cc:9-93: once per call
 *   b1_t *= beta1; b2_t *= beta2; alpha = -lr / (1 - b1_t) * sqrtf(1 - b2_t)
 * (in the dtype of the beta tensors: double for SparseAdam, float for
 * SparseAdamW / SparseAdamWTF, csrc/embedding/adam.h:37, adamw.h:36), then per
 * element, with double products rounded to float at every assignment:
 *   w = w * decay; m = m*beta1 + g*(1-beta1); v = v*beta2 + (1-beta2)*g*g;
 *   w += alpha * (m / (sqrtf(v) + eps))
 * ------------------------------------------------------------------------- */
ORACLE_API double oracle_cal_alpha_f64(double* b1_t, double* b2_t, double lr, double beta1,
                                       double beta2) {
  b1_t[0] *= beta1;
  b2_t[0] *= beta2;
  double bc1 = 1 - b1_t[0];
  double bc2 = 1 - b2_t[0];
  return -lr / bc1 * sqrtf((float)bc2);
}

ORACLE_API float oracle_cal_alpha_f32(float* b1_t, float* b2_t, double lr, double beta1,
                                      double beta2) {
  b1_t[0] = (float)(b1_t[0] * beta1);
  b2_t[0] = (float)(b2_t[0] * beta2);
  float bc1 = 1 - b1_t[0];
  float bc2 = 1 - b2_t[0];
  return (float)(-lr / bc1 * sqrtf(bc2));
}

ORACLE_API void oracle_block_apply_adamw(const int64_t* index, int64_t n, const float* grad,
                                         float* const* emb_blocks, float* const* exp_avg,
                                         float* const* exp_avg_sq, double alpha, double beta1,
                                         double beta2, double weight_decay, double eps,
                                         int64_t block_size, int64_t D) {
  const double omb1 = 1 - beta1, omb2 = 1 - beta2;
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    int64_t idx = index[i];
    int64_t off = (idx % block_size) * D;
    float* w = emb_blocks[idx / block_size] + off;
    float* m = exp_avg[idx / block_size] + off;
    float* v = exp_avg_sq[idx / block_size] + off;
    const float* g = grad + i * D;
    for (int64_t d = 0; d < D; ++d) {
      w[d] = (float)(w[d] * weight_decay);
      float ge = g[d];
      m[d] = (float)(m[d] * beta1 + ge * omb1);
      v[d] = (float)(v[d] * beta2 + omb2 * ge * ge);
      w[d] = (float)(w[d] + alpha * (m[d] / (sqrtf(v[d]) + eps)));
    }
  }
}

/* Sparse Adagrad row update (no reference counterpart; textbook Adagrad as in
 * torch.optim.Adagrad with lr_decay = 0, weight_decay = 0, applied only to the
 * rows that received a gradient):  s += g*g;  w -= lr * g / (sqrt(s) + eps).
 * Arithmetic in float, like torch's fp32 kernel. */
ORACLE_API void oracle_block_apply_adagrad(const int64_t* index, int64_t n, const float* grad,
                                           float* const* emb_blocks, float* const* accum,
                                           float lr, float eps, int64_t block_size,
                                           int64_t D) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    int64_t idx = index[i];
    int64_t off = (idx % block_size) * D;
    float* w = emb_blocks[idx / block_size] + off;
    float* s = accum[idx / block_size] + off;
    const float* g = grad + i * D;
    for (int64_t d = 0; d < D; ++d) {
      s[d] = s[d] + g[d] * g[d];
      w[d] = w[d] - lr * (g[d] / (sqrtf(s[d]) + eps));
    }
  }
}

/* ------------------------------------------------------------------------- *
 * Key tagging and dedup.
 * ids_encode, csrc/ops/ids_encode.cc:5-22 / ids_encode_kernel.cu:16-20:
 *   out = (id & (2^52 - 1)) + (table_id << 52), inputs concatenated.
 * ------------------------------------------------------------------------- */
ORACLE_API void oracle_ids_encode(const int64_t* ids, int64_t n, int64_t table_id,
                                  int64_t* out) {
  const int64_t mask = ((int64_t)1 << 52) - 1;
  for (int64_t i = 0; i < n; ++i)
    out[i] = (ids[i] & mask) + (int64_t)((uint64_t)table_id << 52);
}

/* Order used by the device dedup, csrc/ops/ids_partition_kernel.cu:36-43,95-131:
 * unique ids ascending by rotr64(id, 16) compared as unsigned, inverse int32.
 * Returns the number of unique ids. part_counts[p] = how many unique ids fall
 * in shard p (HashSlice, :45-55: slot = id & 0xFFFF split into num_parts
 * contiguous ranges, the first 65536 % num_parts ranges one longer). */
typedef struct {
  uint64_t key;
  int64_t pos;
} KeyPos;

static int cmp_keypos(const void* a, const void* b) {
  const KeyPos* x = (const KeyPos*)a;
  const KeyPos* y = (const KeyPos*)b;
  if (x->key != y->key) return x->key < y->key ? -1 : 1;
  return x->pos < y->pos ? -1 : (x->pos > y->pos);
}

static int hash_slice(int64_t id, int num_parts) {
  int part_size = 65536 / num_parts, extra = 65536 % num_parts;
  int cur = (int)(id & 0xFFFF);
  int a = cur / (part_size + 1);
  int b = (cur - extra) / part_size;
  return a > b ? a : b;
}

ORACLE_API int64_t oracle_ids_partition(const int64_t* ids, int64_t n, int num_parts,
                                        int64_t* unique_out, int64_t* part_counts,
                                        int32_t* inverse) {
  KeyPos* kp = (KeyPos*)malloc(sizeof(KeyPos) * (size_t)(n > 0 ? n : 1));
  for (int64_t i = 0; i < n; ++i) {
    uint64_t x = (uint64_t)ids[i];
    kp[i].key = (x << 48) | (x >> 16);
    kp[i].pos = i;
  }
  qsort(kp, (size_t)n, sizeof(KeyPos), cmp_keypos);
  for (int p = 0; p < num_parts; ++p) part_counts[p] = 0;
  int64_t u = -1;
  for (int64_t i = 0; i < n; ++i) {
    if (i == 0 || kp[i].key != kp[i - 1].key) {
      ++u;
      unique_out[u] = ids[kp[i].pos];
      part_counts[hash_slice(unique_out[u], num_parts)]++;
    }
    inverse[kp[i].pos] = (int32_t)u;
  }
  free(kp);
  return u + 1;
}

/* ------------------------------------------------------------------------- *
 * Feature-engine scalar ops.
 * uint64 mod: csrc/ops/uint64_mod.cc:4-10, fused_uint64_mod.cc:5-7
 * bucketize:  csrc/ops/fused_bucketized.cc:5-20 (branch !(v < b[mid]) -> count
 *             of boundaries <= v, NaN -> len); bucketize_op.cc:10-13 upper_bound
 * multi hash: csrc/ops/multi_hash.cc:18-26, signed int64 with C %
 * ------------------------------------------------------------------------- */
ORACLE_API void oracle_uint64_mod(const int64_t* x, int64_t n, int64_t mod, int64_t* out) {
  for (int64_t i = 0; i < n; ++i) out[i] = (int64_t)((uint64_t)x[i] % (uint64_t)mod);
}

ORACLE_API void oracle_bucketize(const float* v, int64_t n, const float* b, int32_t blen,
                                 int64_t* out) {
  for (int64_t i = 0; i < n; ++i) {
    int32_t bucket = 0, count = blen;
    while (count > 0) {
      int32_t step = count / 2;
      int32_t left = bucket + step;
      if (!(v[i] < b[left])) {
        bucket = left + 1;
        count -= step + 1;
      } else {
        count = step;
      }
    }
    out[i] = bucket;
  }
}

ORACLE_API void oracle_multi_hash(const int64_t* x, int64_t n, int64_t mul, int64_t prime,
                                  int64_t bucket, int64_t* out) {
  for (int64_t i = 0; i < n; ++i) {
    int64_t t = (int64_t)((uint64_t)x[i] * (uint64_t)mul); /* wraps like the reference */
    out[i] = (((t % prime) + prime) % prime) % bucket;
  }
}

/* ------------------------------------------------------------------------- *
 * String hashes, csrc/ops/fused_hash_kernel.cu:55-97 (MurmurHash64A, seed 0)
 * and :164-369 (FarmHash na::Hash64). Both are published algorithms; written
 * here from their definitions with little-endian unaligned loads.
 * ------------------------------------------------------------------------- */
static uint64_t rd64(const uint8_t* p) {
  uint64_t v;
  memcpy(&v, p, 8);
  return v;
}
static uint32_t rd32(const uint8_t* p) {
  uint32_t v;
  memcpy(&v, p, 4);
  return v;
}

ORACLE_API uint64_t oracle_murmur64(const uint8_t* data, uint64_t n, uint64_t seed) {
  const uint64_t m = 0xc6a4a7935bd1e995ULL;
  uint64_t h = seed ^ (n * m);
  uint64_t full = n / 8;
  for (uint64_t i = 0; i < full; ++i) {
    uint64_t k = rd64(data + 8 * i) * m;
    k ^= k >> 47;
    h = (h ^ (k * m)) * m;
  }
  const uint8_t* tail = data + 8 * full;
  uint64_t rem = n & 7;
  if (rem) {
    for (uint64_t i = rem; i-- > 0;) h ^= (uint64_t)tail[i] << (8 * i);
    h *= m;
  }
  h ^= h >> 47;
  h *= m;
  h ^= h >> 47;
  return h;
}

#define FK0 0xc3a5c85c97cb3127ULL
#define FK1 0xb492b66fbe98f273ULL
#define FK2 0x9ae16a3b2f90404fULL

static uint64_t rotr(uint64_t v, int s) { return s == 0 ? v : (v >> s) | (v << (64 - s)); }
static uint64_t smix(uint64_t v) { return v ^ (v >> 47); }

static uint64_t hlen16(uint64_t u, uint64_t v, uint64_t mul) {
  uint64_t a = (u ^ v) * mul;
  a ^= a >> 47;
  uint64_t b = (v ^ a) * mul;
  b ^= b >> 47;
  return b * mul;
}

typedef struct {
  uint64_t lo, hi;
} U128;

static U128 weak32(uint64_t w, uint64_t x, uint64_t y, uint64_t z, uint64_t a, uint64_t b) {
  a += w;
  b = rotr(b + a + z, 21);
  uint64_t c = a;
  a += x + y;
  b += rotr(a, 44);
  U128 r = {a + z, b + c};
  return r;
}

static U128 weak32p(const uint8_t* s, uint64_t a, uint64_t b) {
  return weak32(rd64(s), rd64(s + 8), rd64(s + 16), rd64(s + 24), a, b);
}

ORACLE_API uint64_t oracle_farmhash64(const uint8_t* s, uint64_t len) {
  if (len <= 16) {
    if (len >= 8) {
      uint64_t mul = FK2 + len * 2, a = rd64(s) + FK2, b = rd64(s + len - 8);
      return hlen16(rotr(b, 37) * mul + a, (rotr(a, 25) + b) * mul, mul);
    }
    if (len >= 4) {
      uint64_t mul = FK2 + len * 2, a = rd32(s);
      return hlen16(len + (a << 3), rd32(s + len - 4), mul);
    }
    if (len > 0) {
      uint32_t y = (uint32_t)s[0] + ((uint32_t)s[len >> 1] << 8);
      uint32_t z = (uint32_t)len + ((uint32_t)s[len - 1] << 2);
      return smix(y * FK2 ^ z * FK0) * FK2;
    }
    return FK2;
  }
  if (len <= 32) {
    uint64_t mul = FK2 + len * 2;
    uint64_t a = rd64(s) * FK1, b = rd64(s + 8);
    uint64_t c = rd64(s + len - 8) * mul, d = rd64(s + len - 16) * FK2;
    return hlen16(rotr(a + b, 43) + rotr(c, 30) + d, a + rotr(b + FK2, 18) + c, mul);
  }
  if (len <= 64) {
    uint64_t mul = FK2 + len * 2;
    uint64_t a = rd64(s) * FK2, b = rd64(s + 8);
    uint64_t c = rd64(s + len - 8) * mul, d = rd64(s + len - 16) * FK2;
    uint64_t y = rotr(a + b, 43) + rotr(c, 30) + d;
    uint64_t z = hlen16(y, a + rotr(b + FK2, 18) + c, mul);
    uint64_t e = rd64(s + 16) * mul, f = rd64(s + 24);
    uint64_t g = (y + rd64(s + len - 32)) * mul, h = (z + rd64(s + len - 24)) * mul;
    return hlen16(rotr(e + f, 43) + rotr(g, 30) + h, e + rotr(f + a, 18) + g, mul);
  }
  const uint64_t seed = 81;
  uint64_t x = seed, y = seed * FK1 + 113, z = smix(y * FK2 + 113) * FK2;
  U128 v = {0, 0}, w = {0, 0};
  x = x * FK2 + rd64(s);
  const uint8_t* end = s + ((len - 1) / 64) * 64;
  const uint8_t* last64 = end + ((len - 1) & 63) - 63;
  do {
    x = rotr(x + y + v.lo + rd64(s + 8), 37) * FK1;
    y = rotr(y + v.hi + rd64(s + 48), 42) * FK1;
    x ^= w.hi;
    y += v.lo + rd64(s + 40);
    z = rotr(z + w.lo, 33) * FK1;
    v = weak32p(s, v.hi * FK1, x + w.lo);
    w = weak32p(s + 32, z + w.hi, y + rd64(s + 16));
    uint64_t t = z; z = x; x = t;
    s += 64;
  } while (s != end);
  uint64_t mul = FK1 + ((z & 0xff) << 1);
  s = last64;
  w.lo += (len - 1) & 63;
  v.lo += w.lo;
  w.lo += v.lo;
  x = rotr(x + y + v.lo + rd64(s + 8), 37) * mul;
  y = rotr(y + v.hi + rd64(s + 48), 42) * mul;
  x ^= w.hi * 9;
  y += v.lo * 9 + rd64(s + 40);
  z = rotr(z + w.lo, 33) * mul;
  v = weak32p(s, v.hi * mul, x + w.lo);
  w = weak32p(s + 32, z + w.hi, y + rd64(s + 16));
  uint64_t t = z; z = x; x = t;
  return hlen16(hlen16(v.lo, w.lo, mul) + smix(y) * FK0 + z, hlen16(v.hi, w.hi, mul) + x, mul);
}

/* fused_hash: strings are values[off[i] .. off[i+1]) ; kind 0 farm, 1 murmur */
ORACLE_API void oracle_hash_strings(const int8_t* values, const int64_t* offsets, int64_t n,
                                    int kind, int64_t* out) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    const uint8_t* s = (const uint8_t*)values + offsets[i];
    uint64_t len = (uint64_t)(offsets[i + 1] - offsets[i]);
    out[i] = (int64_t)(kind == 0 ? oracle_farmhash64(s, len) : oracle_murmur64(s, len, 0));
  }
}
