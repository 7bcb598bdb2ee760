/*
 * recis_hip.h - C ABI of librecis_hip.so: the gfx950 (MI355X) implementation of
 * RecIS's sparse-embedding hot path.
 *
 * Every entry point takes plain device pointers and sizes (no torch types) and
 * an opaque `stream` (a hipStream_t; NULL = the legacy default stream). Unless
 * stated otherwise a call only enqueues work on that stream and returns; it
 * never synchronises the device. All functions return RECIS_OK (0) or an error
 * code, with a human-readable message available from recis_hip_last_error().
 *
 * Each declaration names the reference function it stands in for
 * (paths relative to the alibaba/RecIS tree). The reference dispatches on
 * `tensor.device().is_cuda()` inside each op; these are the device branches.
 */
#ifndef RECIS_HIP_H_
#define RECIS_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RECIS_HIP_ABI_VERSION 2

/* status codes */
#define RECIS_OK 0
#define RECIS_ERR_ARG 1      /* bad argument (shape, dtype, alignment, NULL)  */
#define RECIS_ERR_HIP 2      /* a HIP runtime call failed                     */
#define RECIS_ERR_STATE 3    /* object used in a state that does not allow it */
#define RECIS_ERR_CAPACITY 4 /* a fixed capacity would be exceeded            */

/* element types of row storage / gradients */
#define RECIS_F32 0
#define RECIS_BF16 1
#define RECIS_F16 2
#define RECIS_F64 3 /* rows and gradients of recis_block_apply_adamw only */

/* combiners (csrc/ops/embedding_segment_reduce.h:8 has SUM, MEAN, TILE; MAX is
 * an addition with no reference counterpart) */
#define RECIS_SUM 0
#define RECIS_MEAN 1
#define RECIS_TILE 2
#define RECIS_MAX 3

/* flags */
/* batch plan: unique ids with more than HOT_LEN occurrences are reduced by whole workgroups,
 * one (row, chunk of HOT_CHUNK occurrences) work item each */
#define RECIS_PLAN_HOT_LEN 64
#define RECIS_PLAN_HOT_CHUNK 2048

#define RECIS_PLAN_STAGE_COUNT 1

#define RECIS_FLAG_REV_UNIQUE 1 /* caller guarantees reverse_indices has no duplicates */

/* bits of the device-side soft-error word (recis_hip_poll_device_errors) */
#define RECIS_DEVERR_INDEX_RANGE 1  /* an index fell outside [0, rows)        */
#define RECIS_DEVERR_OFFSETS 2      /* offsets not monotone / outside [0, B]  */
#define RECIS_DEVERR_TABLE_FULL 4   /* id-map probe sequence found no slot    */
#define RECIS_DEVERR_PLAN_OVERFLOW 8 /* batch plan: too many distinct ids fell into one hash bucket */

const char* recis_hip_last_error(void);
int recis_hip_abi_version(void);

/*
 * Optional per-kernel timing for benchmarks (off by default). When on, the heavy kernels
 * of every entry point are bracketed by HIP events on their launch stream;
 * recis_hip_profile_report synchronises the device, writes one line
 * "kernel_name calls total_ms" per kernel into buf and resets the record.
 */
int recis_hip_profile_enable(int on);
int recis_hip_profile_report(char* buf, int64_t cap);

/*
 * Measurement support, no reference counterpart: n rows of row_bytes (a power of two, 16..1024;
 * 16 bytes per lane) of `table` (rows of that width back to back, `rows` of them) at the places
 * idx[0..n), read (write == 0: nothing is written; `sink`, 16 KB of device memory, only keeps the
 * loads alive) or overwritten with a pattern (write != 0), rows_in_flight (1, 2 or 4) rows per
 * lane group at a time. With random idx it shows how many rows per second the device serves when
 * every row is somewhere else, which is what the row kernels of the training step are held
 * against (bench.py --workload probe).
 */
int recis_hip_probe_random_rows(void* table, int64_t rows, int64_t row_bytes, const int32_t* idx,
                                int64_t n, int rows_in_flight, int write, void* sink, void* stream);

/* Synchronises the current device, returns the soft-error bits raised by
 * kernels since the last poll in *bits and clears them. */
int recis_hip_poll_device_errors(int* bits);

/* ------------------------------------------------------------------------- *
 * Pooling: ragged gather + segment reduce
 * ------------------------------------------------------------------------- */

/*
 * Forward of the ragged-mode pooling.
 * Replaces: segment_reduce_forward, csrc/ops/embedding_segment_reduce_kernel.cu:199-273
 *           (kernel :23-75).
 *   unique_emb       [U, D]  rows, emb_dtype
 *   weight           [B] per-occurrence weight (weight_dtype) or NULL (= 1)
 *   reverse_indices  [B] occurrence -> row of unique_emb (int32 or int64);
 *                    NULL means the identity (rows are already materialised
 *                    per occurrence, U == B)
 *   offsets          [S + 1] segment boundaries into the B occurrences
 *   out              SUM/MEAN/MAX: [S, D];  TILE: [B, D]   (out_dtype)
 *   argmax_out       MAX only: [S, D] int32, occurrence index (absolute, into
 *                    the B occurrences) of the winning row, -1 for an empty
 *                    segment; may be NULL when no backward is needed
 * SUM:  out[s] = sum_i w_i * emb[rev_i];  MEAN: the same divided by the segment
 * length (weights are not normalised); TILE: out[i] = w_i * emb[rev_i];
 * MAX: element-wise maximum of emb[rev_i] over the segment (weights ignored,
 * first occurrence wins ties, empty segment -> 0).
 * The output is fully written by the call (no pre-zeroing needed).
 */
int recis_segment_reduce_forward(const void* unique_emb, int emb_dtype,
                                 const void* weight, int weight_dtype,
                                 const void* reverse_indices, int rev_is64,
                                 const void* offsets, int off_is64, void* out,
                                 int out_dtype, int32_t* argmax_out, int64_t B,
                                 int64_t U, int64_t S, int64_t D, int mode,
                                 void* stream);

/*
 * The same forward with the unique rows read where the table keeps them instead of a dense
 * [U, D] copy: row u is row row_index[u] (the id map's answer for unique id u; negative = key
 * absent, reads as zeros) of the block list emb_blocks_dev (device array of n_blocks pointers,
 * 16-byte aligned blocks of block_rows rows). Fuses block_gather
 * (csrc/ops/block_ops.cc:281-290) into segment_reduce_forward
 * (csrc/ops/embedding_segment_reduce_kernel.cu:199-273): the [U, D] intermediate of
 * recis/nn/modules/embedding.py:592-624 (emb_reduce) is neither written nor read. SUM, MEAN and TILE.
 */
int recis_segment_reduce_forward_blocks(const void* const* emb_blocks_dev, int64_t n_blocks,
                                        int64_t block_rows, int64_t row_pitch_bytes,
                                        const int64_t* row_index, int emb_dtype,
                                        const void* weight, int weight_dtype,
                                        const void* reverse_indices, int rev_is64,
                                        const void* offsets, int off_is64, void* out, int out_dtype,
                                        int64_t B, int64_t U, int64_t S, int64_t D, int mode,
                                        void* stream);

/*
 * Backward of the ragged-mode pooling: scatters the pooled gradient back to the
 * unique rows.
 * Replaces: segment_reduce_backward, csrc/ops/embedding_segment_reduce_kernel.cu:276-350
 *           (kernel :79-120).
 *   grad_out     SUM/MEAN/MAX: [S, D]; TILE: [B, D]   (grad_dtype)
 *   argmax       MAX only: what the forward wrote
 *   grad_unique  [U, D] (out_dtype); fully written by the call
 * Without RECIS_FLAG_REV_UNIQUE duplicates in reverse_indices are accumulated
 * with fp32 atomics and out_dtype must be RECIS_F32. With the flag (or
 * reverse_indices == NULL) every row is written by plain stores.
 */
int recis_segment_reduce_backward(const void* grad_out, int grad_dtype,
                                  const void* weight, int weight_dtype,
                                  const void* reverse_indices, int rev_is64,
                                  const void* offsets, int off_is64,
                                  const int32_t* argmax, void* grad_unique,
                                  int out_dtype, int64_t B, int64_t U, int64_t S,
                                  int64_t D, int mode, int flags, void* stream);

/*
 * Sparse-mode pooling (short segments addressed by segment id).
 * Replaces: segment_sum_cuda / segment_mean_cuda, csrc/ops/segment_ops_kernel.cu:192-291
 *           (ops csrc/ops/segment_ops.cc:6-52).
 *   segment_sum:  out[seg[i]] += data[indices[i]] * w[i]; out [num_segments, D] fp32,
 *                 zeroed by the call. use_weight == 0 broadcasts weight[0]
 *                 (weight == NULL means 1).
 *   segment_mean_weight: weight_sum[s] = sum of w_i with seg_i == s;
 *                 weight_norm[i] = w_i / weight_sum[seg_i]; an out-of-range
 *                 segment id keeps the raw weight.
 */
int recis_segment_sum(const void* data, int dtype, int64_t data_rows, const void* weight,
                      int weight_dtype, int use_weight, const void* indices,
                      const void* segment_ids, int idx_is64, float* out, int64_t n,
                      int64_t num_segments, int64_t D, void* stream);
int recis_segment_mean_weight(const float* weight, int use_weight, const void* segment_ids,
                              int idx_is64, float* weight_sum, float* weight_norm, int64_t n,
                              int64_t num_segments, void* stream);

/*
 * out[j] = s with offsets[s] <= j < offsets[s+1], for j in [0, total); out has the
 * integer type of offsets. `total` = offsets[S] is supplied by the caller.
 * Replaces: gen_segment_indices_by_offset, csrc/ops/embedding_segment_reduce_kernel.cu:395-423.
 */
int recis_gen_segment_indices(const void* offsets, int off_is64, int64_t S, void* out,
                              int64_t total, void* stream);

/*
 * Unpooled gather padded / truncated to seq[f] rows per sample, several features
 * per call; weights play no part.
 * Replaces: ragged_tile / ragged_tile_back, csrc/ops/ragged_tile_kernel.cu:214-280.
 *   batch, seq     host arrays [n_features]
 *   value          [n_values] row of `table` per occurrence (int32/int64)
 *   offset         [sum(batch) + 1] merged sample boundaries into value
 *   table          [table_rows, D];  out [sum(batch*seq), D]   (dtype)
 *   backward: dy [sum(batch*seq), D] (dtype) -> d_table [table_rows, D] fp32,
 *   zeroed and accumulated (fp32 atomics) by the call.
 */
int recis_ragged_tile(const int64_t* batch, const int64_t* seq, int64_t n_features,
                      const void* value, int value_is64, int64_t n_values, const void* offset,
                      int off_is64, const void* table, int64_t table_rows, int dtype, void* out,
                      int64_t D, void* stream);
int recis_ragged_tile_back(const int64_t* batch, const int64_t* seq, int64_t n_features,
                           const void* value, int value_is64, int64_t n_values,
                           const void* offset, int off_is64, const void* dy, int dtype,
                           float* d_table, int64_t table_rows, int64_t D, void* stream);

/* ------------------------------------------------------------------------- *
 * IDMap: 64-bit key -> row index, with the row-index allocator
 * ------------------------------------------------------------------------- */

/*
 * Opaque device-resident map. Replaces GpuIdMap (csrc/embedding/gpu_id_map.h:9-33,
 * gpu_id_map.cu:9-121) together with its cuco::dynamic_map and its IdAllocator
 * (csrc/embedding/id_allocator.cc:8-64). Keys -1 and -2 are reserved, as in the
 * reference (gpu_id_map.h:11-16). An object belongs to the device that was
 * current at creation and must be used from one stream at a time.
 */
typedef struct recis_idmap recis_idmap;

/* reserve_keys: number of keys the table should hold without a rebuild. */
int recis_idmap_create(int64_t reserve_keys, recis_idmap** out);
int recis_idmap_destroy(recis_idmap* m);

/*
 * Find-or-insert (GpuIdMap::Lookup, gpu_id_map.cu:19-45). index_out[i] = row of
 * ids[i]; keys not present are inserted and take row indices in input order by
 * the rule of IdAllocator::GenIds (csrc/ops/hashtable_ops.cc:15-27): with n
 * missing keys, the k-th takes free_list[free - n + k] if that position is >= 0,
 * else the fresh index cur - (free - n + k + 1). A key repeated inside one call
 * gets one row; which of its occurrences stands for it in the ranking of the missing keys is
 * not specified, so with duplicate NEW keys in one call the rows of those keys may come out
 * permuted from run to run (callers on the hot path dedup first and never see this).
 * No host synchronisation unless the table must be rebuilt.
 */
int recis_idmap_lookup(recis_idmap* m, const int64_t* ids, int64_t n, int64_t* index_out,
                       void* stream);
/* recis_idmap_lookup for a batch whose size is still on the device (the unique ids of a batch
 * plan whose count the host has not read yet): the first min(*n_dev, n_max) ids are looked up,
 * index_out[i] for i beyond them is left untouched. Lets the host queue the lookup behind the
 * plan and fetch the count while both run. No counterpart in the reference (its
 * GpuIdMap::Lookup sizes everything on the host, gpu_id_map.cu:19-45). */
int recis_idmap_lookup_counted(recis_idmap* m, const int64_t* ids, int64_t n_max,
                               const int64_t* n_dev, int64_t* index_out, void* stream);
/* Tells the map the true size of the last recis_idmap_lookup_counted once the host knows it,
 * so that the bounds below stop counting all n_max ids of that call as possible new keys. */
int recis_idmap_settle_count(recis_idmap* m, int64_t n_true);
/* The same for callers with several counted lookups outstanding on one map (two embedding modules
 * that share a table): recis_idmap_last_call gives the number of the call just queued on the map,
 * recis_idmap_settle_call settles that call, whichever calls followed it. */
int recis_idmap_last_call(recis_idmap* m, int64_t* seq);
int recis_idmap_settle_call(recis_idmap* m, int64_t seq, int64_t n_true);
/* Upper bounds, without waiting for any stream, of the allocator's high-water mark
 * (IdMap::GetIdNum, id_map.h:29) and of the occupied table slots: the values the last finished
 * call published to pinned host memory plus every id of the calls queued since. Either
 * pointer may be NULL. For callers that size row storage ahead of the device. */
int recis_idmap_bounds(recis_idmap* m, int64_t* id_num_ub, int64_t* occupied_ub);
/* GpuIdMap::LookupReadOnly (gpu_id_map.cu:47-62): -1 for a missing key. */
int recis_idmap_lookup_readonly(recis_idmap* m, const int64_t* ids, int64_t n,
                                int64_t* index_out, void* stream);
/* GpuIdMap::DeleteIds (gpu_id_map.cu:84-96): erases ids, appends `index` (all n
 * entries, in order) to the free list (IdAllocator::FreeIds). */
int recis_idmap_erase(recis_idmap* m, const int64_t* ids, const int64_t* index, int64_t n,
                      void* stream);
/* Synchronises `stream`. live = keys present, id_num = allocator high-water mark
 * (IdMap::GetIdNum, id_map.h:29), free_size = free-list length. Any may be NULL. */
int recis_idmap_stats(recis_idmap* m, int64_t* live, int64_t* id_num, int64_t* free_size,
                      int64_t* capacity, void* stream);
/* GpuIdMap::SnapShot (gpu_id_map.cu:64-77): all live (key, row) pairs, unordered.
 * Synchronises; *count = number of live pairs (only min(count, max_out) written). */
int recis_idmap_snapshot(recis_idmap* m, int64_t* ids_out, int64_t* index_out, int64_t max_out,
                         int64_t* count, void* stream);
/* The eviction sweep of a step filter in one pass over the table. Replaces the sequence
 * IdMap::SnapShot + block_filter + masked_select + DeleteIds of
 * recis/nn/modules/hashtable_hook_impl.py:487-551 (do_filter / filter) and hashtable.cc:263-278:
 * every live key whose row has stamp < threshold (stamp slot: int32 or int64, one value per row,
 * blocks of block_rows rows, pointer table on the device) is erased and its row appended to the
 * free list; the evicted (key, row) pairs are written to ids_out / index_out (unordered) for the
 * caller to re-initialise the rows. At most max_out keys are evicted. Synchronises;
 * *count = number of evicted keys. */
int recis_idmap_evict_older(recis_idmap* m, const void* const* stamp_blocks_dev, int64_t n_blocks,
                            int64_t block_rows, int stamp_is64, int64_t threshold,
                            int64_t* ids_out, int64_t* index_out, int64_t max_out, int64_t* count,
                            void* stream);
/* GpuIdMap::Clear (gpu_id_map.cu:98-103). */
int recis_idmap_clear(recis_idmap* m, void* stream);
/* IdMap::Reserve (not implemented for the reference GPU map, gpu_id_map.cu:105-108). */
int recis_idmap_reserve(recis_idmap* m, int64_t n_keys, void* stream);

/*
 * Stand-alone allocator ops over a caller-held free list kept in blocks
 * (device array of block pointers).
 * Replace: generate_ids_cuda_op, free_ids_cuda_op, mask_key_index_cuda_op,
 * scatter_ids_with_mask_cuda_op, csrc/ops/hashtable_ops_kernel.cu:32-173.
 */
int recis_generate_ids(int64_t n, const int64_t* const* free_blocks_dev, int64_t free_count,
                       int64_t cur_count, int64_t free_block_size, int64_t* out, void* stream);
int recis_free_ids(const int64_t* ids, int64_t n, int64_t* const* free_blocks_dev,
                   int64_t free_count, int64_t free_block_size, void* stream);
int recis_mask_key_index(const int64_t* keys, const uint8_t* mask, const int64_t* cumsum,
                         int64_t n, int64_t out_size, int64_t* out_keys, int64_t* out_index,
                         void* stream);
int recis_scatter_ids_with_mask(int64_t* out_ids, int64_t out_size, const int64_t* in_ids,
                                const int64_t* mask_index, int64_t n, void* stream);

/* ------------------------------------------------------------------------- *
 * EmbeddingBlocks: rows stored as a list of equally sized blocks
 * ------------------------------------------------------------------------- */

/*
 * blocks_dev is a DEVICE array of n_blocks pointers to [block_size, row_bytes]
 * arrays; row `idx` lives in block idx / block_size at row idx % block_size.
 * Rows are moved as bytes, so any element type works. Block bases must be
 * aligned to the largest power of two (<= 16) that divides row_bytes.
 *
 * row_pitch_bytes, here and in every entry point below that takes a block list: the
 * distance from one row of a block to the next, 0 when rows lie back to back (the
 * reference's layout, one array per slot). A table that keeps a parameter row and its
 * optimizer state next to each other (w | m | v in one allocation, the pointer tables of
 * the three slots offset by one row width each) passes the combined width, so that one
 * key's rows share DRAM pages and cache lines. The pitch must be a multiple of the
 * element size and of the alignment above (recis_block_gather / recis_block_insert, which
 * move bytes, narrow their vector to what the pitch allows instead). Slots that share one
 * call share one pitch.
 *
 * Replace the device branches of csrc/ops/block_ops.cc:
 *   recis_gather             gather_cuda              (block_ops.cc:262-268)
 *   recis_block_gather       block_gather_cuda        (block_ops.cc:270-282, also
 *                            block_gather_by_range when ids is offset by `beg`)
 *   recis_block_insert       block_insert_cuda / block_insert_with_mask_cuda
 *                            (block_ops.cc:353-360, 385-397); broadcast = emb has
 *                            one row; mask may be NULL
 *   recis_block_filter       block_filter_cuda        (block_ops.cc:284-293):
 *                            mask_out[i] = slot[ids[i]] < threshold (int32/int64 slot)
 * readonly != 0: an index equal to default_key yields a zero row.
 */
int recis_gather(const void* ids, int ids_is64, const void* emb, int64_t rows, void* out,
                 int64_t n, int64_t row_bytes, void* stream);
int recis_block_gather(const int64_t* ids, void* const* blocks_dev, int64_t n_blocks,
                       int64_t block_size, int64_t row_pitch_bytes, int64_t default_key, int readonly, void* out,
                       int64_t n, int64_t row_bytes, void* stream);
int recis_block_insert(const int64_t* ids, const void* emb, int broadcast, const uint8_t* mask,
                       void* const* blocks_dev, int64_t n_blocks, int64_t block_size,
                       int64_t row_pitch_bytes, int64_t n, int64_t row_bytes, void* stream);
int recis_block_filter(const int64_t* ids, void* const* blocks_dev, int64_t n_blocks,
                       int64_t block_size, int64_t threshold, int slot_is64, uint8_t* mask_out,
                       int64_t n, void* stream);

/* ------------------------------------------------------------------------- *
 * Fused sparse optimizer row updates
 * ------------------------------------------------------------------------- */

/*
 * Replaces: block_apply_adamw, csrc/ops/block_apply_adamw_op.cc:114-132.
 * beta1_t / beta2_t: device scalars holding the running powers (float, or double
 * when beta_is_f64), advanced in place; alpha = -lr / (1 - b1_t) * sqrtf(1 - b2_t).
 * Per element of row index[i] (weight_decay is the multiplicative factor):
 *   w *= weight_decay; m = m*beta1 + g*(1-beta1); v = v*beta2 + (1-beta2)*g*g;
 *   w += alpha * (m / (sqrtf(v) + eps))
 * computed as the reference CPU functor does (double products, float sqrt, one
 * rounding per assignment; on 16-bit rows every assignment rounds double -> float ->
 * row type and the last line rounds the step to the row type before it is added, as
 * `Half += double` does in block_apply_adamw_op.cc:55-56). index must not contain duplicates.
 * Rows of RECIS_F64 take RECIS_F64 gradients (the functor's TEmb = double: nothing is rounded but
 * the argument of sqrtf); the other entry points know the three narrower types only.
 */
int recis_block_apply_adamw(const int64_t* index, const void* grad, int grad_dtype,
                            void* const* emb_blocks_dev, void* const* exp_avg_blocks_dev,
                            void* const* exp_avg_sq_blocks_dev, int64_t n_blocks,
                            int64_t block_size, int64_t row_pitch_bytes, int row_dtype,
                            void* beta1_t, void* beta2_t, int beta_is_f64, double lr, double beta1, double beta2,
                            double weight_decay, double eps, int64_t n, int64_t D, void* stream);

/*
 * Sparse Adagrad row update; no reference counterpart (RecIS ships only the Adam
 * family); follows the conventions of block_apply_adamw:
 *   s += g*g;  w -= lr * g / (sqrtf(s) + eps)      (float arithmetic)
 */
int recis_block_apply_adagrad(const int64_t* index, const void* grad, int grad_dtype,
                              void* const* emb_blocks_dev, void* const* accum_blocks_dev,
                              int64_t n_blocks, int64_t block_size, int64_t row_pitch_bytes,
                              int row_dtype, double lr, double eps, int64_t n, int64_t D,
                              void* stream);

/* ------------------------------------------------------------------------- *
 * Key tagging, offset merging, dedup
 * ------------------------------------------------------------------------- */

/*
 * Lists of tensors are passed as HOST arrays of device pointers and sizes.
 * recis_ids_encode   ids_encode_cuda, csrc/ops/ids_encode_kernel.cu:22-59:
 *                    out = concat_t ((ids_t & (2^52-1)) | (table_ids[t] << 52))
 * recis_merge_offsets  merge_offsets, csrc/ops/embedding_segment_reduce_kernel.cu:357-391:
 *                    tensor t contributes its first size_t - 1 entries (all of them
 *                    for the last tensor) plus sum_{u<t} max_values[u]
 */
int recis_ids_encode(const int64_t* const* ids_ptrs, const int64_t* sizes,
                     const int64_t* table_ids, int64_t n_tensors, int64_t* out, void* stream);
int recis_merge_offsets(const void* const* offsets_ptrs, const int64_t* sizes,
                        const int64_t* max_values, int64_t n_tensors, int is64, void* out,
                        void* stream);

/*
 * Dedup: unique ids (in order of first occurrence), inverse (int32 or int64) with
 * unique_out[inverse[i]] == ids[i], and the number of unique ids written to the
 * device word count_out_dev. unique_out must have room for n entries.
 * Replaces the unique half of ids_partition_cuda (csrc/ops/ids_partition_kernel.cu:86-131)
 * and the torch.unique of recis/nn/modules/hashtable.py:278; the reference orders
 * the unique ids by sort key instead (recis_partition_order below puts them in that
 * order).
 */
int recis_unique(const int64_t* ids, int64_t n, int64_t* unique_out, void* inverse_out,
                 int inverse_is64, int64_t* count_out_dev, void* stream);

/*
 * The ordering half of ids_partition_cuda (csrc/ops/ids_partition_kernel.cu:36-55, the sort by
 * PartitionKey): n ids without duplicates are put in ascending order of rotr64(id, 16) taken as
 * unsigned, which is by shard slot (id & 0xFFFF) first: the stable order of (key, position).
 * From 32768 ids up to some 8 million the keys are split into bins by their top bits and every bin is
 * put in order in LDS; the host waits once, early, for a word that says whether every bin fits (ids
 * whose shard slots are very unevenly spread do not). Those, and smaller and larger inputs, take a
 * library sort of (key, position) pairs. Both ways give the same result.
 *   sorted_ids [n]   the ids in that order
 *   order      [n]   order[k] = input position of sorted_ids[k]
 *   rank       [n]   rank[order[k]] = k (the sorted position of every input position)
 * n must fit 32 bits. Scratch comes from the stream's workspace. Waits for the stream (see above).
 */
int recis_partition_order(const int64_t* ids, int64_t n, int64_t* sorted_ids, int32_t* order,
                          int32_t* rank, void* stream);

/*
 * Batch plan: dedup plus the transposed index. Unique ids (no duplicates, every id of the
 * batch present), an int32 inverse with unique_out[inverse[i]] == ids[i], the count, and the
 * occurrences grouped by unique id:
 *   inverse_out   [n]      may be NULL when the caller does not need it
 *   row_start_out [n + 1]  list of unique id u = list[row_start[u] .. row_start[u+1]) for u < U;
 *                          row_start[U] = n; entries past U are not written
 *   list_out      [n]      occurrence indices grouped by unique id
 *   pos_out       [n]      position of occurrence i in list_out (may be NULL)
 *   hot_items_out [2*hot_cap] (row, chunk) work items for ids with more than RECIS_PLAN_HOT_LEN
 *                          occurrences; hot_cap >= n/HOT_LEN + n/HOT_CHUNK + 2, or 0 to skip
 *   counts_out_dev [2]     device words: number of unique ids, number of hot items
 *   unique_count_host      host word or NULL: when given, the call returns only once the number
 *                          of unique ids is known and stores it there
 *   flags                  RECIS_PLAN_STAGE_COUNT: send the count towards the host but do not
 *                          wait; recis_unique_plan_count(stream) fetches it later (one staged
 *                          count per stream: fetch it before the next plan on that stream)
 * The unique ids are ordered as follows: first the few ids that make up a sizeable share of the
 * batch (found by sampling; at most 64), then the ids of the hash buckets (a bucket = the top bits
 * of a 64-bit mix of the id) that hold more than one and a half times the average, then those of
 * the other buckets, buckets in the order of their index and, inside a bucket, ids by their place
 * in the bucket's hash table. The order, the inverse and row_start depend on the input only; the
 * order of the entries inside one id's list and of the hot items is not specified. Ids are partitioned by hash (a histogram and a scatter pass over the ids),
 * every bucket is deduplicated in LDS by one workgroup, and the workgroups learn where their
 * unique ids start from a look-back over one word per bucket: the only global atomics are one
 * ticket per bucket and one addition per hot id.
 * With the plan, a gradient scatter over duplicated ids (the atomic loops of
 * csrc/ops/embedding_segment_reduce_kernel.cu:79-120, segment_ops_kernel.cu:133-165,
 * ragged_tile_kernel.cu:46-60 and the unique + index_add_ of
 * recis/nn/modules/hashtable.py:555-586) becomes a gather-reduce per unique row.
 * No counterpart in the reference (its dedup is the radix sort of
 * csrc/ops/ids_partition_kernel.cu:86-131).
 */
int recis_unique_plan(const int64_t* ids, int64_t n, int64_t* unique_out, int32_t* inverse_out,
                      int32_t* row_start_out, int32_t* list_out, int32_t* pos_out,
                      int32_t* hot_items_out, int64_t hot_cap, int64_t* counts_out_dev,
                      int64_t* unique_count_host, int flags, void* stream);
/*
 * recis_unique_plan and the find-or-insert of its unique ids in an id map in one pass:
 * index_out [n] receives, for u < U, the row of unique id u, exactly as
 * recis_idmap_lookup(m, unique_out, U, index_out) would assign it (missing keys take rows in the
 * order of the unique ids). The workgroup that deduplicates a hash bucket probes the map for the
 * bucket's distinct ids while they are still in LDS (the bucket is a contiguous range of the
 * map's home slots), so the unique ids are not read back and the probe kernel, its scan and its
 * row-assignment pass over all ids (csrc/embedding/gpu_id_map.cu:19-45) shrink to one small
 * launch over the NEW keys. Replaces ids_partition + GpuIdMap::Lookup of
 * recis/nn/modules/hashtable.py:262-293. Keys -1 and -2 raise RECIS_DEVERR_INDEX_RANGE and get
 * row -1. The map's capacity is checked as for recis_idmap_lookup_counted with n ids.
 */
int recis_unique_plan_lookup(recis_idmap* m, const int64_t* ids, int64_t n, int64_t* unique_out,
                             int32_t* inverse_out, int32_t* row_start_out, int32_t* list_out,
                             int32_t* pos_out, int32_t* hot_items_out, int64_t hot_cap,
                             int64_t* counts_out_dev, int64_t* index_out, int64_t* unique_count_host,
                             int flags, void* stream);

/*
 * recis_unique_plan / recis_unique_plan_lookup (map != NULL) of a batch that is given as n_jobs
 * (1..64) arrays laid end to end: array k holds sizes[k] ids, and with table_ids != NULL every id
 * is tagged with its array's table on the way in, as recis_ids_encode does
 * (csrc/ops/ids_encode_kernel.cu:16-20; table_ids == NULL: the plain concatenation). The kernels
 * read the arrays directly, so the tagged batch that ids_encode would write and the plan read
 * back never exists; unique_out holds tagged ids, positions (inverse, lists) count along the
 * concatenation. ids_ptrs / sizes / table_ids are host arrays. Everything else as in
 * recis_unique_plan_lookup (index_out unused without a map).
 */
int recis_unique_plan_jobs(recis_idmap* map, const int64_t* const* ids_ptrs, const int64_t* sizes,
                           const int64_t* table_ids, int64_t n_jobs, int64_t* unique_out,
                           int32_t* inverse_out, int32_t* row_start_out, int32_t* list_out,
                           int32_t* pos_out, int32_t* hot_items_out, int64_t hot_cap,
                           int64_t* counts_out_dev, int64_t* index_out, int64_t* unique_count_host,
                           int flags, void* stream);
/* inverse_out [n] and / or pos_out [n] of a plan that was made without them (either may be NULL),
 * from its row_start, list and counts. No counterpart in the reference. */
int recis_plan_inverse_from_lists(const int32_t* row_start, const int32_t* list, const int64_t* counts_dev,
                                  int64_t n, int32_t* inverse_out, int32_t* pos_out, void* stream);
/* How many times a workgroup of the plan polls the look-back word of an earlier bucket before it
 * gives up, raises RECIS_DEVERR_PLAN_OVERFLOW and goes on with zero (default
 * RECIS_PLAN_SPIN_LIMIT_DEFAULT polls: about a second; a word is due within microseconds). A plan
 * whose wait gave up has a wrong unique base from that bucket on; the error bit is the only sign
 * of it, so callers that never fetch the staged count (which raises the bit) should poll
 * recis_hip_staged_device_errors / recis_hip_poll_device_errors now and then. For tests of that
 * path; the value applies to launches made after the call. */
#define RECIS_PLAN_SPIN_LIMIT_DEFAULT (1u << 22)
int recis_plan_set_spin_limit(int64_t polls);
int recis_plan_get_spin_limit(int64_t* polls);
/* Waits for the count staged by the last recis_unique_plan(…, RECIS_PLAN_STAGE_COUNT, stream). */
int recis_unique_plan_count(int64_t* unique_count_host, void* stream);
/* The soft-error bits (RECIS_DEVERR_*) that were set on the device when the last count of `stream`
 * was staged; read from host memory, never waits, clears nothing. Lets a caller that fetches the
 * staged count every step notice, one step late at most, what recis_hip_poll_device_errors would
 * report after a device-wide wait. */
int recis_hip_staged_device_errors(int* bits, void* stream);

/*
 * recis_unique_plan for callers that cannot allocate (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc). No counterpart in the reference. Same outputs as
 * recis_unique_plan for the same ids, bit for bit wherever that call specifies them (unique ids,
 * inverse, row_start, counts; list / pos up to the order inside one id's list); the count stays on
 * the device (counts_out_dev), nothing is staged for the host. The kernels' scratch is a fixed
 * RECIS_PLAN_NOALLOC_SCRATCH_MIB MiB array inside the library's code object (every device the
 * library runs on holds one until the process ends); the call makes no hipMalloc / hipFree /
 * hipHostMalloc and creates no event or stream. n > RECIS_PLAN_NOALLOC_MAX_IDS returns
 * RECIS_ERR_ARG; on a device with so many compute units that the scratch layout of n ids (its
 * histogram has one row per partition tile, and the tiles are sized by the compute-unit count)
 * passes the array, the call returns RECIS_ERR_CAPACITY instead of launching (no gfx950 part does,
 * up to the maximum). All calls on one device share the one array: two calls that overlap in time on a
 * device (different streams or threads) race; calls queued on one stream do not. (With
 * recis_hip_profile_enable(1) the profiler's own events are created as for every other call.)
 */
#define RECIS_PLAN_NOALLOC_SCRATCH_MIB 16
#define RECIS_PLAN_NOALLOC_MAX_IDS 262144
int recis_unique_plan_noalloc(const int64_t* ids, int64_t n, int64_t* unique_out, int32_t* inverse_out,
                              int32_t* row_start_out, int32_t* list_out, int32_t* pos_out,
                              int32_t* hot_items_out, int64_t hot_cap, int64_t* counts_out_dev,
                              void* stream);

/*
 * Per list entry, the input row it reads and its coefficient, for the backward of
 *   pooled segments: src_pool_out = segment of the occurrence, coef_out = weight (/ length for
 *                    MEAN); coef_out may be NULL when there are no weights and mean == 0
 *   padded gather:   src_tile_out = padded output row of the occurrence, -1 beyond seq[f]; the
 *                    S segments are those of n_features features, batch[f] samples each, feature
 *                    f padded to seq[f] rows per sample
 * Either pair of outputs may be NULL (src_tile_out == NULL: batch / seq / n_features unused).
 * list = list_out of recis_unique_plan (entry k lists occurrence list[k]); offsets [S + 1] are
 * the segments' offsets. Entries of occurrences outside the offsets range get src = -1 (skipped).
 * No reference counterpart: the reference's backward kernels search the offsets per element
 * while they scatter (embedding_segment_reduce_kernel.cu:79-120).
 */
int recis_csr_fill_lists(const int32_t* list, int64_t n, const void* offsets, int off_is64, int64_t S,
                         const void* weight, int weight_dtype, int mean, int32_t* src_pool_out,
                         float* coef_out, const int64_t* batch, const int64_t* seq, int64_t n_features,
                         int32_t* src_tile_out, void* stream);

/*
 * out[u, :] (+)= sum over k in [row_start[u], row_start[u+1]) of coef[k] * rows[src[k], :]
 * for u < U, every row written once, no atomics. Rows with at most RECIS_PLAN_HOT_LEN entries
 * are reduced by lanes of one wave; hot rows through the plan's work items: workgroups store
 * one partial row per RECIS_PLAN_HOT_CHUNK entries into library scratch, a second small
 * launch adds them up in chunk order. Without work items (hot_cap == 0) every row goes the
 * first way. accumulate != 0 adds to what out holds. src < 0 skips the entry; coef may be
 * NULL (= 1). D <= 8192.
 * cover_offsets (device, [cover_S + 1], int32 or int64) or NULL: entries whose src lies outside
 * [cover_offsets[0], cover_offsets[cover_S]) are skipped too (occurrences no segment covers,
 * for the backward of the TILE mode where src is the occurrence itself).
 * U may be an upper bound of the number of unique ids (a caller that has not read the plan's
 * count back yet passes n): rows at and past counts_dev[0], the count the plan left on the device,
 * are skipped (out must then hold U rows, of which the first counts_dev[0] are written). The same
 * holds for every recis_csr_gather_reduce* entry point below.
 */
int recis_csr_gather_reduce(const void* rows, int rows_dtype, int64_t n_rows, const int32_t* src,
                            const void* coef, int coef_dtype, const int32_t* row_start,
                            const int32_t* hot_items, int64_t hot_cap, const int64_t* counts_dev,
                            void* out, int out_dtype, int64_t U, int64_t D, int accumulate,
                            const void* cover_offsets, int cover_is64, int64_t cover_S,
                            void* stream);

/*
 * recis_csr_gather_reduce with the sum of unique id u stored at out[out_rows[u], :] instead of
 * out[u, :] (no reference counterpart). out_rows [U] must name every row of out at most once and
 * stay below the rows out holds: a permutation of 0 .. U-1 when U is the exact count. For a caller
 * that wants the rows in another order than the plan's (ids_partition hands the unique ids out in
 * the order of their shard slots: the backward of the pooling writes the gradient rows in that
 * order at once, where it would otherwise write them in the plan's order and copy them).
 */
int recis_csr_gather_reduce_mapped(const void* rows, int rows_dtype, int64_t n_rows,
                                   const int32_t* src, const void* coef, int coef_dtype,
                                   const int32_t* row_start, const int32_t* hot_items,
                                   int64_t hot_cap, const int64_t* counts_dev, void* out,
                                   int out_dtype, int64_t U, int64_t D, int accumulate,
                                   const void* cover_offsets, int cover_is64, int64_t cover_S,
                                   const int32_t* out_rows, void* stream);

/*
 * recis_csr_gather_reduce over input rows that live in n_parts (1 to 8) separate arrays instead
 * of one (no reference counterpart): src numbers the rows of part 0, then those of part 1, and so
 * on (part f holds part_counts[f] rows of D elements of rows_dtype). No coefficients, fp32 output
 * [U, D]. For callers that get the gradient of several outputs as several tensors (one padded
 * gather per feature) and would otherwise concatenate them first. part_rows and part_counts are
 * host arrays.
 */
int recis_csr_gather_reduce_parts(const void* const* part_rows, const int64_t* part_counts,
                                  int n_parts, int rows_dtype, const int32_t* src,
                                  const int32_t* row_start, const int32_t* hot_items,
                                  int64_t hot_cap, const int64_t* counts_dev, void* out, int64_t U,
                                  int64_t D, int accumulate, void* stream);

/*
 * recis_csr_gather_reduce whose result never reaches memory: the finished sum of row u IS the
 * gradient of table row row_index[u] (a negative index skips the row), and the lane group that
 * holds it applies the optimizer's row update at once. Same outcome, bit for bit, as
 * recis_csr_gather_reduce into an fp32 [U, D] buffer followed by recis_block_apply_adamw /
 * recis_block_apply_adagrad(row_index, buffer, ...): the fp32 gradient that the second call would
 * read is the value the first holds in registers. Saves writing and re-reading the [U, D]
 * gradient and one launch. Replaces the pair segment_reduce_backward
 * (csrc/ops/embedding_segment_reduce_kernel.cu:276-350) + block_apply_adamw
 * (csrc/ops/block_apply_adamw_op.cc:114-132) for callers that apply every gradient as it is
 * produced (no gradient accumulation over several batches, one gradient per row per step). The
 * arguments are those of the two calls; row_dtype is the type of the table's rows, beta1_t /
 * beta2_t advance as in recis_block_apply_adamw (also when U == 0).
 */
int recis_csr_gather_reduce_adamw(const void* rows, int rows_dtype, int64_t n_rows, const int32_t* src,
                                  const void* coef, int coef_dtype, const int32_t* row_start,
                                  const int32_t* hot_items, int64_t hot_cap, const int64_t* counts_dev,
                                  int64_t U, int64_t D, const void* cover_offsets, int cover_is64,
                                  int64_t cover_S, const int64_t* row_index, void* const* emb_blocks_dev,
                                  void* const* exp_avg_blocks_dev, void* const* exp_avg_sq_blocks_dev,
                                  int64_t n_blocks, int64_t block_size, int64_t row_pitch_bytes,
                                  int row_dtype, void* beta1_t, void* beta2_t, int beta_is_f64, double lr, double beta1, double beta2,
                                  double weight_decay, double eps, void* stream);
int recis_csr_gather_reduce_adagrad(const void* rows, int rows_dtype, int64_t n_rows, const int32_t* src,
                                    const void* coef, int coef_dtype, const int32_t* row_start,
                                    const int32_t* hot_items, int64_t hot_cap, const int64_t* counts_dev,
                                    int64_t U, int64_t D, const void* cover_offsets, int cover_is64,
                                    int64_t cover_S, const int64_t* row_index, void* const* emb_blocks_dev,
                                    void* const* accum_blocks_dev, int64_t n_blocks, int64_t block_size,
                                    int64_t row_pitch_bytes, int row_dtype, double lr, double eps,
                                    void* stream);

/*
 * Gather-reduce with TWO inputs over the same occurrence lists: list entry k of unique id u adds
 * a.coef[k] * a.rows[a.src[k]] + b.coef[k] * b.rows[b.src[k]] (a negative src skips that term;
 * coef NULL = 1). A lookup whose rows feed two outputs, a pooled one and an unpooled, padded one
 * (the sequence features of the reference: csrc/ops/embedding_segment_reduce_kernel.cu:276-350
 * and the ragged_tile backward, ragged_tile_kernel.cu), has two gradients per occurrence; the
 * reference scatters each into the unique rows by itself, this sums both in the pass that owns the
 * row.
 *   recis_csr_gather_reduce2          out (fp32 [U, D]) (+)= sum; each input fp32, bf16 or f16 (two
 *                                     half-precision inputs must have one type)
 *   recis_csr_gather_reduce2_adamw    the sum is the gradient of table row row_index[u]: the row
 *   recis_csr_gather_reduce2_adagrad  update is applied at once, as by recis_csr_gather_reduce_adamw
 *                                     / _adagrad; each input fp32 or of the table's row type
 * The result equals recis_csr_gather_reduce(a) followed by recis_csr_gather_reduce(b, accumulate)
 * up to fp32 rounding (here both inputs go through one chain of fused multiply-adds, there the
 * first sum is rounded to the output before the second is added).
 */
typedef struct recis_csr_input {
  const void* rows;   /* [n_rows, D] */
  int rows_dtype;
  int64_t n_rows;
  const int32_t* src; /* [n] input row per list entry */
  const void* coef;   /* [n] per list entry, or NULL */
  int coef_dtype;
  /* the SECOND input may come as n_parts (<= 8) arrays laid end to end in src's numbering, as in
   * recis_csr_gather_reduce_parts (rows and n_rows unused then); n_parts = 0: one array */
  const void* const* part_rows; /* host array of device pointers */
  const int64_t* part_counts;   /* host array: rows per part */
  int n_parts;
} recis_csr_input;
int recis_csr_gather_reduce2(const recis_csr_input* a, const recis_csr_input* b, const int32_t* row_start,
                             const int32_t* hot_items, int64_t hot_cap, const int64_t* counts_dev,
                             void* out, int64_t U, int64_t D, int accumulate, void* stream);
int recis_csr_gather_reduce2_adamw(const recis_csr_input* a, const recis_csr_input* b,
                                   const int32_t* row_start, const int32_t* hot_items, int64_t hot_cap,
                                   const int64_t* counts_dev, int64_t U, int64_t D, const int64_t* row_index,
                                   void* const* emb_blocks_dev, void* const* exp_avg_blocks_dev,
                                   void* const* exp_avg_sq_blocks_dev, int64_t n_blocks, int64_t block_size,
                                   int64_t row_pitch_bytes, int row_dtype, void* beta1_t, void* beta2_t, int beta_is_f64, double lr,
                                   double beta1, double beta2, double weight_decay, double eps, void* stream);
int recis_csr_gather_reduce2_adagrad(const recis_csr_input* a, const recis_csr_input* b,
                                     const int32_t* row_start, const int32_t* hot_items, int64_t hot_cap,
                                     const int64_t* counts_dev, int64_t U, int64_t D, const int64_t* row_index,
                                     void* const* emb_blocks_dev, void* const* accum_blocks_dev,
                                     int64_t n_blocks, int64_t block_size, int64_t row_pitch_bytes,
                                     int row_dtype, double lr, double eps, void* stream);

/*
 * The transpose of recis_csr_gather_reduce (no reference counterpart; it produces what
 * segment_reduce_forward gives for one-id segments and for the TILE mode,
 * embedding_segment_reduce_kernel.cu:23-75): out[dst[k], :] = weight[dst[k]] * row(u) for every
 * list entry k in [row_start[u], row_start[u+1]) of every unique id u < U. Every unique row is
 * read once and stored to all its occurrences (hot rows through the plan's work items, like the
 * gather-reduce). Rows come from a dense [U, D] array (rows) or, when emb_blocks_dev != NULL,
 * straight from a block list: row u is row row_index[u] (negative = zeros) of blocks of
 * block_rows rows. weight ([n_out], per OUTPUT row) may be NULL. Output rows no list entry
 * names are not written. dst outside [0, n_out) raises RECIS_DEVERR_INDEX_RANGE. U may be an
 * upper bound of the number of unique ids (a caller that has not read the plan's count back yet
 * passes n): rows at and past counts_dev[0], the count the plan left on the device, are skipped.
 */
int recis_csr_expand_rows(const void* rows, void* const* emb_blocks_dev, int64_t n_blocks,
                          int64_t block_rows, int64_t row_pitch_bytes, const int64_t* row_index, int rows_dtype,
                          const void* weight, int weight_dtype, const int32_t* row_start,
                          const int32_t* dst, const int32_t* hot_items, int64_t hot_cap,
                          const int64_t* counts_dev, void* out, int out_dtype, int64_t U,
                          int64_t n_out, int64_t D, void* stream);
/*
 * The same for a table with a step filter, rows from a block list only: every row that is read
 * (row_index[u] >= 0) also gets stamp_value_dev[0] written at that row of an int64 slot of the
 * same table (stamp_blocks_dev: its blocks, of block_rows rows like the embedding's), which is
 * what the filter hook's update does after a training lookup
 * (recis/nn/modules/hashtable_hook_impl.py:389-426: update_slot(name, index, global_step)): the
 * stamps ride on the pass that reads the rows anyway instead of taking a launch of their own.
 */
int recis_csr_expand_rows_stamped(const void* rows, void* const* emb_blocks_dev, int64_t n_blocks,
                                  int64_t block_rows, int64_t row_pitch_bytes,
                                  const int64_t* row_index, int rows_dtype,
                                  const void* weight, int weight_dtype, const int32_t* row_start,
                                  const int32_t* dst, const int32_t* hot_items, int64_t hot_cap,
                                  const int64_t* counts_dev, void* out, int out_dtype, int64_t U,
                                  int64_t n_out, int64_t D, void* const* stamp_blocks_dev,
                                  const int64_t* stamp_value_dev, void* stream);

/* ------------------------------------------------------------------------- *
 * Feature-engine scalar ops (lists as HOST arrays of device pointers)
 * ------------------------------------------------------------------------- */

/*
 * recis_fused_hash        fused_hash_cuda, csrc/ops/fused_hash_kernel.cu:421-458:
 *                         out_t[i] = hash(values_t[off_t[i] .. off_t[i+1])), kind 0 =
 *                         FarmHash Hash64, 1 = MurmurHash64A seed 0
 * recis_fused_uint64_mod  fused_uint64_mod_cuda, csrc/ops/fused_uint64_mod_kernel.cu:12-39
 *                         (and uint64_mod_cuda with one tensor): (int64)((uint64)x % mod_t)
 * recis_fused_bucketized  fused_bucketized_cuda, csrc/ops/fused_bucketized_kernel.cu:19-60
 *                         (and bucketize_cuda_op): number of boundaries <= v, NaN -> len
 * recis_fused_multi_hash  fused_multi_hash_cuda, csrc/ops/multi_hash_kernel.cu:11-74:
 *                         one job per (tensor, hash): (((x*mul) % p + p) % p) % bucket
 */
int recis_fused_hash(const int8_t* const* values_ptrs, const int64_t* values_sizes,
                     const void* const* offsets_ptrs, int off_is64, const int64_t* n_strings,
                     int64_t* const* out_ptrs, int64_t n_tensors, int kind, void* stream);
int recis_fused_uint64_mod(const int64_t* const* in_ptrs, const int64_t* sizes,
                           const int64_t* mods, int64_t* const* out_ptrs, int64_t n_tensors,
                           void* stream);
int recis_fused_bucketized(const float* const* in_ptrs, const int64_t* sizes,
                           const float* const* boundaries_ptrs, const int64_t* boundary_lens,
                           int64_t* const* out_ptrs, int64_t n_tensors, void* stream);
/* recis_fused_bucketized followed by recis_fused_uint64_mod(mods) on its outputs, in one pass (a
 * Bucketize -> Mod chain of one feature; the bucket is reduced where it is found). mods: host
 * array, one positive modulus per tensor. */
int recis_fused_bucketized_mod(const float* const* in_ptrs, const int64_t* sizes,
                               const float* const* boundaries_ptrs, const int64_t* boundary_lens,
                               const int64_t* mods, int64_t* const* out_ptrs, int64_t n_tensors,
                               void* stream);
int recis_fused_multi_hash(const int64_t* const* in_ptrs, const int64_t* sizes,
                           const int64_t* muls, const int64_t* primes, const int64_t* buckets,
                           int64_t* const* out_ptrs, int64_t n_jobs, void* stream);

/* ------------------------------------------------------------------------- *
 * Sequence truncation of lists of ragged tensors
 * ------------------------------------------------------------------------- */

/*
 * fused_ragged_cutoff (2-D, inner_ptrs == NULL) and fused_ragged_cutoff_3D, the op functions of
 * csrc/ops/fused_ragged_cutoff.cc:10-140 and :143-287 (kernels post_cutoff_lens_kernel,
 * seg_scan_sum_kernel, seg_gen_offsets_kernel, fused_ragged_cutoff_kernel.cu:29-70,100-160,
 * 260-371), for n_tensors ragged tensors at once. Lists are HOST arrays of device pointers.
 *
 * 2-D, tensor t with offsets outer_ptrs[t] [n_rows[t] + 1]: row r keeps min(len, keep[t])
 * elements, the first ones, or the last ones when drop_left[t]; out_offsets_ptrs[t]
 * [n_rows[t] + 1] receives the new offsets, drop_nums_ptrs[t] / pad_nums_ptrs[t] [n_rows[t]]
 * (each may be NULL) len - keep where len >= keep (else 0) and keep - len where len < keep
 * (else 0). pad_left is not used: a 2-D result is not padded.
 * 3-D, outer offsets [n_rows[t] + 1] over inner rows, inner offsets inner_ptrs[t]
 * [n_inner_rows[t] + 1] over values: every sequence comes out with exactly keep[t] inner rows.
 * A longer one loses inner rows at the end (at the start when drop_left[t]); a shorter one gets
 * empty rows at the end (at the start when pad_left[t]). out_outer_ptrs[t] [n_rows[t] + 1] =
 * k * keep[t]; out_offsets_ptrs[t] [n_rows[t] * keep[t] + 1] = new inner offsets; drop / pad
 * counts are per sequence.
 * Both: src_ptrs[t] (int64 [output rows], caller's scratch, read by recis_ragged_cutoff_copy)
 * receives the position of every output row's first element in the source values;
 * totals_dev [n_tensors] the number of values each tensor keeps. Offsets are int32 or int64
 * (off_is64), the same for inputs and outputs. A source range outside [0, n_values[t]) or an
 * inner row outside [0, n_inner_rows[t]) gives an empty row and raises
 * RECIS_DEVERR_INDEX_RANGE. Nothing here waits for the device.
 */
int recis_ragged_cutoff_rows(const void* const* outer_ptrs, const void* const* inner_ptrs,
                             int off_is64, const int64_t* n_rows, const int64_t* n_inner_rows,
                             const int64_t* n_values, const int64_t* keep,
                             const uint8_t* drop_left, const uint8_t* pad_left, int64_t n_tensors,
                             void* const* out_offsets_ptrs, void* const* out_outer_ptrs,
                             void* const* drop_nums_ptrs, void* const* pad_nums_ptrs,
                             int64_t* const* src_ptrs, int64_t* totals_dev, void* stream);

/*
 * The values of a cutoff (fused_ragged_cutoff_kernel / fused_ragged_cutoff_3D_kernel,
 * fused_ragged_cutoff_kernel.cu:462-556,634-728): out_values_ptrs[t][e] for e < totals[t]
 * (HOST array: what recis_ragged_cutoff_rows left in totals_dev, read back by the caller to
 * size the outputs) = values_ptrs[t][src + (e - offset)] of the output row that holds e.
 * elem_size 1, 2, 4 or 8 bytes. n_out_rows[t] = rows (2-D) or rows * keep (3-D).
 */
int recis_ragged_cutoff_copy(const void* const* values_ptrs, int elem_size,
                             const void* const* out_offsets_ptrs, int off_is64,
                             const int64_t* n_out_rows, const int64_t* const* src_ptrs,
                             const int64_t* totals, void* const* out_values_ptrs,
                             int64_t n_tensors, void* stream);

/* element kinds of recis_dense_to_ragged_rows (the types the reference dispatches on) */
#define RECIS_SEQ_F32 0
#define RECIS_SEQ_F64 1
#define RECIS_SEQ_I32 2
#define RECIS_SEQ_I64 3

/*
 * ragged_to_dense_cuda (csrc/ops/ragged_to_dense_kernel.cu:34-152; CPU twin ragged_to_dense.cc:6-45):
 * out [batch, widths[0], ..., widths[n_dims-1]] (batch = offsets_sizes[0] - 1) takes
 * values[...] where every coordinate lies inside its row, default_value (elem_size raw bytes)
 * elsewhere. offsets_ptrs / offsets_sizes / widths are HOST arrays (n_dims <= 5); the widths are
 * the caller's (the reference takes the longest row of every level, which costs it a read-back
 * per level; a row longer than its width is cut).
 */
int recis_ragged_to_dense(const void* values, int elem_size, int64_t n_values,
                          const void* const* offsets_ptrs, const int64_t* offsets_sizes,
                          int off_is64, const int64_t* widths, int n_dims,
                          const void* default_value, void* out, void* stream);

/*
 * dense_to_ragged_cuda (csrc/ops/dense_to_ragged_kernel.cu:16-83), offsets part: the length of
 * row r of data [rows, cols] is the position after its last element != *invalid_value;
 * out_offsets (int32 [rows + 1]) receives the running sum, src (int64 [rows], caller's scratch)
 * r * cols, total_dev [1] the number of values. The values follow from
 * recis_ragged_cutoff_copy(data, ..., out_offsets, 0, rows, src, total, ...).
 */
int recis_dense_to_ragged_rows(const void* data, int dtype_kind, int64_t rows, int64_t cols,
                               const void* invalid_value, int32_t* out_offsets, int64_t* src,
                               int64_t* total_dev, void* stream);

/*
 * feature_cross_ragged_cuda (csrc/ops/feature_cross_ragged_kernel.cu:286-416; CPU twin
 * feature_cross_ragged.cc:24-98): segment s of the result holds one entry for every pair
 * (distinct id of x's row s, distinct id of y's row s): id = MurmurHash64A of the two 8-byte
 * words with seed 0 (ragged_common.cuh:105-125), weight = product of the weights the two ids
 * carry at their FIRST occurrence in their rows (NULL weights = 1). Entries are ordered by first
 * occurrence, x outermost (the reference's order differs between its CPU and CUDA paths; its
 * test compares rows as multisets). n_seg = min(rows of x, rows of y).
 * recis_feature_cross_rows fills x_rank [nx] / y_rank [ny] (int32 scratch: rank of an element
 * among the distinct ids of its row, -1 for a repeat), y_count [n_seg], out_offsets
 * ([n_seg + 1], the type of the input offsets) and total_dev [1]; the caller reads the total
 * back to size out_val / out_weight for recis_feature_cross_emit. Weights are float32, or
 * float64 when weight_is_f64.
 */
int recis_feature_cross_rows(const int64_t* x_val, const void* x_off, int64_t nx,
                             const int64_t* y_val, const void* y_off, int64_t ny, int off_is64,
                             int64_t n_seg, int32_t* x_rank, int32_t* y_rank, int32_t* y_count,
                             void* out_offsets, int64_t* total_dev, void* stream);
int recis_feature_cross_emit(const int64_t* x_val, const void* x_off, const void* x_weight,
                             int64_t nx, const int64_t* y_val, const void* y_off,
                             const void* y_weight, int64_t ny, int off_is64, int weight_is_f64,
                             int64_t n_seg, const int32_t* x_rank, const int32_t* y_rank,
                             const int32_t* y_count, const void* out_offsets, int64_t total,
                             int64_t* out_val, void* out_weight, void* stream);

/*
 * calc_ragged_index, drop left / pad right (csrc/ops/calc_ragged_index.cc:15-84; the only side
 * combination the reference implements, on the CPU): row r of topk [rows, cols] holds
 * positions in ragged row src = indicator[r] (0 <= src < src_rows) of offset [src_rows + 1],
 * counted from the first element kept by a left truncation of drop_num[src] elements. Kept:
 * e = topk[r, c] + offset[src] + drop_num[src] with offset[src] <= e < offset[src + 1], in column
 * order. out_index (the type of topk, room for rows * cols) receives the kept e of all rows back
 * to back, out_offsets (the type of offset, [rows + 1]) their running count per row, total_dev
 * [1] the count. Each of drop_num / offset / topk / indicator is int32 or int64 (its *_is64).
 * An indicator outside [0, src_rows) keeps nothing and raises the index-range soft error.
 */
int recis_ragged_topk_index(const void* drop_num, int drop_is64, const void* offset, int off_is64,
                            int64_t src_rows, const void* topk, int topk_is64,
                            const void* indicator, int indicator_is64, int64_t rows, int64_t cols,
                            void* out_index, void* out_offsets, int64_t* total_dev, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* RECIS_HIP_H_ */
