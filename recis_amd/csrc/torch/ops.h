// The operators RecIS registers as torch.ops.recis.* (csrc/bind.cc:172-210), with the reference's
// C++ signatures (so that torch infers the same schemas), implemented on librecis_hip.so.
#pragma once

#include <ATen/ATen.h>

#include <string>
#include <tuple>
#include <vector>

#include "plan.h"

namespace recis {
namespace functional {

using Tensor = at::Tensor;
using TensorList = std::vector<at::Tensor>;

// csrc/ops/embedding_segment_reduce.h:9-22
Tensor segment_reduce_forward(Tensor unique_emb, c10::optional<Tensor> weight, Tensor reverse_indices,
                              Tensor offsets, std::string mode);
Tensor segment_reduce_backward(Tensor grad_output, c10::optional<Tensor> weight, Tensor reverse_indices,
                               Tensor offsets, int64_t unique_size, std::string mode);
Tensor merge_offsets(const TensorList& offsets, Tensor& max_value);
Tensor gen_segment_indices_by_offset(Tensor offset);
// csrc/ops/segment_ops.h:5-13
Tensor segment_sum(Tensor data, c10::optional<Tensor> weight, Tensor indices, Tensor segment_ids,
                   at::Scalar num_segments);
Tensor segment_mean(Tensor data, c10::optional<Tensor> weight, Tensor segment_ids, at::Scalar num_segments);
// csrc/ops/block_ops.h:6-51
void block_insert(const Tensor ids, const Tensor embedding, TensorList emb_blocks, int64_t block_size);
void block_insert_with_mask(const Tensor ids, const Tensor embedding, const Tensor mask, TensorList emb_blocks,
                            int64_t block_size);
Tensor block_gather(const Tensor ids, TensorList emb_blocks, int64_t block_size, int64_t default_key,
                    bool readonly);
Tensor block_filter(const Tensor ids, TensorList emb_blocks, int64_t block_size, int64_t step);
Tensor gather(const Tensor ids, const Tensor emb);
// csrc/ops/block_apply_adamw_op.h:6-12
void block_apply_adamw(const Tensor index, const Tensor grad, TensorList emb_blocks, Tensor beta1_t,
                       Tensor beta2_t, Tensor step, TensorList exp_avg, TensorList exp_avg_sq, double lr,
                       double beta1, double beta2, double weight_decay, double eps, int64_t block_size);
// Sparse Adagrad row update: an addition with no counterpart in the reference.
void block_apply_adagrad(const Tensor index, const Tensor grad, TensorList emb_blocks, TensorList accum,
                         double lr, double eps, int64_t block_size);
// csrc/ops/hashtable_ops.h:17-34
Tensor generate_ids_op(const int64_t gen_num, TensorList free_blocks, const int64_t free_count,
                       const int64_t cur_count, const int64_t free_block_size);
void free_ids_op(Tensor free_ids, TensorList free_blocks, const int64_t free_count,
                 const int64_t free_block_size);
std::tuple<Tensor, Tensor> mask_key_index_op(Tensor in_keys, Tensor mask, Tensor out_index, int64_t out_size);
Tensor scatter_ids_with_mask_op(Tensor out_ids, Tensor in_ids, Tensor mask_index);
// csrc/ops/ids_encode.h:15, ids_partition.h:14
Tensor ids_encode(TensorList inputs, Tensor table_ids);
std::tuple<Tensor, Tensor, Tensor> ids_partition(const Tensor& ids, int64_t num_parts);
// csrc/ops/uint64_mod.h, bucketize_op.h, fused_uint64_mod.h, fused_bucketized.h, fused_hash.h, multi_hash.h
Tensor uint64_mod(Tensor inputs, at::Scalar num);
Tensor bucketize_op(Tensor values, Tensor boundaries);
TensorList fused_uint64_mod(TensorList inputs, Tensor mod_vec);
TensorList fused_bucketized(TensorList inputs, TensorList boundaries);
// fused_bucketized followed by fused_uint64_mod of the buckets (one positive modulus per tensor) in one
// pass: an addition (the reference runs the two operators one after the other).
TensorList fused_bucketized_mod(TensorList inputs, TensorList boundaries, std::vector<int64_t> mods);
TensorList fused_hash(TensorList inputs, TensorList input_offsets, const std::string& hash_type);
TensorList fused_multi_hash(TensorList inputs, TensorList muls, TensorList primes, TensorList bucket_num);
// csrc/ops/ragged_tile.h:9-18
TensorList ragged_tile(const std::vector<int64_t>& batch, const std::vector<int64_t>& seq, Tensor value,
                       Tensor offset, Tensor table);
Tensor ragged_tile_back(Tensor batch_seq, const std::vector<int64_t>& batch_info, Tensor value, Tensor offset,
                        Tensor dy);
// csrc/ops/ragged_to_dense.h:5-7, dense_to_ragged.h:8-10
Tensor ragged_to_dense(Tensor values, const TensorList& offsets, at::Scalar default_value);
// csrc/ops/ragged_to_sparse.h: the ragged tensor as a coalesced sparse COO tensor
Tensor ragged_to_sparse(Tensor values, TensorList offset_splits);
std::tuple<Tensor, Tensor> dense_to_ragged(const Tensor& data, bool check_invalid, const Tensor& invalid_value);
// csrc/ops/fused_ragged_cutoff.h:9-14,33-39
std::tuple<TensorList, TensorList, TensorList, TensorList, Tensor, Tensor> fused_ragged_cutoff(
    TensorList value, TensorList offset, Tensor keep_length, Tensor drop_sides, Tensor pad_sides);
std::tuple<TensorList, TensorList, TensorList> fused_ragged_cutoff_3D(TensorList values, TensorList outer_offsets,
                                                                      TensorList inner_offsets,
                                                                      Tensor keep_lengths, Tensor drop_sides,
                                                                      Tensor pad_sides);
// csrc/ops/feature_cross_ragged.h:7-10, calc_ragged_index.h:14-17
std::tuple<Tensor, Tensor, Tensor> feature_cross_ragged(const Tensor& x_value, const Tensor& x_offsets,
                                                        const Tensor& x_weight, const Tensor& y_value,
                                                        const Tensor& y_offsets, const Tensor& y_weight);
std::tuple<Tensor, Tensor> calc_ragged_index(Tensor drop_num, Tensor pad_num, Tensor drop_side, Tensor pad_side,
                                             Tensor offset, Tensor topk_index, Tensor indicator);


// ---- over a batch plan (additions: the reference scatters with atomics instead)
// out[u] = sum over the occurrence list of unique id u of coef[k] * rows[src[k]]: fp32 [U, D]. coef
// and cover may be undefined (see recis_csr_gather_reduce). out_rows (int32 [U], a permutation) or
// undefined: the sum of unique id u goes to row out_rows[u] of the result.
Tensor csr_gather_reduce(const Tensor& rows, const BatchPlanPtr& plan, const Tensor& src, const Tensor& coef,
                         const Tensor& cover, const Tensor& out_rows = Tensor());
// the same over rows that live in up to 8 arrays laid end to end in src's numbering
Tensor csr_gather_reduce_parts(const TensorList& parts, const BatchPlanPtr& plan, const Tensor& src);
// ids_partition notes the unique ids it hands out; known_unique(t) says whether t is one of those
// tensors, unchanged since (same memory, same length, same version counter). The noted tensors are
// kept alive, so their addresses cannot be handed out to another tensor meanwhile.
void note_unique(const Tensor& t);
bool known_unique(const Tensor& t);
// The same for the inverse ids_partition hands out: the plan of that dedup and the place of each of
// its unique ids in the sorted order (rank, int32 [U]) stay available to the backward over that
// inverse (the last two calls).
void note_partition(const Tensor& inverse, const BatchPlanPtr& plan, const Tensor& rank);
bool known_partition(const Tensor& inverse, BatchPlanPtr* plan, Tensor* rank);

}  // namespace functional
}  // namespace recis
