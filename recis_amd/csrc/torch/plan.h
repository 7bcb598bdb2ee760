// torch.classes.recis.BatchPlan: the dedup of one batch of ids plus the occurrence lists per
// unique id, as recis_unique_plan leaves them in device memory (include/recis_hip.h). No
// counterpart in the reference, whose dedup is the radix sort of
// csrc/ops/ids_partition_kernel.cu:86-131 followed by atomic scatters over duplicated ids; the
// plan is what lets every gradient scatter over duplicates run as a gather-reduce per unique row.
#pragma once
#include <cstdlib>

#include <ATen/ATen.h>
#include <torch/custom_class.h>

#include <tuple>
#include <utility>
#include <vector>

#include "recis_hip.h"

namespace recis {

class BatchPlan : public torch::CustomClassHolder {
 public:
  // ids: the batch as one or more id tensors laid end to end; tags (one per tensor) tag every id
  // with its table as ids_encode does. map != nullptr: the unique ids are found or inserted in that
  // id map in the same pass and index_buf holds their rows. wait == false returns without the host
  // copy of the unique count (at most one such plan per stream has its count on the way).
  static c10::intrusive_ptr<BatchPlan> Make(const std::vector<at::Tensor>& ids,
                                            const c10::optional<std::vector<int64_t>>& tags, recis_idmap* map,
                                            bool wait, bool need_inverse, bool need_pos);

  int64_t n() const { return n_; }
  int64_t serial() const { return serial_; }
  int64_t hot_cap() const { return hot_cap_; }
  // The number of unique ids on the host; a plan made with wait == false fetches it here.
  int64_t U();
  // The count if the host has it already, else the number of ids: for kernels that take the count
  // from device memory and only need a bound to size their grid.
  int64_t U_bound() const { return U_ < 0 ? n_ : U_; }
  at::Tensor unique();
  at::Tensor inverse();
  at::Tensor pos();
  const at::Tensor& unique_buf() const { return unique_buf_; }
  const at::Tensor& row_start() const { return row_start_; }
  const at::Tensor& occ() const { return occ_; }
  const at::Tensor& hot_items() const { return hot_items_; }
  const at::Tensor& counts() const { return counts_; }
  c10::optional<at::Tensor> index_buf() const {
    return index_buf_.defined() ? c10::optional<at::Tensor>(index_buf_) : c10::nullopt;
  }
  at::Device device() const { return unique_buf_.device(); }

  // (src, coef) per list entry for the backward of pooled segments, cached per (offsets, weight,
  // mean) so that forward-time and backward-time callers share it.
  std::tuple<at::Tensor, c10::optional<at::Tensor>> SrcCoefForPool(const at::Tensor& offsets,
                                                                   const c10::optional<at::Tensor>& weight,
                                                                   bool mean);
  // src per list entry for the backward of the padded gather (ragged_tile).
  at::Tensor SrcForTile(const std::vector<int64_t>& batch, const std::vector<int64_t>& seq,
                        const at::Tensor& offsets);
  // both of the above for the same segments in one launch: (src_pool, coef_pool, src_tile)
  std::tuple<at::Tensor, c10::optional<at::Tensor>, at::Tensor> SrcForPoolAndTile(
      const at::Tensor& offsets, const c10::optional<at::Tensor>& weight, bool mean,
      const std::vector<int64_t>& batch, const std::vector<int64_t>& seq);

  // The counted lookup a table queued for this plan (owner = the table's address; 0 = none).
  void NoteLookup(const void* owner, int64_t call) { lookup_calls_.emplace_back(owner, call); }
  int64_t LookupCall(const void* owner) const;
  void SetIndexBuf(at::Tensor t) { index_buf_ = std::move(t); }
  const at::Tensor& IndexBufRaw() const { return index_buf_; }

 private:
  void FillLate();
  std::tuple<at::Tensor, at::Tensor, at::Tensor> FillLists(const at::Tensor& offsets, const at::Tensor& weight,
                                                           bool mean, bool want_pool,
                                                           const std::vector<int64_t>* batch,
                                                           const std::vector<int64_t>* seq);
  int64_t n_ = 0, serial_ = 0, hot_cap_ = 0, U_ = -1;
  void* stream_ = nullptr;
  at::Tensor unique_buf_, inverse_, row_start_, occ_, pos_, hot_items_, counts_, index_buf_, unique_;
  std::vector<std::pair<const void*, int64_t>> lookup_calls_;
  // cache of SrcCoefForPool
  const void* fill_offsets_ = nullptr;
  const void* fill_weight_ = nullptr;
  bool fill_mean_ = false, fill_valid_ = false;
  at::Tensor fill_src_, fill_coef_, fill_keep_offsets_, fill_keep_weight_;
};

using BatchPlanPtr = c10::intrusive_ptr<BatchPlan>;

// torch.ops.recis.unique_plan: a plan of `ids` without a table, or (idmap_handle != 0: the address
// of a recis_idmap, for callers that hold one through the C ABI) with the find-or-insert in it.
BatchPlanPtr unique_plan(std::vector<at::Tensor> ids, c10::optional<std::vector<int64_t>> tags, int64_t idmap_handle,
                         bool wait, bool need_inverse, bool need_pos);

// Soft errors of the device (bad row index, full id map, ...) that travelled to host memory with
// the last staged unique count of `stream`, as an exception.
void raise_staged_device_errors(void* stream);

}  // namespace recis
