#include "plan.h"

#include <atomic>
#include <mutex>
#include <unordered_map>

#include "abi_util.h"
#include "ops.h"

namespace recis {

using namespace recis::hipabi;

namespace {

constexpr int64_t kPlanJobs = 64;  // arrays one recis_unique_plan_jobs call takes

std::mutex g_staged_mu;
// stream -> serial of the plan whose count is on its way to that stream's staging word
std::unordered_map<void*, int64_t> g_staged;
std::atomic<int64_t> g_serial{1};

std::string describe_device_errors(int bits) {
  std::string s;
  auto add = [&](int bit, const char* text) {
    if (bits & bit) {
      if (!s.empty()) s += "; ";
      s += text;
    }
  };
  add(RECIS_DEVERR_INDEX_RANGE, "an index outside the rows / blocks the caller passed");
  add(RECIS_DEVERR_OFFSETS, "offsets not monotone or out of range");
  add(RECIS_DEVERR_TABLE_FULL, "the id map found no free slot");
  add(RECIS_DEVERR_PLAN_OVERFLOW, "batch plan: too many distinct ids in one hash bucket");
  return s + " (bits " + std::to_string(bits) + ")";
}

at::Tensor flat_ids(const at::Tensor& t) {
  require_gpu(t, "ids");
  if (t.dim() == 1 && t.scalar_type() == at::kLong && t.is_contiguous()) return t;
  return t.to(at::kLong).contiguous().view({-1});
}

}  // namespace

void raise_staged_device_errors(void* stream) {
  int bits = 0;
  check(recis_hip_staged_device_errors(&bits, stream));
  if (bits) {
    int polled = 0;
    check(recis_hip_poll_device_errors(&polled));  // waits for the device and clears the word
    TORCH_CHECK(false, "librecis_hip: device-side errors in earlier kernels: ", describe_device_errors(bits | polled));
  }
}

BatchPlanPtr BatchPlan::Make(const std::vector<at::Tensor>& ids_in, const c10::optional<std::vector<int64_t>>& tags,
                             recis_idmap* map, bool wait, bool need_inverse, bool need_pos) {
  TORCH_CHECK(!tags.has_value() || tags->size() == ids_in.size(), "unique_plan: ", tags.has_value() ? tags->size() : 0,
              " tags for ", ids_in.size(), " id tensors");
  std::vector<at::Tensor> jobs;
  jobs.reserve(ids_in.size());
  for (const auto& t : ids_in) jobs.push_back(flat_ids(t));
  if (jobs.empty() || static_cast<int64_t>(jobs.size()) > kPlanJobs) {
    // too many arrays for one call (or none): make the batch first
    TORCH_CHECK(!jobs.empty(), "unique_plan: no id tensors");
    at::Tensor batch;
    if (tags.has_value()) {
      batch = functional::ids_encode(jobs, at::tensor(*tags, at::TensorOptions().dtype(at::kLong)));
    } else {
      batch = at::cat(jobs);
    }
    jobs.assign(1, batch);
  }
  const bool tagged = tags.has_value() && ids_in.size() == jobs.size();
  int64_t n = 0;
  for (const auto& t : jobs) n += t.numel();
  const at::Device dev = jobs[0].device();
  c10::DeviceGuard guard(dev);
  auto p = c10::make_intrusive<BatchPlan>();
  p->serial_ = g_serial.fetch_add(1);
  p->n_ = n;
  auto i64 = at::TensorOptions().device(dev).dtype(at::kLong);
  auto i32 = at::TensorOptions().device(dev).dtype(at::kInt);
  p->unique_buf_ = at::empty({n}, i64);
  if (need_inverse) p->inverse_ = at::empty({n}, i32);
  p->row_start_ = at::empty({n + 1}, i32);
  p->occ_ = at::empty({n}, i32);
  if (need_pos) p->pos_ = at::empty({n}, i32);
  p->hot_cap_ = n / RECIS_PLAN_HOT_LEN + n / RECIS_PLAN_HOT_CHUNK + 2;
  p->hot_items_ = at::empty({2 * p->hot_cap_}, i32);
  p->counts_ = at::empty({2}, i64);
  if (map != nullptr) p->index_buf_ = at::empty({n}, i64);
  p->stream_ = stream_of(dev);
  int64_t count = 0;
  {
    // every launch overwrites the stream's staging word: an earlier plan whose count is still
    // outstanding there must read its own device word from now on
    std::lock_guard<std::mutex> lock(g_staged_mu);
    g_staged.erase(p->stream_);
  }
  auto ptrs = host_ptrs<int64_t>(jobs);
  auto sizes = numels(jobs);
  auto i32p = [](const at::Tensor& t) { return t.defined() ? t.data_ptr<int32_t>() : nullptr; };
  check(recis_unique_plan_jobs(map, ptrs.data(), sizes.data(), tagged ? tags->data() : nullptr,
                               static_cast<int64_t>(jobs.size()), p->unique_buf_.data_ptr<int64_t>(), i32p(p->inverse_),
                               i32p(p->row_start_), i32p(p->occ_), i32p(p->pos_), i32p(p->hot_items_), p->hot_cap_,
                               p->counts_.data_ptr<int64_t>(),
                               p->index_buf_.defined() ? p->index_buf_.data_ptr<int64_t>() : nullptr,
                               wait ? &count : nullptr, wait ? 0 : RECIS_PLAN_STAGE_COUNT, p->stream_));
  if (wait) {
    p->U_ = count;
    raise_staged_device_errors(p->stream_);
  } else {
    std::lock_guard<std::mutex> lock(g_staged_mu);
    g_staged[p->stream_] = p->serial_;
  }
  return p;
}

int64_t BatchPlan::U() {
  if (U_ < 0) {
    bool staged = false;
    {
      std::lock_guard<std::mutex> lock(g_staged_mu);
      auto it = g_staged.find(stream_);
      if (it != g_staged.end() && it->second == serial_) {
        staged = true;
        g_staged.erase(it);
      }
    }
    if (staged) {
      c10::DeviceGuard guard(device());
      int64_t count = 0;
      check(recis_unique_plan_count(&count, stream_));
      U_ = count;
      raise_staged_device_errors(stream_);
    } else {  // a later plan took the stream's staging word: read this plan's own device word
      U_ = counts_[0].item<int64_t>();
    }
  }
  return U_;
}

at::Tensor BatchPlan::unique() {
  if (!unique_.defined()) unique_ = unique_buf_.narrow(0, 0, U());
  return unique_;
}

void BatchPlan::FillLate() {
  c10::DeviceGuard guard(device());
  auto i32 = at::TensorOptions().device(device()).dtype(at::kInt);
  at::Tensor inv = inverse_.defined() ? at::Tensor() : at::empty({n_}, i32);
  at::Tensor pos = pos_.defined() ? at::Tensor() : at::empty({n_}, i32);
  if (n_) {
    check(recis_plan_inverse_from_lists(row_start_.data_ptr<int32_t>(), occ_.data_ptr<int32_t>(),
                                        counts_.data_ptr<int64_t>(), n_, inv.defined() ? inv.data_ptr<int32_t>() : nullptr,
                                        pos.defined() ? pos.data_ptr<int32_t>() : nullptr, stream_of(device())));
  }
  if (inv.defined()) inverse_ = inv;
  if (pos.defined()) pos_ = pos;
}

at::Tensor BatchPlan::inverse() {
  if (!inverse_.defined()) FillLate();
  return inverse_;
}

at::Tensor BatchPlan::pos() {
  if (!pos_.defined()) FillLate();
  return pos_;
}

int64_t BatchPlan::LookupCall(const void* owner) const {
  for (auto it = lookup_calls_.rbegin(); it != lookup_calls_.rend(); ++it) {
    if (it->first == owner) return it->second;
  }
  return 0;
}

std::tuple<at::Tensor, at::Tensor, at::Tensor> BatchPlan::FillLists(const at::Tensor& offsets_in,
                                                                    const at::Tensor& weight_in, bool mean,
                                                                    bool want_pool, const std::vector<int64_t>* batch,
                                                                    const std::vector<int64_t>* seq) {
  require_gpu(offsets_in, "offsets");
  at::Tensor offsets = offsets_in.contiguous();
  const at::Device dev = offsets.device();
  c10::DeviceGuard guard(dev);
  const int64_t S = offsets.numel() - 1;
  auto i32 = at::TensorOptions().device(dev).dtype(at::kInt);
  at::Tensor src, coef, tile, weight;
  if (weight_in.defined()) {
    require_gpu(weight_in, "weight");
    weight = weight_in.contiguous();
  }
  if (want_pool) {
    src = at::empty({n_}, i32);
    if (weight.defined() || mean) coef = at::empty({n_}, i32.dtype(at::kFloat));
  }
  if (batch != nullptr) {
    TORCH_CHECK(batch->size() == seq->size(), "batch and seq differ in length");
    tile = at::empty({n_}, i32);
  }
  if (n_) {
    check(recis_csr_fill_lists(occ_.data_ptr<int32_t>(), n_, offsets.data_ptr(), index_kind(offsets, "offsets"), S,
                               weight.defined() ? weight.data_ptr() : nullptr,
                               weight.defined() ? dtype_code(weight.scalar_type()) : 0, mean ? 1 : 0,
                               src.defined() ? src.data_ptr<int32_t>() : nullptr,
                               coef.defined() ? coef.data_ptr<float>() : nullptr, batch ? batch->data() : nullptr,
                               batch ? seq->data() : nullptr, batch ? static_cast<int64_t>(batch->size()) : 0,
                               tile.defined() ? tile.data_ptr<int32_t>() : nullptr, stream_of(dev)));
  }
  return std::make_tuple(src, coef, tile);
}

std::tuple<at::Tensor, c10::optional<at::Tensor>> BatchPlan::SrcCoefForPool(const at::Tensor& offsets,
                                                                             const c10::optional<at::Tensor>& weight,
                                                                             bool mean) {
  const bool has_w = weight.has_value() && weight->defined();
  if (offsets.numel() - 1 == n_ && !has_w) {
    return std::make_tuple(occ_, c10::optional<at::Tensor>());  // one id per segment: an occurrence is its own segment
  }
  const void* wp = has_w ? weight->data_ptr() : nullptr;
  if (fill_valid_ && fill_offsets_ == offsets.data_ptr() && fill_weight_ == wp && fill_mean_ == mean) {
    return std::make_tuple(fill_src_, fill_coef_.defined() ? c10::optional<at::Tensor>(fill_coef_) : c10::nullopt);
  }
  auto filled = FillLists(offsets, has_w ? *weight : at::Tensor(), mean, true, nullptr, nullptr);
  fill_offsets_ = offsets.data_ptr();
  fill_weight_ = wp;
  fill_keep_offsets_ = offsets;  // alive as long as the cache entry: its address cannot be handed out again
  fill_keep_weight_ = has_w ? *weight : at::Tensor();
  fill_mean_ = mean;
  fill_valid_ = true;
  fill_src_ = std::get<0>(filled);
  fill_coef_ = std::get<1>(filled);
  return std::make_tuple(fill_src_, fill_coef_.defined() ? c10::optional<at::Tensor>(fill_coef_) : c10::nullopt);
}

at::Tensor BatchPlan::SrcForTile(const std::vector<int64_t>& batch, const std::vector<int64_t>& seq,
                                 const at::Tensor& offsets) {
  return std::get<2>(FillLists(offsets, at::Tensor(), false, false, &batch, &seq));
}

std::tuple<at::Tensor, c10::optional<at::Tensor>, at::Tensor> BatchPlan::SrcForPoolAndTile(
    const at::Tensor& offsets, const c10::optional<at::Tensor>& weight, bool mean, const std::vector<int64_t>& batch,
    const std::vector<int64_t>& seq) {
  const bool has_w = weight.has_value() && weight->defined();
  auto filled = FillLists(offsets, has_w ? *weight : at::Tensor(), mean, true, &batch, &seq);
  fill_offsets_ = offsets.data_ptr();
  fill_weight_ = has_w ? weight->data_ptr() : nullptr;
  fill_keep_offsets_ = offsets;
  fill_keep_weight_ = has_w ? *weight : at::Tensor();
  fill_mean_ = mean;
  fill_valid_ = true;
  fill_src_ = std::get<0>(filled);
  fill_coef_ = std::get<1>(filled);
  return std::make_tuple(fill_src_, fill_coef_.defined() ? c10::optional<at::Tensor>(fill_coef_) : c10::nullopt,
                         std::get<2>(filled));
}

BatchPlanPtr unique_plan(std::vector<at::Tensor> ids, c10::optional<std::vector<int64_t>> tags, int64_t idmap_handle,
                         bool wait, bool need_inverse, bool need_pos) {
  return BatchPlan::Make(ids, tags, reinterpret_cast<recis_idmap*>(idmap_handle), wait, need_inverse, need_pos);
}

}  // namespace recis
