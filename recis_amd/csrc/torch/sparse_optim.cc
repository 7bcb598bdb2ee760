#include "sparse_optim.h"

#include <ATen/ATen.h>
#include <ATen/record_function.h>
#include <c10/core/GradMode.h>

#include "abi_util.h"
#include "ops.h"

namespace recis {
namespace optim {

using namespace recis::hipabi;

namespace {

// What the two-input launches take for one gradient (recis_csr_input), with the host tables of a
// gradient that comes in parts kept alive beside it.
struct CsrInputHolder {
  recis_csr_input in{};
  std::vector<const void*> part_ptrs;
  std::vector<int64_t> part_counts;
  std::vector<at::Tensor> rows;  // contiguous versions, alive over the launch
};

void fill_input(const PlannedGrad& g, CsrInputHolder* h) {
  for (const auto& r : g.rows) {
    require_gpu(r, "gradient rows");
    TORCH_CHECK(r.dim() == 2, "gradient rows must be [rows, D]");
    h->rows.push_back(r.contiguous());
  }
  h->in.rows_dtype = dtype_code(h->rows[0].scalar_type());
  h->in.src = g.src.data_ptr<int32_t>();
  h->in.coef = g.coef.defined() ? g.coef.data_ptr() : nullptr;
  h->in.coef_dtype = g.coef.defined() ? dtype_code(g.coef.scalar_type()) : 0;
  if (g.in_parts) {
    for (const auto& r : h->rows) {
      h->part_ptrs.push_back(r.data_ptr());
      h->part_counts.push_back(r.size(0));
    }
    h->in.part_rows = h->part_ptrs.data();
    h->in.part_counts = h->part_counts.data();
    h->in.n_parts = static_cast<int>(h->rows.size());
  } else {
    h->in.rows = h->rows[0].data_ptr();
    h->in.n_rows = h->rows[0].size(0);
  }
}

struct PlannedHead {
  const PlannedGrad* g;
  at::Tensor rows, index;
  int64_t U, D;
};

// Checks shared by the one-input launches; U is the host's count when it has it, else a bound.
PlannedHead head_of(const PlannedGrad& g, const embedding::SlotPtr& emb) {
  PlannedHead h;
  h.g = &g;
  require_gpu(g.rows[0], "gradient rows");
  h.rows = g.rows[0].contiguous();
  TORCH_CHECK(h.rows.dim() == 2, "gradient rows must be [rows, D]");
  h.D = h.rows.size(1);
  TORCH_CHECK(h.D == emb->FlatSize(), "gradient rows have ", h.D, " columns, the table's rows ", emb->FlatSize());
  h.U = g.plan->U_bound();
  h.index = g.index;
  TORCH_CHECK(h.index.is_cuda() && h.index.scalar_type() == at::kLong && h.index.is_contiguous(),
              "row index must be a contiguous int64 GPU tensor");
  TORCH_CHECK(h.index.numel() >= h.U || h.index.numel() >= g.plan->U(), "row_index holds ", h.index.numel(),
              " rows for ", g.plan->U(), " unique ids");
  if (h.index.numel() < h.U) h.U = g.plan->U();
  return h;
}

}  // namespace

void SparseOptimizer::step() {
  c10::NoGradGuard no_grad;
  for (auto& p : params_) {
    if (!p.second.defined() || !p.second->has_grad()) continue;
    // the scope the reference opens around its update (csrc/embedding/adam.cc:128-131), so that
    // torch.profiler traces line up
    RECORD_FUNCTION(c10::str(Label(), "/", p.first, "/", "Update"), std::vector<c10::IValue>());
    if (grad_accum_steps_ == 1) {
      // the gradient is still a sum to be taken: sum and update in one launch
      std::vector<PlannedGrad> planned = p.second->TakePlannedGrad();
      if (!planned.empty()) {
        UpdatePlanned(p.second, planned);
        continue;
      }
    }
    auto pair = p.second->GradPairs(grad_accum_steps_);
    Update(p.second, std::get<0>(pair), std::get<1>(pair));
  }
}

void SparseOptimizer::add_parameters(const c10::Dict<std::string, HashTablePtr>& parameters) {
  // a Dict iterates in insertion order, so the slots of every table are appended in a fixed order
  for (const auto& item : parameters) {
    for (const auto& p : params_) {
      TORCH_CHECK(p.second.get() != item.value().get(), "some parameters appear in more than one parameter group.");
    }
    InitParamState(item.key(), item.value());
    params_.emplace_back(item.key(), item.value());
  }
}

void SparseOptimizer::zero_grad() {
  for (auto& p : params_) p.second->ClearGrad();
}

// ------------------------------------------------------------------------------------ Adam family
template <AdamDecay kDecay>
SparseAdamFamily<kDecay>::SparseAdamFamily(double lr, double beta1, double beta2, double eps, double weight_decay)
    : SparseOptimizer(lr), beta1_(beta1), beta2_(beta2), eps_(eps), weight_decay_(weight_decay) {
  TORCH_CHECK(lr >= 0, "Invalid learning rate: ", lr);
  TORCH_CHECK(eps >= 0, "Invalid epsilon value: ", eps);
  TORCH_CHECK(0 <= beta1 && beta1 < 1.0, "Invalid beta parameter at index 0: ", beta1);
  TORCH_CHECK(0 <= beta2 && beta2 < 1.0, "Invalid beta parameter at index 1: ", beta2);
  TORCH_CHECK(weight_decay >= 0, "Invalid weight_decay value: ", weight_decay);
}

template <AdamDecay kDecay>
c10::intrusive_ptr<SparseAdamFamily<kDecay>> SparseAdamFamily<kDecay>::Make(
    const c10::Dict<std::string, HashTablePtr>& hashtables, double lr, double beta1, double beta2, double eps,
    double weight_decay, bool amsgrad) {
  (void)amsgrad;  // carried by the reference's options and never read (csrc/embedding/adam.cc:55-74)
  auto opt = c10::make_intrusive<SparseAdamFamily<kDecay>>(lr, beta1, beta2, eps, weight_decay);
  opt->add_parameters(hashtables);
  return opt;
}

template <AdamDecay kDecay>
const char* SparseAdamFamily<kDecay>::Prefix() {
  return kDecay == AdamDecay::kNone ? "sparse_adam_" : kDecay == AdamDecay::kLrTimesWd ? "sparse_adamw_" : "sparse_adamw_tf_";
}

template <AdamDecay kDecay>
void SparseAdamFamily<kDecay>::InitParamState(const std::string& name, const HashTablePtr& table) {
  (void)name;
  auto sg = table->RawSlotGroup();
  AdamState st;
  // SparseAdam keeps its running beta powers in float64 (csrc/embedding/adam.h:37), the other two in
  // float32 scalars
  auto beta_opt = at::TensorOptions().device(table->device()).dtype(kDecay == AdamDecay::kNone ? at::kDouble : at::kFloat);
  std::vector<int64_t> beta_shape;
  if (kDecay == AdamDecay::kNone) beta_shape.push_back(1);
  st.beta1 = at::ones(beta_shape, beta_opt);
  st.beta2 = at::ones(beta_shape, beta_opt);
  st.step = at::zeros({1}, at::TensorOptions().device(table->device()).dtype(at::kLong));
  // the two moments live next to the parameter row they belong to
  auto moments = sg->AppendPackedSlots({std::string(Prefix()) + "exp_avg", std::string(Prefix()) + "exp_avg_sq"}, 0.0);
  st.exp_avg = moments[0];
  st.exp_avg_sq = moments[1];
  state_[table.get()] = st;
}

template <AdamDecay kDecay>
const char* SparseAdamFamily<kDecay>::Label() const {
  return kDecay == AdamDecay::kNone ? "FusedSparseAdam" : kDecay == AdamDecay::kLrTimesWd ? "FusedSparseAdamW"
                                                                                           : "FusedSparseAdamWTF";
}

// decay multiplier: 1 for SparseAdam (its weight_decay option is ignored, csrc/embedding/adam.cc:70-73),
// 1 - lr * wd for SparseAdamW (adamw.cc:64), 1 - wd for SparseAdamWTF (adamw_tf.cc:64)
template <AdamDecay kDecay>
double SparseAdamFamily<kDecay>::Decay() const {
  return kDecay == AdamDecay::kNone ? 1.0 : kDecay == AdamDecay::kLrTimesWd ? 1.0 - lr_ * weight_decay_
                                                                             : 1.0 - weight_decay_;
}

template <AdamDecay kDecay>
void SparseAdamFamily<kDecay>::Update(const HashTablePtr& table, const at::Tensor& index, const at::Tensor& grad) {
  auto emb = table->RawSlotGroup()->EmbSlot();
  AdamState& st = state_.at(table.get());
  recis::functional::block_apply_adamw(index, grad, emb->Chunks(), st.beta1, st.beta2, st.step, st.exp_avg->Chunks(),
                                       st.exp_avg_sq->Chunks(), lr_, beta1_, beta2_, Decay(), eps_, emb->ChunkRows());
}

template <AdamDecay kDecay>
void SparseAdamFamily<kDecay>::UpdatePlanned(const HashTablePtr& table, const std::vector<PlannedGrad>& planned) {
  auto emb = table->RawSlotGroup()->EmbSlot();
  AdamState& st = state_.at(table.get());
  c10::DeviceGuard guard(table->device());
  const auto& chunks = emb->Chunks();
  TORCH_CHECK(!chunks.empty() && st.exp_avg->Chunks().size() == chunks.size() &&
                  st.exp_avg_sq->Chunks().size() == chunks.size(),
              "state slots must have as many blocks as the embedding slot");
  at::Tensor t_emb = block_ptr_table(chunks), t_m = block_ptr_table(st.exp_avg->Chunks()),
             t_v = block_ptr_table(st.exp_avg_sq->Chunks());
  auto tab = [](const at::Tensor& t) { return reinterpret_cast<void* const*>(t.data_ptr()); };
  const int64_t n_blocks = static_cast<int64_t>(chunks.size());
  const int beta_f64 = st.beta1.scalar_type() == at::kDouble ? 1 : 0;
  const int64_t pitch = shared_row_pitch_bytes({&chunks[0], &st.exp_avg->Chunks()[0], &st.exp_avg_sq->Chunks()[0]});
  const BatchPlan& plan = *planned[0].plan;
  void* stream = stream_of(table->device());
  if (planned.size() == 1) {
    const PlannedHead h = head_of(planned[0], emb);
    const PlannedGrad& g = planned[0];
    check(recis_csr_gather_reduce_adamw(
        h.rows.data_ptr(), dtype_code(h.rows.scalar_type()), h.rows.size(0), g.src.data_ptr<int32_t>(),
        g.coef.defined() ? g.coef.data_ptr() : nullptr, g.coef.defined() ? dtype_code(g.coef.scalar_type()) : 0,
        plan.row_start().data_ptr<int32_t>(), plan.hot_items().data_ptr<int32_t>(), plan.hot_cap(),
        plan.counts().data_ptr<int64_t>(), h.U, h.D, g.cover.defined() ? g.cover.data_ptr() : nullptr,
        g.cover.defined() ? index_kind(g.cover, "offsets") : 0, g.cover.defined() ? g.cover.numel() - 1 : 0,
        h.index.data_ptr<int64_t>(), tab(t_emb), tab(t_m), tab(t_v), n_blocks, emb->ChunkRows(), pitch,
        dtype_code(emb->Dtype()), st.beta1.data_ptr(), st.beta2.data_ptr(), beta_f64, lr_, beta1_, beta2_, Decay(), eps_,
        stream));
    return;
  }
  CsrInputHolder a, b;
  fill_input(planned[0], &a);
  fill_input(planned[1], &b);
  const int64_t D = a.rows[0].size(1);
  TORCH_CHECK(b.rows[0].size(1) == D && D == emb->FlatSize(), "gradient rows and table rows differ in width");
  const int64_t U = std::min<int64_t>(plan.U_bound(), planned[0].index.numel());
  check(recis_csr_gather_reduce2_adamw(
      &a.in, &b.in, plan.row_start().data_ptr<int32_t>(), plan.hot_items().data_ptr<int32_t>(), plan.hot_cap(),
      plan.counts().data_ptr<int64_t>(), U, D, planned[0].index.data_ptr<int64_t>(), tab(t_emb), tab(t_m), tab(t_v),
      n_blocks, emb->ChunkRows(), pitch, dtype_code(emb->Dtype()), st.beta1.data_ptr(), st.beta2.data_ptr(), beta_f64,
      lr_, beta1_, beta2_, Decay(), eps_, stream));
}

template <AdamDecay kDecay>
std::tuple<c10::Dict<std::string, HashTablePtr>, c10::Dict<std::string, at::Tensor>>
SparseAdamFamily<kDecay>::state_dict() {
  c10::Dict<std::string, HashTablePtr> tables;
  c10::Dict<std::string, at::Tensor> steps;
  for (const auto& p : params_) {
    const AdamState& st = state_.at(p.second.get());
    // the names carry no table name in the reference either (csrc/embedding/adam.cc:88-96)
    steps.insert_or_assign(std::string(Prefix()) + "beta2", st.beta2);
    steps.insert_or_assign(std::string(Prefix()) + "beta1", st.beta1);
    steps.insert_or_assign(std::string(Prefix()) + "step", st.step);
  }
  return std::make_tuple(tables, steps);
}

template class SparseAdamFamily<AdamDecay::kNone>;
template class SparseAdamFamily<AdamDecay::kLrTimesWd>;
template class SparseAdamFamily<AdamDecay::kWd>;

// ------------------------------------------------------------------------------------ Adagrad
c10::intrusive_ptr<SparseAdagrad> SparseAdagrad::Make(const c10::Dict<std::string, HashTablePtr>& hashtables, double lr,
                                                      double eps) {
  auto opt = c10::make_intrusive<SparseAdagrad>(lr, eps);
  opt->add_parameters(hashtables);
  return opt;
}

void SparseAdagrad::InitParamState(const std::string& name, const HashTablePtr& table) {
  (void)name;
  auto sg = table->RawSlotGroup();
  accum_[table.get()] = sg->AppendPackedSlots({"sparse_adagrad_accum"}, 0.0)[0];
}

void SparseAdagrad::Update(const HashTablePtr& table, const at::Tensor& index, const at::Tensor& grad) {
  auto emb = table->RawSlotGroup()->EmbSlot();
  recis::functional::block_apply_adagrad(index, grad, emb->Chunks(), accum_.at(table.get())->Chunks(), lr_, eps_,
                                         emb->ChunkRows());
}

void SparseAdagrad::UpdatePlanned(const HashTablePtr& table, const std::vector<PlannedGrad>& planned) {
  auto emb = table->RawSlotGroup()->EmbSlot();
  auto accum = accum_.at(table.get());
  c10::DeviceGuard guard(table->device());
  const auto& chunks = emb->Chunks();
  TORCH_CHECK(!chunks.empty() && accum->Chunks().size() == chunks.size(),
              "state slot must have as many blocks as the embedding slot");
  at::Tensor t_emb = block_ptr_table(chunks), t_acc = block_ptr_table(accum->Chunks());
  auto tab = [](const at::Tensor& t) { return reinterpret_cast<void* const*>(t.data_ptr()); };
  const int64_t n_blocks = static_cast<int64_t>(chunks.size());
  const int64_t pitch = shared_row_pitch_bytes({&chunks[0], &accum->Chunks()[0]});
  const BatchPlan& plan = *planned[0].plan;
  void* stream = stream_of(table->device());
  if (planned.size() == 1) {
    const PlannedHead h = head_of(planned[0], emb);
    const PlannedGrad& g = planned[0];
    check(recis_csr_gather_reduce_adagrad(
        h.rows.data_ptr(), dtype_code(h.rows.scalar_type()), h.rows.size(0), g.src.data_ptr<int32_t>(),
        g.coef.defined() ? g.coef.data_ptr() : nullptr, g.coef.defined() ? dtype_code(g.coef.scalar_type()) : 0,
        plan.row_start().data_ptr<int32_t>(), plan.hot_items().data_ptr<int32_t>(), plan.hot_cap(),
        plan.counts().data_ptr<int64_t>(), h.U, h.D, g.cover.defined() ? g.cover.data_ptr() : nullptr,
        g.cover.defined() ? index_kind(g.cover, "offsets") : 0, g.cover.defined() ? g.cover.numel() - 1 : 0,
        h.index.data_ptr<int64_t>(), tab(t_emb), tab(t_acc), n_blocks, emb->ChunkRows(), pitch, dtype_code(emb->Dtype()),
        lr_, eps_, stream));
    return;
  }
  CsrInputHolder a, b;
  fill_input(planned[0], &a);
  fill_input(planned[1], &b);
  const int64_t D = a.rows[0].size(1);
  TORCH_CHECK(b.rows[0].size(1) == D && D == emb->FlatSize(), "gradient rows and table rows differ in width");
  const int64_t U = std::min<int64_t>(plan.U_bound(), planned[0].index.numel());
  check(recis_csr_gather_reduce2_adagrad(&a.in, &b.in, plan.row_start().data_ptr<int32_t>(),
                                         plan.hot_items().data_ptr<int32_t>(), plan.hot_cap(),
                                         plan.counts().data_ptr<int64_t>(), U, D, planned[0].index.data_ptr<int64_t>(),
                                         tab(t_emb), tab(t_acc), n_blocks, emb->ChunkRows(), pitch,
                                         dtype_code(emb->Dtype()), lr_, eps_, stream));
}

std::tuple<c10::Dict<std::string, HashTablePtr>, c10::Dict<std::string, at::Tensor>> SparseAdagrad::state_dict() {
  return std::make_tuple(c10::Dict<std::string, HashTablePtr>(), c10::Dict<std::string, at::Tensor>());
}

}  // namespace optim
}  // namespace recis
