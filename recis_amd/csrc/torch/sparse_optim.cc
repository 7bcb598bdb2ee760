#include "sparse_optim.h"

#include <ATen/ATen.h>
#include <c10/core/GradMode.h>

#include "ops.h"

namespace recis {
namespace optim {

void SparseOptimizer::step() {
  c10::NoGradGuard no_grad;
  for (auto& p : params_) {
    if (!p.second.defined() || !p.second->has_grad()) continue;
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
  auto emb = sg->EmbSlot();
  auto blocks = emb->Chunks();
  std::vector<int64_t> partial{1};
  if (!blocks.empty()) {
    auto s = blocks[0].sizes();
    partial.insert(partial.end(), s.begin() + 1, s.end());
  } else {
    partial.push_back(emb->FlatSize());
  }
  AdamState st;
  // SparseAdam keeps its running beta powers in float64 (csrc/embedding/adam.h:37), the other two in
  // float32 scalars
  auto beta_opt = at::TensorOptions().device(table->device()).dtype(kDecay == AdamDecay::kNone ? at::kDouble : at::kFloat);
  std::vector<int64_t> beta_shape;
  if (kDecay == AdamDecay::kNone) beta_shape.push_back(1);
  st.beta1 = at::ones(beta_shape, beta_opt);
  st.beta2 = at::ones(beta_shape, beta_opt);
  st.step = at::zeros({1}, at::TensorOptions().device(table->device()).dtype(at::kLong));
  st.exp_avg = sg->AppendSlot(std::string(Prefix()) + "exp_avg", emb->Dtype(), partial, 0.0);
  st.exp_avg_sq = sg->AppendSlot(std::string(Prefix()) + "exp_avg_sq", emb->Dtype(), partial, 0.0);
  state_[table.get()] = st;
}

template <AdamDecay kDecay>
void SparseAdamFamily<kDecay>::Update(const HashTablePtr& table, const at::Tensor& index, const at::Tensor& grad) {
  auto emb = table->RawSlotGroup()->EmbSlot();
  AdamState& st = state_.at(table.get());
  // decay multiplier: 1 for SparseAdam (its weight_decay option is ignored, csrc/embedding/adam.cc:70-73),
  // 1 - lr * wd for SparseAdamW (adamw.cc:64), 1 - wd for SparseAdamWTF (adamw_tf.cc:64)
  const double decay = kDecay == AdamDecay::kNone ? 1.0 : kDecay == AdamDecay::kLrTimesWd ? 1.0 - lr_ * weight_decay_
                                                                                           : 1.0 - weight_decay_;
  recis::functional::block_apply_adamw(index, grad, emb->Chunks(), st.beta1, st.beta2, st.step, st.exp_avg->Chunks(),
                                       st.exp_avg_sq->Chunks(), lr_, beta1_, beta2_, decay, eps_, emb->ChunkRows());
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
  auto emb = sg->EmbSlot();
  std::vector<int64_t> partial{1};
  auto blocks = emb->Chunks();
  if (!blocks.empty()) {
    auto s = blocks[0].sizes();
    partial.insert(partial.end(), s.begin() + 1, s.end());
  } else {
    partial.push_back(emb->FlatSize());
  }
  accum_[table.get()] = sg->AppendSlot("sparse_adagrad_accum", emb->Dtype(), partial, 0.0);
}

void SparseAdagrad::Update(const HashTablePtr& table, const at::Tensor& index, const at::Tensor& grad) {
  auto emb = table->RawSlotGroup()->EmbSlot();
  recis::functional::block_apply_adagrad(index, grad, emb->Chunks(), accum_.at(table.get())->Chunks(), lr_, eps_,
                                         emb->ChunkRows());
}

std::tuple<c10::Dict<std::string, HashTablePtr>, c10::Dict<std::string, at::Tensor>> SparseAdagrad::state_dict() {
  return std::make_tuple(c10::Dict<std::string, HashTablePtr>(), c10::Dict<std::string, at::Tensor>());
}

}  // namespace optim
}  // namespace recis
