// torch.classes.recis.{SparseAdam, SparseAdamW, SparseAdamWTF} (csrc/bind.cc:112-143; reference
// classes csrc/embedding/adam.h:69-117, adamw.h, adamw_tf.h, base csrc/embedding/optim.h:85-167),
// plus SparseAdagrad, an addition that follows the same conventions. State lives in extra slots of
// the table (same dtype and row shape as the embedding slot, zero initialised); one fused row
// kernel of librecis_hip.so updates the touched rows.
#pragma once

#include <ATen/core/Dict.h>

#include <string>
#include <tuple>
#include <unordered_map>
#include <vector>

#include "table.h"

namespace recis {
namespace optim {

class SparseOptimizer : public torch::CustomClassHolder {
 public:
  explicit SparseOptimizer(double lr) : lr_(lr) {}
  virtual ~SparseOptimizer() = default;
  void step();
  void add_parameters(const c10::Dict<std::string, HashTablePtr>& parameters);
  void zero_grad();
  void set_grad_accum_steps(int64_t steps) { grad_accum_steps_ = steps; }
  void set_lr(double lr) { lr_ = lr; }
  // the reference leaves this empty (csrc/embedding/adam.cc:210-212): slots come back with the table
  void load_state_dict(c10::Dict<std::string, HashTablePtr> hashtables, c10::Dict<std::string, at::Tensor> steps) {}

 protected:
  virtual void InitParamState(const std::string& name, const HashTablePtr& table) = 0;
  virtual void Update(const HashTablePtr& table, const at::Tensor& index, const at::Tensor& grad) = 0;
  // One optimizer step for `table` straight from gradients that are still sums to be taken (one, or
  // the two of one plan): the gradient of a unique id is summed over its occurrence list and applied
  // to its row by the lanes that summed it (recis_csr_gather_reduce*_adamw / _adagrad); the [U, D]
  // gradient is never written. Bit for bit what summing first and Update give.
  virtual void UpdatePlanned(const HashTablePtr& table, const std::vector<PlannedGrad>& planned) = 0;
  virtual const char* Label() const = 0;  // the name the profiler scope carries
  double lr_;
  int64_t grad_accum_steps_ = 1;
  std::vector<std::pair<std::string, HashTablePtr>> params_;  // in the order they were added
};

struct AdamState {
  at::Tensor beta1, beta2, step;
  embedding::SlotPtr exp_avg, exp_avg_sq;
};

// kDecay: how the weight_decay option enters the multiplicative decay of the row.
enum class AdamDecay { kNone, kLrTimesWd, kWd };

template <AdamDecay kDecay>
class SparseAdamFamily : public SparseOptimizer {
 public:
  SparseAdamFamily(double lr, double beta1, double beta2, double eps, double weight_decay);
  static c10::intrusive_ptr<SparseAdamFamily> Make(const c10::Dict<std::string, HashTablePtr>& hashtables, double lr,
                                                   double beta1, double beta2, double eps, double weight_decay,
                                                   bool amsgrad);
  std::tuple<c10::Dict<std::string, HashTablePtr>, c10::Dict<std::string, at::Tensor>> state_dict();

 protected:
  void InitParamState(const std::string& name, const HashTablePtr& table) override;
  void Update(const HashTablePtr& table, const at::Tensor& index, const at::Tensor& grad) override;
  void UpdatePlanned(const HashTablePtr& table, const std::vector<PlannedGrad>& planned) override;
  const char* Label() const override;
  static const char* Prefix();
  double Decay() const;

 private:
  double beta1_, beta2_, eps_, weight_decay_;
  std::unordered_map<Hashtable*, AdamState> state_;
};

using SparseAdam = SparseAdamFamily<AdamDecay::kNone>;
using SparseAdamW = SparseAdamFamily<AdamDecay::kLrTimesWd>;
using SparseAdamWTF = SparseAdamFamily<AdamDecay::kWd>;

class SparseAdagrad : public SparseOptimizer {
 public:
  SparseAdagrad(double lr, double eps) : SparseOptimizer(lr), eps_(eps) {}
  static c10::intrusive_ptr<SparseAdagrad> Make(const c10::Dict<std::string, HashTablePtr>& hashtables, double lr,
                                                double eps);
  std::tuple<c10::Dict<std::string, HashTablePtr>, c10::Dict<std::string, at::Tensor>> state_dict();

 protected:
  void InitParamState(const std::string& name, const HashTablePtr& table) override;
  void Update(const HashTablePtr& table, const at::Tensor& index, const at::Tensor& grad) override;
  void UpdatePlanned(const HashTablePtr& table, const std::vector<PlannedGrad>& planned) override;
  const char* Label() const override { return "FusedSparseAdagrad"; }

 private:
  double eps_;
  std::unordered_map<Hashtable*, embedding::SlotPtr> accum_;
};

}  // namespace optim
}  // namespace recis
