// torch.classes.recis.{Generator, ChildrenInfo, Slot, SlotGroup, HashtableImpl}: the custom classes
// the reference registers at csrc/bind.cc:47-109, with GPU-resident storage behind the C ABI of
// librecis_hip.so. The key -> row map is a recis_idmap; every slot is a short list of large chunks,
// each a whole number of [block_size, D] blocks, which the row kernels address directly while
// Slot::values() hands out one aliasing view per block as the reference does.
#pragma once

#include <ATen/ATen.h>
#include <torch/custom_class.h>

#include <string>
#include <tuple>
#include <unordered_map>
#include <vector>

#include "recis_hip.h"

namespace recis {
namespace embedding {

// Row initialiser (csrc/embedding/initializer.h:15-66). One class for the whole family: the kind
// selects the distribution, the parameters are kept as C++ floats like the reference's members.
class Generator : public torch::CustomClassHolder {
 public:
  enum class Kind { kEmpty, kConstant, kUniform, kNormal, kXavierUniform, kXavierNormal, kKaimingUniform,
                    kKaimingNormal, kTruncNormal };
  Generator(Kind kind, const std::vector<int64_t>& shape, at::ScalarType dtype, double p0 = 0, double p1 = 0,
            double p2 = 0, double p3 = 0, bool fan_out = false, double gain = 1.0,
            c10::optional<at::Generator> rng = c10::nullopt);
  // A new tensor of `shape` (the generator's own shape when empty). Initialisers that depend on the
  // fans take them from fan_shape when given (callers that allocate several blocks in one tensor),
  // else from the generated shape.
  at::Tensor Generate(const std::vector<int64_t>& shape = {}, const std::vector<int64_t>& fan_shape = {});
  void set_device(at::Device device);
  const std::vector<int64_t>& Shape() const { return shape_; }
  at::TensorOptions TensorOption() const { return options_; }
  static at::Tensor DoGenerator(c10::intrusive_ptr<Generator> g) { return g->Generate(); }

 private:
  void Fill(at::Tensor& t, const std::vector<int64_t>& fan_shape);
  Kind kind_;
  std::vector<int64_t> shape_;
  at::TensorOptions options_;
  float p0_, p1_, p2_, p3_;
  bool fan_out_;
  double gain_;
  c10::optional<at::Generator> rng_;
};

using GeneratorPtr = c10::intrusive_ptr<Generator>;
GeneratorPtr MakeConstantGenerator(const std::vector<int64_t>& shape, at::ScalarType dtype, double init_val);
GeneratorPtr MakeUniformGenerator(const std::vector<int64_t>& shape, at::ScalarType dtype, double a, double b,
                                  c10::optional<at::Generator> generator);
GeneratorPtr MakeNormalGenerator(const std::vector<int64_t>& shape, at::ScalarType dtype, double mean, double std,
                                 c10::optional<at::Generator> generator);
GeneratorPtr MakeXavierUniFormGenerator(const std::vector<int64_t>& shape, at::ScalarType dtype, double gain,
                                        c10::optional<at::Generator> generator);
GeneratorPtr MakeXavierNormalGenerator(const std::vector<int64_t>& shape, at::ScalarType dtype, double gain,
                                       c10::optional<at::Generator> generator);
GeneratorPtr MakeKaimingUniformGenerator(const std::vector<int64_t>& shape, at::ScalarType dtype, double a,
                                         const std::string& mode_s, const std::string& nonlinearity_s,
                                         c10::optional<at::Generator> generator);
GeneratorPtr MakeKaimingNormalGenerator(const std::vector<int64_t>& shape, at::ScalarType dtype, double a,
                                        const std::string& mode_s, const std::string& nonlinearity_s,
                                        c10::optional<at::Generator> generator);
GeneratorPtr MakeTruncNormalGenerator(const std::vector<int64_t>& shape, at::ScalarType type, double mean,
                                      double std, double a, double b, c10::optional<at::Generator> generator);

// 12-bit table tag / 52-bit id packing of coalesced tables (csrc/embedding/children_info.h:12-37).
class ChildrenInfo : public torch::CustomClassHolder {
 public:
  ChildrenInfo(bool coalesce, const std::vector<std::string>& children);
  int64_t IndexBitsNum() const { return 12; }
  int64_t IdBitsNum() const { return 52; }
  int64_t IndexMask() const { return static_cast<int64_t>(~((uint64_t(1) << 52) - 1)); }
  int64_t IdMask() const { return (int64_t(1) << 52) - 1; }
  int64_t MaxChildrenNum() const { return 4095; }
  int64_t EncodeId(int64_t id, int64_t index) const;
  std::vector<std::string> Children() const { return children_; }
  int64_t ChildIndex(const std::string& name) const;
  bool HasChild(const std::string& name) const;
  std::string ChildAt(int64_t index) const;
  bool IsCoalesce() const { return coalesce_; }

 private:
  bool coalesce_;
  std::vector<std::string> children_;
};

// One named column of the table (csrc/embedding/slot_group.h:17-58).
class Slot : public torch::CustomClassHolder {
 public:
  Slot(const std::string& name, int64_t block_size, at::ScalarType dtype, const std::vector<int64_t>& partial_shape,
       GeneratorPtr generator, at::Device device, int64_t chunk_rows);
  int64_t BlockSize() const { return block_size_; }
  const std::string& Name() const { return name_; }
  int64_t FlatSize() const { return flat_size_; }
  at::ScalarType Dtype() const { return dtype_; }
  at::Tensor Value();                     // all visible rows in one tensor (a copy)
  std::vector<at::Tensor> ValuesDeref();  // one [block_size, D] view per block: aliases live storage
  at::Tensor IndexSelect(const at::Tensor& index, int64_t beg, int64_t end);
  void IndexInsert(const at::Tensor& index, at::Tensor value);
  void IndexInsert(const at::Tensor& index, at::Tensor value, const at::Tensor& accept_indicator);
  at::Tensor GenVal(int64_t rows);
  // what the row kernels take as (blocks, block_size)
  const std::vector<at::Tensor>& Chunks() const { return chunks_; }
  int64_t ChunkRows() const { return chunk_rows_; }
  void EnsureChunks(int64_t n_chunks);
  void SetVisibleBlocks(int64_t n) { visible_blocks_ = n; }
  void Clear();

 private:
  at::Tensor Conform(at::Tensor value) const;
  std::string name_;
  int64_t block_size_;
  at::ScalarType dtype_;
  std::vector<int64_t> row_shape_;
  GeneratorPtr generator_;
  at::Device device_;
  int64_t chunk_rows_;
  int64_t flat_size_;
  std::vector<at::Tensor> chunks_;
  int64_t visible_blocks_ = 0;
};

using SlotPtr = c10::intrusive_ptr<Slot>;

// All slots of one table; they grow together (csrc/embedding/slot_group.h:60-101).
class SlotGroup : public torch::CustomClassHolder {
 public:
  SlotGroup(int64_t block_size, at::Device device, int64_t chunk_rows);
  static const char* EmbSlotName() { return "embedding"; }
  SlotPtr AppendSlot(const std::string& name, at::ScalarType dtype, const std::vector<int64_t>& partial_shape,
                     GeneratorPtr generator);
  SlotPtr AppendSlot(const std::string& name, at::ScalarType dtype, const std::vector<int64_t>& partial_shape,
                     double init_val = 0.0);
  void AppendEmbSlot(at::ScalarType dtype, const std::vector<int64_t>& partial_shape, GeneratorPtr generator);
  void AppendStepFilterSlot(const std::string& name, int64_t init_step);
  SlotPtr GetSlotByName(const std::string& name);
  SlotPtr GetSlotByIndex(int64_t index);
  int64_t GetSlotIndex(const std::string& name);
  SlotPtr EmbSlot() { return GetSlotByIndex(emb_slot_index_); }
  std::vector<SlotPtr> Slots() { return slots_; }
  int64_t BlockSize() const { return block_size_; }
  int64_t BlockNum() const { return block_num_; }
  int64_t CapacityRows() const { return n_chunks_ * chunk_rows_; }
  int64_t ChunkRows() const { return chunk_rows_; }
  void EnsureRows(int64_t rows);
  void SetBlockNum(int64_t block_num);
  void Clear();

 private:
  int64_t block_size_;
  at::Device device_;
  int64_t chunk_rows_;
  int64_t emb_slot_index_ = -1;
  int64_t n_chunks_ = 0;
  int64_t block_num_ = 0;
  std::unordered_map<std::string, int64_t> name_to_index_;
  std::vector<SlotPtr> slots_;
};

}  // namespace embedding
}  // namespace recis

// The table itself (csrc/embedding/hashtable.h:30-113); registered as HashtableImpl.
class Hashtable : public torch::CustomClassHolder {
 public:
  const int64_t kNullIndex{-1};
  static c10::intrusive_ptr<Hashtable> Make(int64_t block_size, const std::vector<int64_t>& embedding_shape,
                                            at::ScalarType dtype, at::Device device, bool coalesce,
                                            const std::vector<std::string>& children,
                                            c10::intrusive_ptr<recis::embedding::Generator> generator,
                                            int64_t slice_begin, int64_t slice_end, int64_t slice_size);
  Hashtable(int64_t block_size, const std::vector<int64_t>& embedding_shape, at::ScalarType dtype, at::Device device,
            bool coalesce, const std::vector<std::string>& children,
            c10::intrusive_ptr<recis::embedding::Generator> generator, int64_t slice_begin, int64_t slice_end,
            int64_t slice_size);
  ~Hashtable() override;
  std::tuple<at::Tensor, at::Tensor> EmbeddingLookup(const at::Tensor& ids, bool readonly);
  at::Tensor InsertLookupIndex(const at::Tensor& ids);
  at::Tensor InsertLookupIndexWithIndicator(const at::Tensor& ids, const at::Tensor& indicator);
  at::Tensor LookupIndexReadOnly(const at::Tensor& ids);
  void Insert(const at::Tensor& ids, const at::Tensor& embedding);
  void UpdateSlot(const std::string& slot_name, const at::Tensor& index, at::Tensor value);
  void AppendStepFilterSlot(const std::string& filter_name, int64_t init_step);
  void AppendFilterSlot(const std::string& filter_name, at::ScalarType dtype, int64_t slot_dim,
                        c10::intrusive_ptr<recis::embedding::Generator> generator);
  void Clear();
  void ClearId();
  int64_t ids_num();
  at::Tensor ids();
  std::tuple<at::Tensor, at::Tensor> ids_map();
  void Delete(const at::Tensor& ids, const at::Tensor& index, const std::string& preserve_slot);
  bool has_grad() const { return !grad_.empty(); }
  void AcceptGrad(const at::Tensor& grad_index, const at::Tensor& grad);
  at::Tensor grad(int64_t accumulate_steps);
  // (row index, gradient rows) merged over the accepted gradients, duplicates summed per row: what
  // the sparse optimizers consume.
  std::tuple<at::Tensor, at::Tensor> GradPairs(int64_t accumulate_steps);
  void ClearGrad();
  c10::intrusive_ptr<recis::embedding::SlotGroup> SlotGroup();
  c10::intrusive_ptr<recis::embedding::SlotGroup> RawSlotGroup() { return slot_group_; }
  c10::intrusive_ptr<recis::embedding::ChildrenInfo> ChildrenInfo() { return children_info_; }
  c10::intrusive_ptr<recis::embedding::Slot> GetSlot(const std::string& name);
  std::vector<int64_t> SliceInfo() const { return {slice_begin_, slice_end_, slice_size_}; }
  at::Device device() const { return device_; }

 private:
  void MakeRoom(int64_t incoming);
  void SyncBlockNum();
  at::Tensor OnDevice(const at::Tensor& ids) const;
  at::Device device_;
  at::ScalarType dtype_;
  recis_idmap* id_map_ = nullptr;
  c10::intrusive_ptr<recis::embedding::SlotGroup> slot_group_;
  c10::intrusive_ptr<recis::embedding::ChildrenInfo> children_info_;
  int64_t slice_begin_, slice_end_, slice_size_;
  std::vector<at::Tensor> grad_index_;
  std::vector<at::Tensor> grad_;
};

using HashTablePtr = c10::intrusive_ptr<Hashtable>;
