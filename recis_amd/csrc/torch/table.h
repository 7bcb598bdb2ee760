// torch.classes.recis.{Generator, ChildrenInfo, Slot, SlotGroup, HashtableImpl}: the custom classes
// the reference registers at csrc/bind.cc:47-109, with GPU-resident storage behind the C ABI of
// librecis_hip.so. The key -> row map is a recis_idmap; every slot is a short list of large chunks,
// each a whole number of [block_size, D] blocks, which the row kernels address directly while
// Slot::values() hands out one aliasing view per block as the reference does.
#pragma once

#include <ATen/ATen.h>
#include <torch/custom_class.h>

#include <memory>
#include <string>
#include <tuple>
#include <unordered_map>
#include <vector>

#include "plan.h"
#include "recis_hip.h"

namespace recis {
namespace embedding {

// Row initialiser (csrc/embedding/initializer.h:15-66). One class for the whole family: the kind
// selects the distribution, the parameters are kept as C++ floats like the reference's members.
class Generator : public torch::CustomClassHolder {
 public:
  enum class Kind { kEmpty, kConstant, kUniform, kNormal, kXavierUniform, kXavierNormal, kKaimingUniform,
                    kKaimingNormal, kTruncNormal, kFromTensor };
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
  // kFromTensor: the rows are handed out from `source`, in order, starting over at its end.
  void SetSource(at::Tensor source) { source_ = std::move(source); }

 private:
  void Fill(at::Tensor& t, const std::vector<int64_t>& fan_shape);
  Kind kind_;
  std::vector<int64_t> shape_;
  at::TensorOptions options_;
  float p0_, p1_, p2_, p3_;
  bool fan_out_;
  double gain_;
  c10::optional<at::Generator> rng_;
  at::Tensor source_;
  int64_t cursor_ = 0;
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
// An addition: rows taken from a given [rows, D...] tensor, in order (tables that start from rows the
// caller already has, e.g. the parity tests that give both sides the same storage).
GeneratorPtr MakeTensorGenerator(const std::vector<int64_t>& shape, at::ScalarType dtype, at::Tensor source);

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

// The key -> row map of one table. Shared by the table and its slots, so that a slot handle that
// outlives a lookup (or the table object) still knows how many rows the table holds.
struct IdMapHolder {
  explicit IdMapHolder(recis_idmap* m, at::Device d) : map(m), device(d) {}
  ~IdMapHolder();
  IdMapHolder(const IdMapHolder&) = delete;
  IdMapHolder& operator=(const IdMapHolder&) = delete;
  int64_t IdNum() const;  // the allocator's high-water mark; waits for the stream
  recis_idmap* map;
  at::Device device;
};

// One named column of the table (csrc/embedding/slot_group.h:17-58).
class Slot : public torch::CustomClassHolder {
 public:
  Slot(const std::string& name, int64_t block_size, at::ScalarType dtype, const std::vector<int64_t>& partial_shape,
       GeneratorPtr generator, at::Device device, int64_t chunk_rows, std::shared_ptr<IdMapHolder> map);
  int64_t BlockSize() const { return block_size_; }
  const std::string& Name() const { return name_; }
  int64_t FlatSize() const { return flat_size_; }
  at::ScalarType Dtype() const { return dtype_; }
  std::vector<int64_t> RowShape() const { return row_shape_; }
  at::Tensor Value();                     // all visible rows in one tensor (a copy)
  std::vector<at::Tensor> ValuesDeref();  // one [block_size, D] view per block: aliases live storage
  at::Tensor IndexSelect(const at::Tensor& index, int64_t beg, int64_t end);
  void IndexInsert(const at::Tensor& index, at::Tensor value);
  void IndexInsert(const at::Tensor& index, at::Tensor value, const at::Tensor& accept_indicator);
  at::Tensor GenVal(int64_t rows);
  // what the row kernels take as (blocks, block_size)
  const std::vector<at::Tensor>& Chunks() const { return chunks_; }
  int64_t ChunkRows() const { return chunk_rows_; }
  void SetChunkRows(int64_t chunk_rows);  // only while no storage exists
  void EnsureChunks(int64_t n_chunks);    // (a slot that owns its storage)
  void Clear();
  // A slot whose rows live in an allocation it shares with other slots of the table (see
  // SlotGroup::AppendPackedSlots): the group hands it one strided [chunk_rows, D] view per chunk.
  bool Packed() const { return packed_; }
  void SetPacked() { packed_ = true; }
  at::Tensor NewChunkValues();  // initial values of one chunk, from the slot's generator
  void SetChunk(int64_t c, at::Tensor view);  // replaces chunk c, or appends it when c == Chunks().size()

 private:
  // block_num = (id_num + block_size) / block_size (csrc/embedding/hashtable.cc:255-261), read from
  // the id map at the time of the call: the reference's values() grows with every lookup, so a handle
  // taken before an insert must see the blocks the insert added.
  int64_t VisibleBlocks() const;
  at::Tensor Conform(at::Tensor value) const;
  std::string name_;
  int64_t block_size_;
  at::ScalarType dtype_;
  std::vector<int64_t> row_shape_;
  GeneratorPtr generator_;
  at::Device device_;
  int64_t chunk_rows_;
  int64_t flat_size_;
  std::shared_ptr<IdMapHolder> map_;
  std::vector<at::Tensor> chunks_;
  bool packed_ = false;
};

using SlotPtr = c10::intrusive_ptr<Slot>;

// All slots of one table; they grow together (csrc/embedding/slot_group.h:60-101).
class SlotGroup : public torch::CustomClassHolder {
 public:
  SlotGroup(int64_t block_size, at::Device device, int64_t chunk_rows, std::shared_ptr<IdMapHolder> map);
  static const char* EmbSlotName() { return "embedding"; }
  SlotPtr AppendSlot(const std::string& name, at::ScalarType dtype, const std::vector<int64_t>& partial_shape,
                     GeneratorPtr generator);
  SlotPtr AppendSlot(const std::string& name, at::ScalarType dtype, const std::vector<int64_t>& partial_shape,
                     double init_val = 0.0);
  void AppendEmbSlot(at::ScalarType dtype, const std::vector<int64_t>& partial_shape, GeneratorPtr generator);
  // Appends constant-initialised slots of the embedding's dtype and row shape (an optimizer's
  // state). With RECIS_PACKED_STATE=1 in the environment they share one allocation with the
  // embedding slot: row r of a chunk holds emb | state 0 | state 1 ... back to back, so the rows one
  // key's update touches lie in the same cache lines and DRAM page. Every slot still answers
  // values() / index_select / index_insert as before; its blocks are strided views. Storage that
  // exists is moved into the new layout chunk by chunk: views handed out earlier keep the old memory
  // and no longer alias the table.
  // The default is the reference's layout, one array per slot (csrc/embedding/slot_group.cc:40-75),
  // because that measured no slower: the fused update is bound by the loads each wave keeps in
  // flight, not by the lines it touches (D = 16 fp32, 2e8-row table: update 106 vs 112 us, but the
  // forward expansion 91 vs 85 us, its 64-byte rows no longer sharing 128-byte lines with their
  // neighbours; densely touched tables fetch 6 % more).
  std::vector<SlotPtr> AppendPackedSlots(const std::vector<std::string>& names, double init_val);
  void AppendStepFilterSlot(const std::string& name, int64_t init_step);
  SlotPtr GetSlotByName(const std::string& name);
  SlotPtr GetSlotByIndex(int64_t index);
  int64_t GetSlotIndex(const std::string& name);
  bool HasSlot(const std::string& name) const { return name_to_index_.count(name) > 0; }
  SlotPtr EmbSlot() { return GetSlotByIndex(emb_slot_index_); }
  std::vector<SlotPtr> Slots() { return slots_; }
  int64_t BlockSize() const { return block_size_; }
  int64_t BlockNum() const;
  int64_t CapacityRows() const { return n_chunks_ * chunk_rows_; }
  int64_t ChunkRows() const { return chunk_rows_; }
  void SetChunkRows(int64_t chunk_rows);  // only while no storage exists
  void EnsureRows(int64_t rows);
  void Clear();

 private:
  int64_t block_size_;
  at::Device device_;
  int64_t chunk_rows_;
  std::shared_ptr<IdMapHolder> map_;
  int64_t emb_slot_index_ = -1;
  int64_t n_chunks_ = 0;
  std::unordered_map<std::string, int64_t> name_to_index_;
  std::vector<SlotPtr> slots_;
  // the slots that share an allocation (the embedding slot first) and that allocation's chunks,
  // [chunk_rows, packed_.size() * D] each
  at::Tensor PackedView(const at::Tensor& store, int64_t member, int64_t members, const SlotPtr& slot) const;
  void AddPackedChunk();
  std::vector<int64_t> packed_;
  std::vector<at::Tensor> packed_chunks_;
};

}  // namespace embedding
}  // namespace recis

// A gradient handed to the table before it is summed: the gradient of unique id u of `plan` (table
// row index[u]; negative = the table does not hold the key) is the sum over u's occurrence list of
// coef * rows[src].
struct PlannedGrad {
  at::Tensor index;
  recis::BatchPlanPtr plan;
  std::vector<at::Tensor> rows;  // one array, or (in_parts) several laid end to end in src's numbering
  bool in_parts = false;
  at::Tensor src, coef, cover;   // coef / cover may be undefined
  int64_t key = 0;               // 0 = none
  bool may_miss = false;
};

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
  // ---- the reference's surface (csrc/bind.cc:92-109)
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
  bool has_grad() const { return !grad_.empty() || !planned_.empty(); }
  void AcceptGrad(const at::Tensor& grad_index, const at::Tensor& grad);
  at::Tensor grad(int64_t accumulate_steps);
  // (row index, gradient rows) merged over the accepted gradients, duplicates summed per row: what
  // the sparse optimizers consume.
  std::tuple<at::Tensor, at::Tensor> GradPairs(int64_t accumulate_steps);
  void ClearGrad();
  c10::intrusive_ptr<recis::embedding::SlotGroup> SlotGroup() { return slot_group_; }
  c10::intrusive_ptr<recis::embedding::SlotGroup> RawSlotGroup() { return slot_group_; }
  c10::intrusive_ptr<recis::embedding::ChildrenInfo> ChildrenInfo() { return children_info_; }
  c10::intrusive_ptr<recis::embedding::Slot> GetSlot(const std::string& name);
  std::vector<int64_t> SliceInfo() const { return {slice_begin_, slice_end_, slice_size_}; }
  at::Device device() const { return device_; }
  at::ScalarType dtype() const { return dtype_; }
  std::vector<int64_t> EmbeddingShape() const { return embedding_shape_; }

  // ---- additions: pre-sizing, the batch plan, gradients handed over unsummed, the fused sweep
  // Pre-sizes the id map and makes the row storage grow in one chunk of at least `rows` rows per
  // slot; before the table holds any row.
  void Reserve(int64_t rows);
  // Dedup of `ids` (a list of id tensors laid end to end, tagged with `tags` as ids_encode does) and
  // find-or-insert of the distinct ids in one pass (recis_unique_plan_jobs): the plan's index_buf
  // holds the row of every unique id. Replaces ids_partition / torch.unique + IdMap::Lookup of the
  // training lookup (recis/nn/modules/hashtable.py:262-293). Room is made for the rows every id of
  // the batch could need (wait == false) or for the distinct ids (wait == true).
  recis::BatchPlanPtr PlanLookup(const std::vector<at::Tensor>& ids, const c10::optional<std::vector<int64_t>>& tags,
                                 bool wait, bool need_inverse, bool need_pos);
  // The rows of `plan`'s unique ids if PlanLookup of THIS table made it (the full-length buffer: its
  // first plan.U entries count), else None.
  c10::optional<at::Tensor> PlanIndex(const recis::BatchPlanPtr& plan);
  // Find-or-insert of a plan's unique ids queued before the host knows how many there are; returns
  // the full-length index buffer. `make_room`: room for the rows every id of the plan could need.
  at::Tensor LookupIndexCounted(const recis::BatchPlanPtr& plan, bool make_room);
  void SettleCount(int64_t n_true, const c10::optional<recis::BatchPlanPtr>& plan);
  at::Tensor SettleLookup(const at::Tensor& index_buf, int64_t n_true, const recis::BatchPlanPtr& plan);
  at::Tensor LookupIndex(const at::Tensor& ids, bool readonly);
  // out[i] = weight[i] * row(unique id of occurrence i): every unique row is read once out of the
  // blocks and written to all its occurrences (recis_csr_expand_rows_stamped). `stamp_slot` +
  // `stamp_value` (one int64 on the device): the rows read also get that value in that int64 slot.
  at::Tensor ExpandRows(const recis::BatchPlanPtr& plan, const at::Tensor& row_index,
                        const c10::optional<at::Tensor>& weight, const c10::optional<std::string>& stamp_slot,
                        const c10::optional<at::Tensor>& stamp_value);
  // PlanLookup + ExpandRows for a group of dense id columns ([B] or [B, 1] int64 GPU tensors, one id
  // per sample: every segment holds one id, so sum == mean == the row itself) in ONE call from
  // Python: (plan, full-length row index, [N, D] rows, column after column). None when a column is
  // something else (the caller then takes the general path).
  c10::optional<std::tuple<recis::BatchPlanPtr, at::Tensor, at::Tensor>> DenseLookupExpand(
      const std::vector<at::Tensor>& cols, const c10::optional<std::vector<int64_t>>& tags,
      const c10::optional<std::string>& stamp_slot, const c10::optional<at::Tensor>& stamp_value);
  // The backward of an output that was handed out in parts (`split` rows each): `grads` are the parts'
  // gradients as autograd delivers them (None = zeros). Consecutive slices of one buffer are used in
  // place, anything else is concatenated; then the count of `plan` is settled (`settle`) and the
  // gradient accepted unsummed (AcceptPlannedGrad with src / coef; src undefined = the occurrence
  // itself, one id per segment).
  void AcceptSplitGrad(const at::Tensor& index, const recis::BatchPlanPtr& plan,
                       const std::vector<c10::optional<at::Tensor>>& grads, const std::vector<int64_t>& split,
                       const c10::optional<at::Tensor>& src, const c10::optional<at::Tensor>& coef, int64_t key,
                       bool may_miss, bool settle);
  // accept_grad whose caller knows that grad_index has no duplicates (`unique`), and / or that two
  // calls with one `key` (!= 0) hand over gradients for the same rows in the same order (the second
  // is then added onto the first).
  void AcceptGradEx(const at::Tensor& grad_index, const at::Tensor& grad, bool unique, int64_t key);
  // See PlannedGrad. If it stays the only gradient of the step (or one of the two of one plan and
  // key), an optimizer that can sums it and applies the row update in one launch; anything else that
  // asks for the gradient gets it summed first.
  void AcceptPlannedGrad(const at::Tensor& index, const recis::BatchPlanPtr& plan, const std::vector<at::Tensor>& rows,
                         bool in_parts, const at::Tensor& src, const c10::optional<at::Tensor>& coef,
                         const c10::optional<at::Tensor>& cover, int64_t key, bool may_miss);
  // The planned gradients if they are all this table received since the last ClearGrad (and forgets
  // them), else empty: one or two entries; of two, the first is one array.
  std::vector<PlannedGrad> TakePlannedGrad();
  // [gradients waiting unsummed, gradients held summed]
  std::vector<int64_t> PendingGrads() const {
    return {static_cast<int64_t>(planned_.size()), static_cast<int64_t>(grad_.size())};
  }
  // Eviction sweep in one pass over the map: erase every key whose row has stamp_slot < threshold,
  // free the rows, re-initialise every other slot there; returns the evicted (ids, index).
  std::tuple<at::Tensor, at::Tensor> EvictOlder(const std::string& stamp_slot, int64_t threshold);
  // (live keys, allocator high-water mark, free-list length, slot capacity); waits for the stream
  std::vector<int64_t> IdMapStats();
  recis_idmap* id_map() const { return map_->map; }

 private:
  void MakeRoom(int64_t incoming);
  at::Tensor OnDevice(const at::Tensor& ids) const;
  bool OneLaunchSums(const PlannedGrad& a, const PlannedGrad& b) const;
  at::Tensor SumOf(const PlannedGrad& g) const;
  void AcceptSummed(const PlannedGrad& g, at::Tensor summed);
  void SumPlanned();
  at::Device device_;
  at::ScalarType dtype_;
  std::vector<int64_t> embedding_shape_;
  std::shared_ptr<recis::embedding::IdMapHolder> map_;
  c10::intrusive_ptr<recis::embedding::SlotGroup> slot_group_;
  c10::intrusive_ptr<recis::embedding::ChildrenInfo> children_info_;
  int64_t slice_begin_, slice_end_, slice_size_;
  std::vector<at::Tensor> grad_index_;
  std::vector<at::Tensor> grad_;
  std::vector<bool> grad_unique_;
  std::vector<std::pair<int64_t, size_t>> grad_keys_;
  std::vector<PlannedGrad> planned_;
  // the index tensor the last embedding_lookup returned, and whether the ids it was given are
  // known to hold no duplicates (they came out of ids_partition): accept_grad of exactly that tensor
  // needs no dedup
  at::Tensor last_lookup_index_;
  bool last_lookup_unique_ = false;
};

using HashTablePtr = c10::intrusive_ptr<Hashtable>;
