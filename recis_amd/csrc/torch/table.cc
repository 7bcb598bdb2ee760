#include "table.h"

#include <cmath>

#include "abi_util.h"
#include "ops.h"

using recis::hipabi::check;
using recis::hipabi::stream_of;

namespace recis {
namespace embedding {

// ------------------------------------------------------------------------------------ Generator
Generator::Generator(Kind kind, const std::vector<int64_t>& shape, at::ScalarType dtype, double p0, double p1,
                     double p2, double p3, bool fan_out, double gain, c10::optional<at::Generator> rng)
    : kind_(kind),
      shape_(shape),
      options_(at::TensorOptions().device(at::kCPU).dtype(dtype)),
      p0_(static_cast<float>(p0)),
      p1_(static_cast<float>(p1)),
      p2_(static_cast<float>(p2)),
      p3_(static_cast<float>(p3)),
      fan_out_(fan_out),
      gain_(gain),
      rng_(std::move(rng)) {}

void Generator::set_device(at::Device device) {
  options_ = options_.device(device);
  TORCH_CHECK(!rng_.has_value() || rng_->device().type() == device.type(), "the torch.Generator of this initialiser lives on ",
              rng_->device(), " but the rows are drawn on ", device, ": pass a generator of the table's device");
}

at::Tensor Generator::Generate(const std::vector<int64_t>& shape, const std::vector<int64_t>& fan_shape) {
  const std::vector<int64_t>& used = shape.empty() ? shape_ : shape;
  at::Tensor t = at::empty(used, options_);
  if (t.numel()) Fill(t, fan_shape.empty() ? used : fan_shape);
  return t;
}

namespace {
// fan_in / fan_out as torch::nn::init computes them for a tensor of this shape.
void fans(const std::vector<int64_t>& shape, double* fan_in, double* fan_out) {
  TORCH_CHECK(shape.size() >= 2, "Fan in and fan out can not be computed for tensor with fewer than 2 dimensions");
  int64_t receptive = 1;
  for (size_t d = 2; d < shape.size(); ++d) receptive *= shape[d];
  *fan_in = static_cast<double>(shape[1] * receptive);
  *fan_out = static_cast<double>(shape[0] * receptive);
}

float normal_cdf(float x) { return static_cast<float>((1.0 + std::erf(x / std::sqrt(2.0))) / 2.0); }
}  // namespace

// Each branch performs the arithmetic of the torch call the reference makes (initializer.cc:26-230),
// in its order of operations, so that the same RNG state gives the same rows.
void Generator::Fill(at::Tensor& t, const std::vector<int64_t>& fan_shape) {
  double fan_in = 0, fan_out = 0;
  switch (kind_) {
    case Kind::kEmpty:
      return;
    case Kind::kConstant:
      if (at::isIntegralType(t.scalar_type(), true)) {
        t.fill_(static_cast<int64_t>(p0_));
      } else {
        t.fill_(p0_);
      }
      return;
    case Kind::kUniform:
      t.uniform_(p0_, p1_, rng_);
      return;
    case Kind::kNormal:
      t.normal_(p0_, p1_, rng_);
      return;
    case Kind::kXavierUniform: {
      fans(fan_shape, &fan_in, &fan_out);
      const double std = p0_ * std::sqrt(2.0 / (fan_in + fan_out));
      const double a = std::sqrt(3.0) * std;
      t.uniform_(-a, a);
      return;
    }
    case Kind::kXavierNormal: {
      fans(fan_shape, &fan_in, &fan_out);
      t.normal_(0, p0_ * std::sqrt(2.0 / (fan_in + fan_out)));
      return;
    }
    case Kind::kKaimingUniform:
    case Kind::kKaimingNormal: {
      fans(fan_shape, &fan_in, &fan_out);
      const double std = gain_ / std::sqrt(fan_out_ ? fan_out : fan_in);
      if (kind_ == Kind::kKaimingUniform) {
        const double bound = std::sqrt(3.0) * std;
        t.uniform_(-bound, bound);
      } else {
        t.normal_(0, std);
      }
      return;
    }
    case Kind::kTruncNormal: {
      // inverse-CDF sampling between the absolute bounds p2_ (a) and p3_ (b); p0_ = mean, p1_ = std
      const float l = normal_cdf((p2_ - p0_) / p1_);
      const float u = normal_cdf((p3_ - p0_) / p1_);
      t.uniform_(2 * l - 1, 2 * u - 1, rng_);
      t.erfinv_();
      t.mul_(p1_ * std::sqrt(2.0));
      t.add_(p0_);
      t.clamp_(p2_, p3_);
      return;
    }
  }
}

GeneratorPtr MakeConstantGenerator(const std::vector<int64_t>& shape, at::ScalarType dtype, double init_val) {
  return c10::make_intrusive<Generator>(Generator::Kind::kConstant, shape, dtype, init_val);
}
GeneratorPtr MakeUniformGenerator(const std::vector<int64_t>& shape, at::ScalarType dtype, double a, double b,
                                  c10::optional<at::Generator> generator) {
  return c10::make_intrusive<Generator>(Generator::Kind::kUniform, shape, dtype, a, b, 0, 0, false, 1.0, generator);
}
GeneratorPtr MakeNormalGenerator(const std::vector<int64_t>& shape, at::ScalarType dtype, double mean, double std,
                                 c10::optional<at::Generator> generator) {
  return c10::make_intrusive<Generator>(Generator::Kind::kNormal, shape, dtype, mean, std, 0, 0, false, 1.0, generator);
}
GeneratorPtr MakeXavierUniFormGenerator(const std::vector<int64_t>& shape, at::ScalarType dtype, double gain,
                                        c10::optional<at::Generator> generator) {
  return c10::make_intrusive<Generator>(Generator::Kind::kXavierUniform, shape, dtype, gain, 0, 0, 0, false, 1.0,
                                        generator);
}
GeneratorPtr MakeXavierNormalGenerator(const std::vector<int64_t>& shape, at::ScalarType dtype, double gain,
                                       c10::optional<at::Generator> generator) {
  return c10::make_intrusive<Generator>(Generator::Kind::kXavierNormal, shape, dtype, gain, 0, 0, 0, false, 1.0,
                                        generator);
}

namespace {
bool fan_mode_is_out(const std::string& mode) {
  TORCH_CHECK(mode == "fan_in" || mode == "fan_out", mode, " not in [fan_in, fan_out]");
  return mode == "fan_out";
}

// torch::nn::init::calculate_gain for the names the reference accepts (its spellings included,
// initializer.cc:232-265); `a` is rounded to float first, as the reference's member is.
double gain_of(const std::string& nonlinearity, double a) {
  static const char* unit[] = {"liner", "conv_1d", "conv_2d", "conv_3d", "conv_transpose_1d", "conv_transpose_2d",
                               "conv_transpose_3d", "sigmod"};
  for (const char* name : unit) {
    if (nonlinearity == name) return 1.0;
  }
  if (nonlinearity == "tanh") return 5.0 / 3.0;
  if (nonlinearity == "relu") return std::sqrt(2.0);
  if (nonlinearity == "leaky_relu") {
    const double slope = static_cast<float>(a);
    return std::sqrt(2.0 / (1 + std::pow(slope, 2)));
  }
  TORCH_CHECK(false, nonlinearity,
              " not in  [liner, conv_1d, conv_2d, cond3d, conv_transpose_1d, conv_transpose_2d, conv_transpose_3d,"
              "sigmod, tanh, relu, leaky_relu]");
}
}  // namespace

GeneratorPtr MakeKaimingUniformGenerator(const std::vector<int64_t>& shape, at::ScalarType dtype, double a,
                                         const std::string& mode_s, const std::string& nonlinearity_s,
                                         c10::optional<at::Generator> generator) {
  return c10::make_intrusive<Generator>(Generator::Kind::kKaimingUniform, shape, dtype, a, 0, 0, 0,
                                        fan_mode_is_out(mode_s), gain_of(nonlinearity_s, a), generator);
}
GeneratorPtr MakeKaimingNormalGenerator(const std::vector<int64_t>& shape, at::ScalarType dtype, double a,
                                        const std::string& mode_s, const std::string& nonlinearity_s,
                                        c10::optional<at::Generator> generator) {
  return c10::make_intrusive<Generator>(Generator::Kind::kKaimingNormal, shape, dtype, a, 0, 0, 0,
                                        fan_mode_is_out(mode_s), gain_of(nonlinearity_s, a), generator);
}
GeneratorPtr MakeTruncNormalGenerator(const std::vector<int64_t>& shape, at::ScalarType type, double mean,
                                      double std, double a, double b, c10::optional<at::Generator> generator) {
  return c10::make_intrusive<Generator>(Generator::Kind::kTruncNormal, shape, type, mean, std, a, b, false, 1.0,
                                        generator);
}

// ------------------------------------------------------------------------------------ ChildrenInfo
ChildrenInfo::ChildrenInfo(bool coalesce, const std::vector<std::string>& children)
    : coalesce_(coalesce), children_(children) {
  TORCH_CHECK(static_cast<int64_t>(children_.size()) <= MaxChildrenNum(), "too many children: ", children_.size());
  TORCH_CHECK(coalesce_ || children_.size() == 1, "a table that is not coalesced has exactly one child, got ",
              children_.size());
}

int64_t ChildrenInfo::EncodeId(int64_t id, int64_t index) const {
  return static_cast<int64_t>((static_cast<uint64_t>(id) & static_cast<uint64_t>(IdMask())) |
                              (static_cast<uint64_t>(index) << 52));
}

int64_t ChildrenInfo::ChildIndex(const std::string& name) const {
  for (size_t i = 0; i < children_.size(); ++i) {
    if (children_[i] == name) return static_cast<int64_t>(i);
  }
  TORCH_CHECK(false, "no child named ", name);
}

bool ChildrenInfo::HasChild(const std::string& name) const {
  for (const auto& c : children_) {
    if (c == name) return true;
  }
  return false;
}

std::string ChildrenInfo::ChildAt(int64_t index) const {
  TORCH_CHECK(index >= 0 && index < static_cast<int64_t>(children_.size()), "child index ", index, " out of range");
  return children_[index];
}

// ------------------------------------------------------------------------------------ Slot
Slot::Slot(const std::string& name, int64_t block_size, at::ScalarType dtype,
           const std::vector<int64_t>& partial_shape, GeneratorPtr generator, at::Device device, int64_t chunk_rows)
    : name_(name),
      block_size_(block_size),
      dtype_(dtype),
      row_shape_(partial_shape.begin() + (partial_shape.empty() ? 0 : 1), partial_shape.end()),
      generator_(std::move(generator)),
      device_(device),
      chunk_rows_(chunk_rows),
      flat_size_(1) {
  for (int64_t d : row_shape_) flat_size_ *= d;
  generator_->set_device(device);
}

std::vector<at::Tensor> Slot::ValuesDeref() {
  const int64_t per = chunk_rows_ / block_size_;
  std::vector<at::Tensor> out;
  out.reserve(visible_blocks_);
  for (int64_t b = 0; b < visible_blocks_; ++b) {
    out.push_back(chunks_[b / per].narrow(0, (b % per) * block_size_, block_size_));
  }
  return out;
}

at::Tensor Slot::Value() {
  const int64_t rows = visible_blocks_ * block_size_;
  std::vector<int64_t> shape{0};
  shape.insert(shape.end(), row_shape_.begin(), row_shape_.end());
  if (rows == 0) return at::empty(shape, at::TensorOptions().dtype(dtype_).device(device_));
  std::vector<at::Tensor> parts;
  const int64_t full = rows / chunk_rows_, rest = rows % chunk_rows_;
  for (int64_t c = 0; c < full; ++c) parts.push_back(chunks_[c]);
  if (rest) parts.push_back(chunks_[full].narrow(0, 0, rest));
  return at::cat(parts, 0);
}

at::Tensor Slot::IndexSelect(const at::Tensor& index, int64_t beg, int64_t end) {
  return recis::functional::block_gather(index.reshape({-1}).slice(0, beg, end), chunks_, chunk_rows_, -1, false);
}

at::Tensor Slot::Conform(at::Tensor value) const {
  if (value.dim() == 0) value = value.view({1});
  if (value.dim() == 1 && row_shape_.size() == 1 && row_shape_[0] == 1) value = value.view({-1, 1});
  return value.to(at::TensorOptions().device(device_).dtype(dtype_));
}

void Slot::IndexInsert(const at::Tensor& index, at::Tensor value) {
  recis::functional::block_insert(index, Conform(std::move(value)), chunks_, chunk_rows_);
}

void Slot::IndexInsert(const at::Tensor& index, at::Tensor value, const at::Tensor& accept_indicator) {
  recis::functional::block_insert_with_mask(index, Conform(std::move(value)), accept_indicator, chunks_, chunk_rows_);
}

at::Tensor Slot::GenVal(int64_t rows) {
  std::vector<int64_t> shape{rows};
  shape.insert(shape.end(), row_shape_.begin(), row_shape_.end());
  return generator_->Generate(shape);
}

void Slot::EnsureChunks(int64_t n_chunks) {
  std::vector<int64_t> shape{chunk_rows_}, fan{block_size_};
  shape.insert(shape.end(), row_shape_.begin(), row_shape_.end());
  fan.insert(fan.end(), row_shape_.begin(), row_shape_.end());
  // one tensor for several blocks; fan-dependent initialisers still see one [block_size, D] block
  while (static_cast<int64_t>(chunks_.size()) < n_chunks) chunks_.push_back(generator_->Generate(shape, fan));
}

void Slot::Clear() {
  chunks_.clear();
  visible_blocks_ = 0;
}

// ------------------------------------------------------------------------------------ SlotGroup
SlotGroup::SlotGroup(int64_t block_size, at::Device device, int64_t chunk_rows)
    : block_size_(block_size), device_(device), chunk_rows_(chunk_rows) {}

SlotPtr SlotGroup::AppendSlot(const std::string& name, at::ScalarType dtype,
                              const std::vector<int64_t>& partial_shape, GeneratorPtr generator) {
  TORCH_CHECK(name_to_index_.find(name) == name_to_index_.end(), "slot ", name, " already exists");
  auto slot = c10::make_intrusive<Slot>(name, block_size_, dtype, partial_shape, std::move(generator), device_,
                                        chunk_rows_);
  slot->EnsureChunks(n_chunks_);  // a late slot catches up with the table
  slot->SetVisibleBlocks(block_num_);
  name_to_index_[name] = static_cast<int64_t>(slots_.size());
  slots_.push_back(slot);
  return slot;
}

SlotPtr SlotGroup::AppendSlot(const std::string& name, at::ScalarType dtype,
                              const std::vector<int64_t>& partial_shape, double init_val) {
  std::vector<int64_t> shape{block_size_};
  if (partial_shape.size() > 1) shape.insert(shape.end(), partial_shape.begin() + 1, partial_shape.end());
  return AppendSlot(name, dtype, partial_shape, MakeConstantGenerator(shape, dtype, init_val));
}

void SlotGroup::AppendEmbSlot(at::ScalarType dtype, const std::vector<int64_t>& partial_shape,
                              GeneratorPtr generator) {
  AppendSlot(EmbSlotName(), dtype, partial_shape, std::move(generator));
  emb_slot_index_ = static_cast<int64_t>(slots_.size()) - 1;
}

void SlotGroup::AppendStepFilterSlot(const std::string& name, int64_t init_step) {
  AppendSlot(name, at::kLong, {block_size_, 1}, static_cast<double>(init_step));
}

SlotPtr SlotGroup::GetSlotByName(const std::string& name) {
  auto it = name_to_index_.find(name);
  TORCH_CHECK(it != name_to_index_.end(), "no slot named ", name);
  return slots_[it->second];
}

SlotPtr SlotGroup::GetSlotByIndex(int64_t index) {
  TORCH_CHECK(index >= 0 && index < static_cast<int64_t>(slots_.size()), "slot index ", index, " out of range");
  return slots_[index];
}

int64_t SlotGroup::GetSlotIndex(const std::string& name) {
  auto it = name_to_index_.find(name);
  TORCH_CHECK(it != name_to_index_.end(), "no slot named ", name);
  return it->second;
}

void SlotGroup::EnsureRows(int64_t rows) {
  const int64_t need = (rows + chunk_rows_ - 1) / chunk_rows_;
  if (need > n_chunks_) {
    n_chunks_ = need;
    for (auto& s : slots_) s->EnsureChunks(need);
  }
}

void SlotGroup::SetBlockNum(int64_t block_num) {
  if (block_num > block_num_) {
    EnsureRows(block_num * block_size_);
    block_num_ = block_num;
    for (auto& s : slots_) s->SetVisibleBlocks(block_num);
  }
}

void SlotGroup::Clear() {
  for (auto& s : slots_) s->Clear();
  n_chunks_ = 0;
  block_num_ = 0;
}

}  // namespace embedding
}  // namespace recis

// ------------------------------------------------------------------------------------ Hashtable
namespace {
constexpr int64_t kChunkBytes = 8 << 20;
}

Hashtable::Hashtable(int64_t block_size, const std::vector<int64_t>& embedding_shape, at::ScalarType dtype,
                     at::Device device, bool coalesce, const std::vector<std::string>& children,
                     c10::intrusive_ptr<recis::embedding::Generator> generator, int64_t slice_begin,
                     int64_t slice_end, int64_t slice_size)
    : device_(device), dtype_(dtype), slice_begin_(slice_begin), slice_end_(slice_end), slice_size_(slice_size) {
  TORCH_CHECK(device.is_cuda(), "tables live in GPU memory in this build; got device ", device);
  TORCH_CHECK(block_size > 0, "block_size must be positive");
  if (!device_.has_index()) device_ = at::Device(device.type(), c10::hip::current_device());
  int64_t row_bytes = static_cast<int64_t>(c10::elementSize(dtype));
  for (int64_t d : embedding_shape) row_bytes *= d;
  const int64_t chunk_rows = std::max<int64_t>(1, kChunkBytes / std::max<int64_t>(1, row_bytes * block_size)) * block_size;
  slot_group_ = c10::make_intrusive<recis::embedding::SlotGroup>(block_size, device_, chunk_rows);
  std::vector<int64_t> partial_shape{block_size};
  partial_shape.insert(partial_shape.end(), embedding_shape.begin(), embedding_shape.end());
  slot_group_->AppendEmbSlot(dtype, partial_shape, std::move(generator));
  children_info_ = c10::make_intrusive<recis::embedding::ChildrenInfo>(coalesce, children);
  c10::DeviceGuard guard(device_);
  check(recis_idmap_create(0, &id_map_));
}

Hashtable::~Hashtable() {
  if (id_map_ != nullptr) recis_idmap_destroy(id_map_);
}

c10::intrusive_ptr<Hashtable> Hashtable::Make(int64_t block_size, const std::vector<int64_t>& embedding_shape,
                                              at::ScalarType dtype, at::Device device, bool coalesce,
                                              const std::vector<std::string>& children,
                                              c10::intrusive_ptr<recis::embedding::Generator> generator,
                                              int64_t slice_begin, int64_t slice_end, int64_t slice_size) {
  return c10::make_intrusive<Hashtable>(block_size, embedding_shape, dtype, device, coalesce, children,
                                        std::move(generator), slice_begin, slice_end, slice_size);
}

at::Tensor Hashtable::OnDevice(const at::Tensor& ids) const {
  at::Tensor t = ids.to(at::TensorOptions().device(device_).dtype(at::kLong));
  return t.contiguous();
}

// After a find-or-insert of `incoming` keys: rows up to the allocator's high-water mark (+1 spare)
// must exist before any row kernel runs. The map keeps an upper bound of the mark on the host (what
// the last finished call published plus every id queued since); the exact mark is read back only
// when that bound passes the capacity.
void Hashtable::MakeRoom(int64_t incoming) {
  auto& sg = *slot_group_;
  int64_t ub = 0;
  check(recis_idmap_bounds(id_map_, &ub, nullptr));
  if (ub + 1 > sg.CapacityRows()) {
    ub = ids_num();  // synchronises
    const bool roomy = sg.ChunkRows() <= 32 * std::max<int64_t>(incoming, 1);
    const int64_t want = ub + 1 + std::max<int64_t>((roomy ? 16 : 2) * incoming, sg.BlockSize());
    if (want > sg.CapacityRows() && (roomy || ub + 1 + incoming > sg.CapacityRows())) sg.EnsureRows(want);
  }
  if (sg.CapacityRows() == 0) sg.EnsureRows(1);
}

// block_num = (id_num + block_size) / block_size (csrc/embedding/hashtable.cc:255-261)
void Hashtable::SyncBlockNum() {
  auto& sg = *slot_group_;
  sg.SetBlockNum((ids_num() + sg.BlockSize()) / sg.BlockSize());
}

int64_t Hashtable::ids_num() {
  c10::DeviceGuard guard(device_);
  int64_t id_num = 0;
  check(recis_idmap_stats(id_map_, nullptr, &id_num, nullptr, nullptr, stream_of(device_)));
  return id_num;
}

at::Tensor Hashtable::InsertLookupIndex(const at::Tensor& ids) {
  c10::DeviceGuard guard(device_);
  at::Tensor i = OnDevice(ids);
  at::Tensor index = at::empty(i.sizes(), i.options());
  check(recis_idmap_lookup(id_map_, i.data_ptr<int64_t>(), i.numel(), index.data_ptr<int64_t>(), stream_of(device_)));
  MakeRoom(i.numel());
  return index;
}

at::Tensor Hashtable::LookupIndexReadOnly(const at::Tensor& ids) {
  c10::DeviceGuard guard(device_);
  at::Tensor i = OnDevice(ids);
  at::Tensor index = at::empty(i.sizes(), i.options());
  check(recis_idmap_lookup_readonly(id_map_, i.data_ptr<int64_t>(), i.numel(), index.data_ptr<int64_t>(),
                                    stream_of(device_)));
  return index;
}

std::tuple<at::Tensor, at::Tensor> Hashtable::EmbeddingLookup(const at::Tensor& ids, bool readonly) {
  at::Tensor index;
  if (readonly) {
    index = LookupIndexReadOnly(ids);
    MakeRoom(0);
  } else {
    index = InsertLookupIndex(ids);
  }
  auto emb_slot = slot_group_->EmbSlot();
  at::Tensor emb = recis::functional::block_gather(index, emb_slot->Chunks(), emb_slot->ChunkRows(), kNullIndex, readonly);
  return std::make_tuple(index, emb);
}

// Rows of the ids whose indicator is set (inserted when new), 0 for the others
// (csrc/embedding/hashtable.cc:237-248).
at::Tensor Hashtable::InsertLookupIndexWithIndicator(const at::Tensor& ids, const at::Tensor& indicator) {
  at::Tensor i = OnDevice(ids), ind = indicator.to(device_);
  at::Tensor index = at::zeros_like(i);
  index.masked_scatter_(ind, InsertLookupIndex(at::masked_select(i, ind)));
  return index;
}

void Hashtable::Insert(const at::Tensor& ids, const at::Tensor& embedding) {
  auto slot = slot_group_->EmbSlot();
  TORCH_CHECK(embedding.scalar_type() == slot->Dtype(), "embeding type must be [", slot->Dtype(), "] but get ",
              embedding.scalar_type());
  TORCH_CHECK(ids.size(0) == embedding.size(0), "size of ids and embedding dismatch, ids: ", ids.size(0),
              " embedding: ", embedding.size(0));
  at::Tensor index = InsertLookupIndex(ids);
  slot->IndexInsert(index, embedding);
}

void Hashtable::UpdateSlot(const std::string& slot_name, const at::Tensor& index, at::Tensor value) {
  auto slot = slot_group_->GetSlotByName(slot_name);
  TORCH_CHECK(value.scalar_type() == slot->Dtype(), "embedding type must be [", slot->Dtype(), "] but get ",
              value.scalar_type());
  slot->IndexInsert(OnDevice(index), std::move(value));
}

void Hashtable::AppendStepFilterSlot(const std::string& filter_name, int64_t init_step) {
  slot_group_->AppendStepFilterSlot(filter_name, init_step);
}

void Hashtable::AppendFilterSlot(const std::string& filter_name, at::ScalarType dtype, int64_t slot_dim,
                                 c10::intrusive_ptr<recis::embedding::Generator> generator) {
  slot_group_->AppendSlot(filter_name, dtype, {0, slot_dim}, std::move(generator));
}

void Hashtable::Clear() {
  ClearGrad();
  ClearId();
  slot_group_->Clear();
}

void Hashtable::ClearId() {
  c10::DeviceGuard guard(device_);
  check(recis_idmap_clear(id_map_, stream_of(device_)));
}

std::tuple<at::Tensor, at::Tensor> Hashtable::ids_map() {
  c10::DeviceGuard guard(device_);
  int64_t live = 0, count = 0;
  void* stream = stream_of(device_);
  check(recis_idmap_stats(id_map_, &live, nullptr, nullptr, nullptr, stream));
  auto opt = at::TensorOptions().device(device_).dtype(at::kLong);
  at::Tensor ids = at::empty({live}, opt), index = at::empty({live}, opt);
  check(recis_idmap_snapshot(id_map_, ids.data_ptr<int64_t>(), index.data_ptr<int64_t>(), live, &count, stream));
  TORCH_CHECK(count == live, "id map changed during the snapshot: ", count, " keys, expected ", live);
  return std::make_tuple(ids, index);
}

at::Tensor Hashtable::ids() { return std::get<0>(ids_map()); }

// Erase keys, free their rows, re-initialise every slot but preserve_slot at those rows
// (csrc/embedding/hashtable.cc:263-278).
void Hashtable::Delete(const at::Tensor& ids, const at::Tensor& index, const std::string& preserve_slot) {
  if (ids.numel() == 0) return;
  c10::DeviceGuard guard(device_);
  at::Tensor i = OnDevice(ids).view({-1}), x = OnDevice(index).view({-1});
  TORCH_CHECK(i.numel() == x.numel(), "ids and index differ in length");
  check(recis_idmap_erase(id_map_, i.data_ptr<int64_t>(), x.data_ptr<int64_t>(), i.numel(), stream_of(device_)));
  const int64_t keep = preserve_slot.empty() ? -1 : slot_group_->GetSlotIndex(preserve_slot);
  auto slots = slot_group_->Slots();
  for (int64_t s = 0; s < static_cast<int64_t>(slots.size()); ++s) {
    if (s != keep) slots[s]->IndexInsert(x, slots[s]->GenVal(i.numel()));
  }
}

void Hashtable::AcceptGrad(const at::Tensor& grad_index, const at::Tensor& grad) {
  TORCH_CHECK(grad_index.scalar_type() == at::kLong, "grad_index must be int64");
  TORCH_CHECK(grad.scalar_type() == dtype_ ||
                  (grad.scalar_type() == at::kFloat && (dtype_ == at::kBFloat16 || dtype_ == at::kHalf)),
              "grad dtype ", grad.scalar_type(), " does not match the table (", dtype_, ")");
  grad_index_.push_back(grad_index);
  grad_.push_back(grad);
}

// The sparse COO gradient as the reference builds it (csrc/embedding/hashtable.cc:90-134),
// including its layout when rows repeat: the inverse positions as indices and an N-row value buffer
// whose first U rows hold the sums.
at::Tensor Hashtable::grad(int64_t accumulate_steps) {
  at::Tensor index = at::cat(grad_index_, 0), g = at::cat(grad_, 0);
  auto uniq = at::_unique(index, /*sorted=*/false, /*return_inverse=*/true);
  const at::Tensor& values = std::get<0>(uniq);
  const at::Tensor& inverse = std::get<1>(uniq);
  std::vector<int64_t> shape = g.sizes().vec();
  at::Tensor final_indices, final_grad;
  if (index.numel() == values.numel()) {
    final_indices = index.view({1, -1});
    final_grad = g;
    shape[0] = index.numel() ? index.max().item<int64_t>() + 1 : 0;
  } else {
    final_indices = inverse.view({1, -1});
    shape[0] = inverse.numel();
    final_grad = at::zeros(shape, g.options());
    final_grad.index_add_(0, inverse.view({-1}), g);
    shape[0] = values.numel() ? values.max().item<int64_t>() + 1 : 0;
  }
  final_grad = final_grad / accumulate_steps;
  at::Tensor sparse = at::_sparse_coo_tensor_unsafe(final_indices, final_grad, shape, final_grad.options().layout(at::kSparse));
  return sparse.detach_();
}

std::tuple<at::Tensor, at::Tensor> Hashtable::GradPairs(int64_t accumulate_steps) {
  at::Tensor index = grad_index_.size() == 1 ? grad_index_[0] : at::cat(grad_index_, 0);
  at::Tensor g = grad_.size() == 1 ? grad_[0] : at::cat(grad_, 0);
  auto uniq = at::_unique(index, /*sorted=*/false, /*return_inverse=*/true);
  if (std::get<0>(uniq).numel() != index.numel()) {
    std::vector<int64_t> shape = g.sizes().vec();
    shape[0] = std::get<0>(uniq).numel();
    at::Tensor summed = at::zeros(shape, g.options());
    summed.index_add_(0, std::get<1>(uniq).view({-1}), g);
    index = std::get<0>(uniq);
    g = summed;
  }
  if (accumulate_steps != 1) g = g / accumulate_steps;
  return std::make_tuple(index, g);
}

void Hashtable::ClearGrad() {
  grad_index_.clear();
  grad_.clear();
}

c10::intrusive_ptr<recis::embedding::SlotGroup> Hashtable::SlotGroup() {
  SyncBlockNum();
  return slot_group_;
}

c10::intrusive_ptr<recis::embedding::Slot> Hashtable::GetSlot(const std::string& name) {
  SyncBlockNum();
  return slot_group_->GetSlotByName(name);
}
