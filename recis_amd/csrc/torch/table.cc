#include "table.h"

#include <ATen/record_function.h>

#include <cmath>
#include <cstdlib>
#include <set>

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
    case Kind::kFromTensor: {
      const int64_t have = source_.size(0);
      for (int64_t done = 0, rows = t.size(0); done < rows;) {
        const int64_t take = std::min(rows - done, have - cursor_);
        t.narrow(0, done, take).copy_(source_.narrow(0, cursor_, take));
        done += take;
        cursor_ = (cursor_ + take) % have;
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

GeneratorPtr MakeTensorGenerator(const std::vector<int64_t>& shape, at::ScalarType dtype, at::Tensor source) {
  TORCH_CHECK(source.dim() >= 1 && source.size(0) > 0, "the source tensor must hold at least one row");
  auto g = c10::make_intrusive<Generator>(Generator::Kind::kFromTensor, shape, dtype);
  g->SetSource(source.to(dtype));
  return g;
}

// ------------------------------------------------------------------------------------ ChildrenInfo
ChildrenInfo::ChildrenInfo(bool coalesce, const std::vector<std::string>& children)
    : coalesce_(coalesce), children_(children) {
  // csrc/embedding/children_info.cc:38-48
  TORCH_CHECK(!children_.empty(), "empty children");
  TORCH_CHECK(static_cast<int64_t>(children_.size()) < MaxChildrenNum(), "children size[", children_.size(),
              "] exceeds max children size[", MaxChildrenNum(), "]");
  TORCH_CHECK(coalesce_ || children_.size() == 1, "non coalesce has more than one child");
  std::set<std::string> names(children_.begin(), children_.end());
  TORCH_CHECK(names.size() == children_.size(), "duplicate child[", children_, "]");
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

// ------------------------------------------------------------------------------------ IdMapHolder
IdMapHolder::~IdMapHolder() {
  if (map != nullptr) recis_idmap_destroy(map);
}

int64_t IdMapHolder::IdNum() const {
  c10::DeviceGuard guard(device);
  int64_t id_num = 0;
  check(recis_idmap_stats(map, nullptr, &id_num, nullptr, nullptr, stream_of(device)));
  return id_num;
}

// ------------------------------------------------------------------------------------ Slot
Slot::Slot(const std::string& name, int64_t block_size, at::ScalarType dtype,
           const std::vector<int64_t>& partial_shape, GeneratorPtr generator, at::Device device, int64_t chunk_rows,
           std::shared_ptr<IdMapHolder> map)
    : name_(name),
      block_size_(block_size),
      dtype_(dtype),
      row_shape_(partial_shape.begin() + (partial_shape.empty() ? 0 : 1), partial_shape.end()),
      generator_(std::move(generator)),
      device_(device),
      chunk_rows_(chunk_rows),
      flat_size_(1),
      map_(std::move(map)) {
  for (int64_t d : row_shape_) flat_size_ *= d;
  generator_->set_device(device);
}

int64_t Slot::VisibleBlocks() const {
  if (chunks_.empty()) return 0;
  const int64_t blocks = (map_->IdNum() + block_size_) / block_size_;
  const int64_t have = static_cast<int64_t>(chunks_.size()) * (chunk_rows_ / block_size_);
  return std::min(blocks, have);
}

std::vector<at::Tensor> Slot::ValuesDeref() {
  const int64_t per = chunk_rows_ / block_size_, visible = VisibleBlocks();
  std::vector<at::Tensor> out;
  out.reserve(visible);
  for (int64_t b = 0; b < visible; ++b) {
    out.push_back(chunks_[b / per].narrow(0, (b % per) * block_size_, block_size_));
  }
  return out;
}

at::Tensor Slot::Value() {
  const int64_t rows = VisibleBlocks() * block_size_;
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

void Slot::SetChunkRows(int64_t chunk_rows) {
  TORCH_CHECK(chunks_.empty(), "slot ", name_, " already has storage");
  chunk_rows_ = chunk_rows;
}

at::Tensor Slot::NewChunkValues() {
  std::vector<int64_t> shape{chunk_rows_}, fan{block_size_};
  shape.insert(shape.end(), row_shape_.begin(), row_shape_.end());
  fan.insert(fan.end(), row_shape_.begin(), row_shape_.end());
  // one tensor for several blocks; fan-dependent initialisers still see one [block_size, D] block
  return generator_->Generate(shape, fan);
}

void Slot::EnsureChunks(int64_t n_chunks) {
  TORCH_CHECK(!packed_, "slot ", name_, " does not own its storage");
  while (static_cast<int64_t>(chunks_.size()) < n_chunks) chunks_.push_back(NewChunkValues());
}

void Slot::SetChunk(int64_t c, at::Tensor view) {
  TORCH_CHECK(c >= 0 && c <= static_cast<int64_t>(chunks_.size()), "chunk ", c, " out of order");
  if (c == static_cast<int64_t>(chunks_.size()))
    chunks_.push_back(std::move(view));
  else
    chunks_[c] = std::move(view);
}

void Slot::Clear() { chunks_.clear(); }

// ------------------------------------------------------------------------------------ SlotGroup
SlotGroup::SlotGroup(int64_t block_size, at::Device device, int64_t chunk_rows, std::shared_ptr<IdMapHolder> map)
    : block_size_(block_size), device_(device), chunk_rows_(chunk_rows), map_(std::move(map)) {}

SlotPtr SlotGroup::AppendSlot(const std::string& name, at::ScalarType dtype,
                              const std::vector<int64_t>& partial_shape, GeneratorPtr generator) {
  TORCH_CHECK(name_to_index_.find(name) == name_to_index_.end(), "slot ", name, " already exists");
  auto slot = c10::make_intrusive<Slot>(name, block_size_, dtype, partial_shape, std::move(generator), device_,
                                        chunk_rows_, map_);
  slot->EnsureChunks(n_chunks_);  // a late slot catches up with the table
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

at::Tensor SlotGroup::PackedView(const at::Tensor& store, int64_t member, int64_t members,
                                 const SlotPtr& slot) const {
  (void)members;
  std::vector<int64_t> shape{chunk_rows_};
  const auto row = slot->RowShape();
  shape.insert(shape.end(), row.begin(), row.end());
  return store.narrow(1, member * slot->FlatSize(), slot->FlatSize()).view(shape);
}

void SlotGroup::AddPackedChunk() {
  const int64_t members = static_cast<int64_t>(packed_.size());
  const SlotPtr& emb = slots_[packed_[0]];
  at::Tensor store = at::empty({chunk_rows_, members * emb->FlatSize()},
                               at::TensorOptions().dtype(emb->Dtype()).device(device_));
  const int64_t c = static_cast<int64_t>(packed_chunks_.size());
  for (int64_t g = 0; g < members; ++g) {
    const SlotPtr& slot = slots_[packed_[g]];
    at::Tensor view = PackedView(store, g, members, slot);
    view.copy_(slot->NewChunkValues());
    slot->SetChunk(c, view);
  }
  packed_chunks_.push_back(store);
}

std::vector<SlotPtr> SlotGroup::AppendPackedSlots(const std::vector<std::string>& names, double init_val) {
  TORCH_CHECK(emb_slot_index_ >= 0, "the table has no embedding slot yet");
  SlotPtr emb = slots_[emb_slot_index_];
  std::vector<int64_t> partial{1};
  const auto row = emb->RowShape();
  partial.insert(partial.end(), row.begin(), row.end());
  const char* knob = std::getenv("RECIS_PACKED_STATE");
  std::vector<SlotPtr> added;
  if (knob == nullptr || std::string(knob) != "1") {
    for (const auto& name : names) added.push_back(AppendSlot(name, emb->Dtype(), partial, init_val));
    return added;
  }
  for (const auto& name : names)
    TORCH_CHECK(name_to_index_.find(name) == name_to_index_.end(), "slot ", name, " already exists");
  const size_t had = packed_.size();
  if (packed_.empty()) {
    packed_.push_back(emb_slot_index_);
    emb->SetPacked();
  }
  std::vector<int64_t> shape{block_size_};
  shape.insert(shape.end(), row.begin(), row.end());
  for (const auto& name : names) {
    auto slot = c10::make_intrusive<Slot>(name, block_size_, emb->Dtype(), partial,
                                          MakeConstantGenerator(shape, emb->Dtype(), init_val), device_, chunk_rows_,
                                          map_);
    slot->SetPacked();
    name_to_index_[name] = static_cast<int64_t>(slots_.size());
    packed_.push_back(static_cast<int64_t>(slots_.size()));
    slots_.push_back(slot);
    added.push_back(slot);
  }
  // storage that exists moves into the wider layout, one chunk at a time (the old chunk is let go
  // as soon as its rows are copied)
  const int64_t members = static_cast<int64_t>(packed_.size());
  std::vector<at::Tensor> stores;
  for (int64_t c = 0; c < n_chunks_; ++c) {
    at::Tensor store = at::empty({chunk_rows_, members * emb->FlatSize()},
                                 at::TensorOptions().dtype(emb->Dtype()).device(device_));
    for (int64_t g = 0; g < members; ++g) {
      const SlotPtr& slot = slots_[packed_[g]];
      at::Tensor view = PackedView(store, g, members, slot);
      const bool old = g < static_cast<int64_t>(std::max<size_t>(had, 1));
      view.copy_(old ? slot->Chunks()[c] : slot->NewChunkValues());
      slot->SetChunk(c, view);
    }
    if (c < static_cast<int64_t>(packed_chunks_.size())) packed_chunks_[c] = at::Tensor();
    stores.push_back(store);
  }
  packed_chunks_ = std::move(stores);
  return added;
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

int64_t SlotGroup::BlockNum() const {
  if (n_chunks_ == 0) return 0;
  return std::min((map_->IdNum() + block_size_) / block_size_, CapacityRows() / block_size_);
}

void SlotGroup::SetChunkRows(int64_t chunk_rows) {
  TORCH_CHECK(n_chunks_ == 0, "the table already has storage");
  chunk_rows_ = chunk_rows;
  for (auto& s : slots_) s->SetChunkRows(chunk_rows);
}

void SlotGroup::EnsureRows(int64_t rows) {
  const int64_t need = (rows + chunk_rows_ - 1) / chunk_rows_;
  if (need > n_chunks_) {
    n_chunks_ = need;
    while (!packed_.empty() && static_cast<int64_t>(packed_chunks_.size()) < need) AddPackedChunk();
    for (auto& s : slots_)
      if (!s->Packed()) s->EnsureChunks(need);
  }
}

void SlotGroup::Clear() {
  for (auto& s : slots_) s->Clear();
  packed_chunks_.clear();
  n_chunks_ = 0;
}

}  // namespace embedding
}  // namespace recis

// ------------------------------------------------------------------------------------ Hashtable
namespace {
constexpr int64_t kChunkBytes = 8 << 20;
using recis::BatchPlanPtr;
using recis::hipabi::block_ptr_table;
using recis::hipabi::dtype_code;
using recis::hipabi::index_kind;

int64_t row_bytes_of(at::ScalarType dtype, const std::vector<int64_t>& shape) {
  int64_t b = static_cast<int64_t>(c10::elementSize(dtype));
  for (int64_t d : shape) b *= d;
  return b;
}
}  // namespace

Hashtable::Hashtable(int64_t block_size, const std::vector<int64_t>& embedding_shape, at::ScalarType dtype,
                     at::Device device, bool coalesce, const std::vector<std::string>& children,
                     c10::intrusive_ptr<recis::embedding::Generator> generator, int64_t slice_begin,
                     int64_t slice_end, int64_t slice_size)
    : device_(device),
      dtype_(dtype),
      embedding_shape_(embedding_shape),
      slice_begin_(slice_begin),
      slice_end_(slice_end),
      slice_size_(slice_size) {
  children_info_ = c10::make_intrusive<recis::embedding::ChildrenInfo>(coalesce, children);  // validates the names
  TORCH_CHECK(block_size > 0, "block_size must be positive");
  TORCH_CHECK(device.is_cuda(), "tables live in GPU memory in this build; got device ", device);
  if (!device_.has_index()) device_ = at::Device(device.type(), c10::hip::current_device());
  {
    c10::DeviceGuard guard(device_);
    recis_idmap* m = nullptr;
    check(recis_idmap_create(0, &m));
    map_ = std::make_shared<recis::embedding::IdMapHolder>(m, device_);
  }
  const int64_t row_bytes = row_bytes_of(dtype, embedding_shape);
  const int64_t chunk_rows = std::max<int64_t>(1, kChunkBytes / std::max<int64_t>(1, row_bytes * block_size)) * block_size;
  slot_group_ = c10::make_intrusive<recis::embedding::SlotGroup>(block_size, device_, chunk_rows, map_);
  std::vector<int64_t> partial_shape{block_size};
  partial_shape.insert(partial_shape.end(), embedding_shape.begin(), embedding_shape.end());
  slot_group_->AppendEmbSlot(dtype, partial_shape, std::move(generator));
}

c10::intrusive_ptr<Hashtable> Hashtable::Make(int64_t block_size, const std::vector<int64_t>& embedding_shape,
                                              at::ScalarType dtype, at::Device device, bool coalesce,
                                              const std::vector<std::string>& children,
                                              c10::intrusive_ptr<recis::embedding::Generator> generator,
                                              int64_t slice_begin, int64_t slice_end, int64_t slice_size) {
  return c10::make_intrusive<Hashtable>(block_size, embedding_shape, dtype, device, coalesce, children,
                                        std::move(generator), slice_begin, slice_end, slice_size);
}

void Hashtable::Reserve(int64_t rows) {
  if (rows <= 0) return;
  c10::DeviceGuard guard(device_);
  const int64_t bs = slot_group_->BlockSize();
  slot_group_->SetChunkRows((rows + 1 + bs - 1) / bs * bs);
  check(recis_idmap_reserve(map_->map, rows, stream_of(device_)));
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
  check(recis_idmap_bounds(map_->map, &ub, nullptr));
  if (ub + 1 > sg.CapacityRows()) {
    ub = ids_num();  // synchronises
    // Leave room for many calls of this size, unless storage grows in chunks far larger than a batch
    // (a pre-sized table): rows are cheap, pipeline bubbles are not.
    const bool roomy = sg.ChunkRows() <= 32 * std::max<int64_t>(incoming, 1);
    const int64_t want = ub + 1 + std::max<int64_t>((roomy ? 16 : 2) * incoming, sg.BlockSize());
    if (want > sg.CapacityRows() && (roomy || ub + 1 + incoming > sg.CapacityRows())) sg.EnsureRows(want);
  }
  if (sg.CapacityRows() == 0) sg.EnsureRows(1);
}

int64_t Hashtable::ids_num() { return map_->IdNum(); }

std::vector<int64_t> Hashtable::IdMapStats() {
  c10::DeviceGuard guard(device_);
  std::vector<int64_t> v(4, 0);
  check(recis_idmap_stats(map_->map, &v[0], &v[1], &v[2], &v[3], stream_of(device_)));
  int bits = 0;
  check(recis_hip_poll_device_errors(&bits));  // the call above has waited for the stream already
  TORCH_CHECK(bits == 0, "librecis_hip: device-side errors in earlier kernels (bits ", bits, ")");
  return v;
}

at::Tensor Hashtable::InsertLookupIndex(const at::Tensor& ids) {
  c10::DeviceGuard guard(device_);
  at::Tensor i = OnDevice(ids);
  at::Tensor index = at::empty(i.sizes(), i.options());
  check(recis_idmap_lookup(map_->map, i.data_ptr<int64_t>(), i.numel(), index.data_ptr<int64_t>(), stream_of(device_)));
  MakeRoom(i.numel());
  return index;
}

at::Tensor Hashtable::LookupIndexReadOnly(const at::Tensor& ids) {
  c10::DeviceGuard guard(device_);
  at::Tensor i = OnDevice(ids);
  at::Tensor index = at::empty(i.sizes(), i.options());
  check(recis_idmap_lookup_readonly(map_->map, i.data_ptr<int64_t>(), i.numel(), index.data_ptr<int64_t>(),
                                    stream_of(device_)));
  return index;
}

at::Tensor Hashtable::LookupIndex(const at::Tensor& ids, bool readonly) {
  return readonly ? LookupIndexReadOnly(ids) : InsertLookupIndex(ids);
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
  last_lookup_index_ = index;
  last_lookup_unique_ = recis::functional::known_unique(ids);
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
  check(recis_idmap_clear(map_->map, stream_of(device_)));
}

std::tuple<at::Tensor, at::Tensor> Hashtable::ids_map() {
  c10::DeviceGuard guard(device_);
  int64_t live = 0, count = 0;
  void* stream = stream_of(device_);
  check(recis_idmap_stats(map_->map, &live, nullptr, nullptr, nullptr, stream));
  auto opt = at::TensorOptions().device(device_).dtype(at::kLong);
  at::Tensor ids = at::empty({live}, opt), index = at::empty({live}, opt);
  check(recis_idmap_snapshot(map_->map, ids.data_ptr<int64_t>(), index.data_ptr<int64_t>(), live, &count, stream));
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
  check(recis_idmap_erase(map_->map, i.data_ptr<int64_t>(), x.data_ptr<int64_t>(), i.numel(), stream_of(device_)));
  const int64_t keep = preserve_slot.empty() ? -1 : slot_group_->GetSlotIndex(preserve_slot);
  auto slots = slot_group_->Slots();
  for (int64_t s = 0; s < static_cast<int64_t>(slots.size()); ++s) {
    if (s != keep) slots[s]->IndexInsert(x, slots[s]->GenVal(i.numel()));
  }
}

std::tuple<at::Tensor, at::Tensor> Hashtable::EvictOlder(const std::string& stamp_slot, int64_t threshold) {
  c10::DeviceGuard guard(device_);
  auto stamps = slot_group_->GetSlotByName(stamp_slot);
  TORCH_CHECK((stamps->Dtype() == at::kLong || stamps->Dtype() == at::kInt) && stamps->FlatSize() == 1,
              "the stamp slot must be int32/int64 of width 1");
  void* stream = stream_of(device_);
  int64_t live = 0, count = 0;
  check(recis_idmap_stats(map_->map, &live, nullptr, nullptr, nullptr, stream));
  auto opt = at::TensorOptions().device(device_).dtype(at::kLong);
  at::Tensor ids = at::empty({live}, opt), index = at::empty({live}, opt);
  if (!stamps->Chunks().empty()) {
    at::Tensor tab = block_ptr_table(stamps->Chunks());
    check(recis_idmap_evict_older(map_->map, reinterpret_cast<const void* const*>(tab.data_ptr()),
                                  static_cast<int64_t>(stamps->Chunks().size()), stamps->ChunkRows(),
                                  stamps->Dtype() == at::kLong ? 1 : 0, threshold, ids.data_ptr<int64_t>(),
                                  index.data_ptr<int64_t>(), live, &count, stream));
  }
  ids = ids.narrow(0, 0, count);
  index = index.narrow(0, 0, count);
  if (count) {
    const int64_t keep = slot_group_->GetSlotIndex(stamp_slot);
    auto slots = slot_group_->Slots();
    for (int64_t s = 0; s < static_cast<int64_t>(slots.size()); ++s) {
      if (s != keep) slots[s]->IndexInsert(index, slots[s]->GenVal(count));
    }
  }
  return std::make_tuple(ids, index);
}

// ------------------------------------------------------------------------------------ batch plan
BatchPlanPtr Hashtable::PlanLookup(const std::vector<at::Tensor>& ids, const c10::optional<std::vector<int64_t>>& tags,
                                   bool wait, bool need_inverse, bool need_pos) {
  c10::DeviceGuard guard(device_);
  BatchPlanPtr plan = recis::BatchPlan::Make(ids, tags, map_->map, wait, need_inverse, need_pos);
  int64_t call = 0;
  check(recis_idmap_last_call(map_->map, &call));
  plan->NoteLookup(this, call);
  MakeRoom(wait ? plan->U() : plan->n());
  return plan;
}

c10::optional<at::Tensor> Hashtable::PlanIndex(const BatchPlanPtr& plan) {
  if (plan->LookupCall(this) != 0 && plan->IndexBufRaw().defined()) return plan->IndexBufRaw();
  return c10::nullopt;
}

at::Tensor Hashtable::LookupIndexCounted(const BatchPlanPtr& plan, bool make_room) {
  c10::DeviceGuard guard(device_);
  at::Tensor out = at::empty_like(plan->unique_buf());
  check(recis_idmap_lookup_counted(map_->map, plan->unique_buf().data_ptr<int64_t>(), plan->unique_buf().numel(),
                                   plan->counts().data_ptr<int64_t>(), out.data_ptr<int64_t>(), stream_of(device_)));
  int64_t call = 0;
  check(recis_idmap_last_call(map_->map, &call));
  plan->NoteLookup(this, call);
  if (make_room) MakeRoom(plan->n());
  return out;
}

void Hashtable::SettleCount(int64_t n_true, const c10::optional<BatchPlanPtr>& plan) {
  const int64_t call = plan.has_value() && plan->defined() ? (*plan)->LookupCall(this) : 0;
  if (call == 0) {
    check(recis_idmap_settle_count(map_->map, n_true));
  } else {
    check(recis_idmap_settle_call(map_->map, call, n_true));
  }
}

at::Tensor Hashtable::SettleLookup(const at::Tensor& index_buf, int64_t n_true, const BatchPlanPtr& plan) {
  SettleCount(n_true, plan);
  MakeRoom(n_true);
  return index_buf.narrow(0, 0, n_true);
}

at::Tensor Hashtable::ExpandRows(const BatchPlanPtr& plan, const at::Tensor& row_index,
                                 const c10::optional<at::Tensor>& weight, const c10::optional<std::string>& stamp_slot,
                                 const c10::optional<at::Tensor>& stamp_value) {
  c10::DeviceGuard guard(device_);
  auto emb = slot_group_->EmbSlot();
  const auto& chunks = emb->Chunks();
  TORCH_CHECK(!chunks.empty(), "the table has no rows yet");
  TORCH_CHECK(row_index.is_cuda() && row_index.scalar_type() == at::kLong && row_index.is_contiguous(),
              "row_index must be a contiguous int64 GPU tensor");
  const int64_t D = emb->FlatSize(), n = plan->n();
  at::Tensor w;
  if (weight.has_value() && weight->defined()) {
    recis::hipabi::require_gpu(*weight, "weight");
    w = weight->contiguous();
  }
  at::Tensor table = block_ptr_table(chunks), stamp_table;
  const int64_t* stamp_ptr = nullptr;
  if (stamp_slot.has_value()) {
    auto stamps = slot_group_->GetSlotByName(*stamp_slot);
    TORCH_CHECK(stamps->Dtype() == at::kLong && stamps->FlatSize() == 1 && stamps->Chunks().size() == chunks.size(),
                "the stamp slot must be an int64 slot of width 1 of this table");
    TORCH_CHECK(stamp_value.has_value() && stamp_value->is_cuda() && stamp_value->scalar_type() == at::kLong &&
                    stamp_value->numel() == 1,
                "the stamp value must be a one-element int64 GPU tensor");
    stamp_table = block_ptr_table(stamps->Chunks());
    stamp_ptr = stamp_value->data_ptr<int64_t>();
  }
  at::Tensor out = at::empty({n, D}, chunks[0].options());
  const int code = dtype_code(dtype_);
  check(recis_csr_expand_rows_stamped(
      nullptr, reinterpret_cast<void* const*>(table.data_ptr()), static_cast<int64_t>(chunks.size()), emb->ChunkRows(),
      recis::hipabi::row_pitch_bytes(chunks[0]), row_index.data_ptr<int64_t>(), code, w.defined() ? w.data_ptr() : nullptr,
      w.defined() ? dtype_code(w.scalar_type()) : 0, plan->row_start().data_ptr<int32_t>(),
      plan->occ().data_ptr<int32_t>(), plan->hot_items().data_ptr<int32_t>(), plan->hot_cap(),
      plan->counts().data_ptr<int64_t>(), out.data_ptr(), code, plan->U_bound(), n, D,
      stamp_table.defined() ? reinterpret_cast<void* const*>(stamp_table.data_ptr()) : nullptr, stamp_ptr,
      stream_of(device_)));
  return out;
}

c10::optional<std::tuple<BatchPlanPtr, at::Tensor, at::Tensor>> Hashtable::DenseLookupExpand(
    const std::vector<at::Tensor>& cols, const c10::optional<std::vector<int64_t>>& tags,
    const c10::optional<std::string>& stamp_slot, const c10::optional<at::Tensor>& stamp_value) {
  if (cols.empty()) return c10::nullopt;
  for (const auto& c : cols) {
    const bool column = c.defined() && c.is_cuda() && c.scalar_type() == at::kLong && c.is_contiguous() &&
                        (c.dim() == 1 || (c.dim() == 2 && c.size(1) == 1)) && c.device() == device_;
    if (!column) return c10::nullopt;
  }
  BatchPlanPtr plan = PlanLookup(cols, tags, /*wait=*/false, /*need_inverse=*/false, /*need_pos=*/false);
  at::Tensor index = plan->IndexBufRaw();
  at::Tensor out = ExpandRows(plan, index, c10::nullopt, stamp_slot, stamp_value);
  return std::make_tuple(plan, index, out);
}

void Hashtable::AcceptSplitGrad(const at::Tensor& index_in, const BatchPlanPtr& plan,
                                const std::vector<c10::optional<at::Tensor>>& grads, const std::vector<int64_t>& split,
                                const c10::optional<at::Tensor>& src, const c10::optional<at::Tensor>& coef, int64_t key,
                                bool may_miss, bool settle) {
  TORCH_CHECK(grads.size() == split.size() && !grads.empty(), "one gradient per part");
  const int64_t D = slot_group_->EmbSlot()->FlatSize();
  int64_t rows = 0;
  for (int64_t r : split) rows += r;
  // consecutive slices of one buffer? then the whole gradient is that buffer, in place
  at::Tensor whole;
  const c10::optional<at::Tensor>& g0 = grads[0];
  if (g0.has_value() && g0->defined() && g0->is_contiguous() && g0->dim() == 2 && g0->size(1) == D) {
    const char* at_byte = static_cast<const char*>(g0->data_ptr());
    const void* storage = g0->storage().data();
    bool adjacent = true;
    for (size_t f = 0; f < grads.size() && adjacent; ++f) {
      const c10::optional<at::Tensor>& g = grads[f];
      adjacent = g.has_value() && g->defined() && g->scalar_type() == g0->scalar_type() && g->is_contiguous() &&
                 g->dim() == 2 && g->size(0) == split[f] && g->size(1) == D && g->data_ptr() == at_byte &&
                 g->storage().data() == storage;
      at_byte += split[f] * D * g0->element_size();
    }
    if (adjacent) whole = at::as_strided(*g0, {rows, D}, {D, 1}, g0->storage_offset());
  }
  if (!whole.defined()) {
    at::Tensor like;
    for (const auto& g : grads) {
      if (g.has_value() && g->defined()) {
        like = *g;
        break;
      }
    }
    if (!like.defined()) return;  // no gradient reached any part
    std::vector<at::Tensor> parts;
    for (size_t f = 0; f < grads.size(); ++f) {
      parts.push_back(grads[f].has_value() && grads[f]->defined() ? grads[f]->reshape({split[f], D})
                                                                  : at::zeros({split[f], D}, like.options()));
    }
    whole = at::cat(parts, 0);
  }
  at::Tensor index = index_in;
  if (settle) {
    const int64_t U = plan->U();
    SettleCount(U, plan);
    if (index.numel() > U) index = index.narrow(0, 0, U);
  }
  AcceptPlannedGrad(index, plan, {whole}, false, src.has_value() && src->defined() ? *src : plan->occ(), coef,
                    c10::nullopt, key, may_miss);
}

// ------------------------------------------------------------------------------------ gradients
void Hashtable::AcceptGrad(const at::Tensor& grad_index, const at::Tensor& grad) {
  // the index tensor the last embedding_lookup returned for ids that are known to be distinct has
  // no duplicates either
  const bool unique = last_lookup_unique_ && last_lookup_index_.defined() &&
                      grad_index.data_ptr() == last_lookup_index_.data_ptr() &&
                      grad_index.numel() == last_lookup_index_.numel() &&
                      grad_index._version() == last_lookup_index_._version();
  AcceptGradEx(grad_index, grad, unique, 0);
}

void Hashtable::AcceptGradEx(const at::Tensor& grad_index, const at::Tensor& grad, bool unique, int64_t key) {
  TORCH_CHECK(grad_index.scalar_type() == at::kLong, "grad_index must be int64");
  SumPlanned();  // a gradient waiting to be summed comes first, as it was handed over first
  TORCH_CHECK(grad.scalar_type() == dtype_ ||
                  (grad.scalar_type() == at::kFloat && (dtype_ == at::kBFloat16 || dtype_ == at::kHalf)),
              "grad dtype ", grad.scalar_type(), " does not match the table (", dtype_, ")");
  if (key != 0) {
    for (const auto& k : grad_keys_) {
      if (k.first == key && grad_[k.second].sizes() == grad.sizes()) {
        grad_[k.second] = grad_[k.second] + grad;
        return;
      }
    }
    grad_keys_.emplace_back(key, grad_.size());
  }
  grad_index_.push_back(grad_index);
  grad_.push_back(grad);
  grad_unique_.push_back(unique);
}

void Hashtable::AcceptPlannedGrad(const at::Tensor& index, const BatchPlanPtr& plan, const std::vector<at::Tensor>& rows,
                                  bool in_parts, const at::Tensor& src, const c10::optional<at::Tensor>& coef,
                                  const c10::optional<at::Tensor>& cover, int64_t key, bool may_miss) {
  TORCH_CHECK(!rows.empty() && (in_parts || rows.size() == 1), "accept_planned_grad: one array, or several in parts");
  PlannedGrad g;
  g.index = index;
  g.plan = plan;
  g.rows = rows;
  g.in_parts = in_parts;
  g.src = src;
  if (coef.has_value() && coef->defined()) g.coef = *coef;
  if (cover.has_value() && cover->defined()) g.cover = *cover;
  g.key = key;
  g.may_miss = may_miss;
  if (grad_.empty() && planned_.size() == 1 && OneLaunchSums(planned_[0], g)) {
    planned_.push_back(std::move(g));
    return;
  }
  if (!grad_.empty() || !planned_.empty()) {
    SumPlanned();
    AcceptSummed(g, SumOf(g));
    return;
  }
  planned_.push_back(std::move(g));
}

// Whether two unsummed gradients are the two inputs of one recis_csr_gather_reduce2* launch: of one
// plan and the same rows (one key), whole (no cover), each float32 or of the table's type, at most
// one of them in parts (which then has no coefficients and at most 8 parts).
bool Hashtable::OneLaunchSums(const PlannedGrad& a, const PlannedGrad& b) const {
  if (a.plan.get() != b.plan.get() || a.key == 0 || a.key != b.key || a.may_miss != b.may_miss ||
      a.cover.defined() || b.cover.defined()) {
    return false;
  }
  if (a.index.sizes() != b.index.sizes()) return false;
  if (a.in_parts && b.in_parts) return false;
  for (const PlannedGrad* g : {&a, &b}) {
    if (g->in_parts && (g->coef.defined() || g->rows.size() > 8)) return false;
    const auto t = g->rows[0].scalar_type();
    if (t != at::kFloat && t != dtype_) return false;
  }
  return true;
}

at::Tensor Hashtable::SumOf(const PlannedGrad& g) const {
  if (!g.in_parts) return recis::functional::csr_gather_reduce(g.rows[0], g.plan, g.src, g.coef, g.cover);
  return recis::functional::csr_gather_reduce_parts(g.rows, g.plan, g.src);
}

void Hashtable::AcceptSummed(const PlannedGrad& g, at::Tensor summed) {
  at::Tensor index = g.index.numel() > summed.size(0) ? g.index.narrow(0, 0, summed.size(0)) : g.index;
  if (g.may_miss) {  // keys the table does not hold take no gradient
    at::Tensor keep = index.ge(0);
    index = index.masked_select(keep);
    summed = summed.index({keep});
  }
  if (summed.scalar_type() != dtype_ && dtype_ == at::kFloat) summed = summed.to(dtype_);
  AcceptGradEx(index, summed, true, g.key);
}

void Hashtable::SumPlanned() {
  std::vector<PlannedGrad> planned;
  planned.swap(planned_);
  for (const auto& g : planned) AcceptSummed(g, SumOf(g));
}

std::vector<PlannedGrad> Hashtable::TakePlannedGrad() {
  if (planned_.empty() || !grad_.empty()) return {};
  if (planned_.size() == 1 && planned_[0].in_parts) return {};  // parts alone: no fused row update takes them
  std::vector<PlannedGrad> planned;
  planned.swap(planned_);
  if (planned.size() == 2 && planned[0].in_parts) std::swap(planned[0], planned[1]);
  return planned;
}

// The sparse COO gradient as the reference builds it (csrc/embedding/hashtable.cc:90-134),
// including its layout when rows repeat: the inverse positions as indices and an N-row value buffer
// whose first U rows hold the sums.
at::Tensor Hashtable::grad(int64_t accumulate_steps) {
  SumPlanned();
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
  SumPlanned();
  TORCH_CHECK(!grad_.empty(), "the table holds no gradient");
  at::Tensor index = grad_index_.size() == 1 ? grad_index_[0] : at::cat(grad_index_, 0);
  at::Tensor g = grad_.size() == 1 ? grad_[0] : at::cat(grad_, 0);
  if (!(grad_unique_.size() == 1 && grad_unique_[0])) {  // one gradient over distinct rows needs no merge
    auto uniq = at::_unique(index, /*sorted=*/false, /*return_inverse=*/true);
    if (std::get<0>(uniq).numel() != index.numel()) {
      std::vector<int64_t> shape = g.sizes().vec();
      shape[0] = std::get<0>(uniq).numel();
      at::Tensor summed = at::zeros(shape, g.options());
      summed.index_add_(0, std::get<1>(uniq).view({-1}), g);
      index = std::get<0>(uniq);
      g = summed;
    }
  }
  if (accumulate_steps != 1) g = g / accumulate_steps;
  return std::make_tuple(index, g);
}

void Hashtable::ClearGrad() {
  grad_index_.clear();
  grad_.clear();
  grad_unique_.clear();
  grad_keys_.clear();
  planned_.clear();
}

c10::intrusive_ptr<recis::embedding::Slot> Hashtable::GetSlot(const std::string& name) {
  return slot_group_->GetSlotByName(name);
}
