// torch.ops.recis.* on librecis_hip.so: argument checks, output allocation with the torch allocator
// on the current stream, then one or two calls through the C ABI. No operator here has a CPU
// branch: a CPU tensor is an error (the reference dispatches on tensor.device().is_cuda() inside
// every op; these are the device branches only).
#include "ops.h"

#include <c10/hip/HIPStream.h>

#include <cstring>
#include <map>
#include <mutex>

#include "abi_util.h"

namespace recis {
namespace hipabi {

const at::Tensor& check_blocks(const std::vector<at::Tensor>& blocks, int64_t block_size) {
  TORCH_CHECK(!blocks.empty(), "empty block list");
  const at::Tensor& b0 = blocks[0];
  for (const auto& b : blocks) {
    require_gpu(b, "blocks");
    TORCH_CHECK(b.scalar_type() == b0.scalar_type() && b.sizes().slice(1) == b0.sizes().slice(1) &&
                    rows_dense(b) && b.stride(0) == b0.stride(0) && b.device() == b0.device(),
                "blocks must hold contiguous rows at one pitch and share dtype, device and row shape");
    TORCH_CHECK(b.size(0) >= block_size, "block with ", b.size(0), " rows is smaller than block_size ",
                block_size);
  }
  return b0;
}

int64_t row_pitch_bytes(const at::Tensor& block) {
  return block.is_contiguous() ? 0 : block.stride(0) * static_cast<int64_t>(block.element_size());
}

int64_t shared_row_pitch_bytes(std::initializer_list<const at::Tensor*> first_blocks) {
  const at::Tensor& b0 = **first_blocks.begin();
  for (const at::Tensor* b : first_blocks)
    TORCH_CHECK(b->stride(0) == b0.stride(0) && b->scalar_type() == b0.scalar_type(),
                "slots that are updated together must share dtype and row pitch");
  return row_pitch_bytes(b0);
}

at::Tensor block_ptr_table(const std::vector<at::Tensor>& blocks) {
  static std::mutex mu;
  static std::map<std::vector<int64_t>, at::Tensor> cache;
  std::vector<int64_t> key;
  key.reserve(blocks.size() + 1);
  key.push_back(blocks[0].device().index());
  for (const auto& b : blocks) key.push_back(reinterpret_cast<int64_t>(b.data_ptr()));
  std::lock_guard<std::mutex> lock(mu);
  auto it = cache.find(key);
  if (it != cache.end()) return it->second;
  if (cache.size() > 256) cache.clear();
  at::Tensor host = at::empty({static_cast<int64_t>(blocks.size())}, at::TensorOptions().dtype(at::kLong));
  std::memcpy(host.data_ptr(), key.data() + 1, blocks.size() * sizeof(int64_t));
  at::Tensor table = host.to(blocks[0].device());
  cache.emplace(std::move(key), table);
  return table;
}

std::vector<int64_t> host_values(const at::Tensor& t) {
  at::Tensor h = t.reshape({-1}).to(at::kCPU, at::kLong).contiguous();
  const int64_t* p = h.data_ptr<int64_t>();
  return std::vector<int64_t>(p, p + h.numel());
}

}  // namespace hipabi

namespace functional {

using namespace recis::hipabi;

namespace {

std::mutex g_unique_mu;  // guards the notes of ids_partition's outputs (note_unique / note_partition)

int mode_code(const std::string& mode) {
  if (mode == "sum") return RECIS_SUM;
  if (mode == "mean") return RECIS_MEAN;
  if (mode == "tile") return RECIS_TILE;
  if (mode == "max") return RECIS_MAX;
  TORCH_CHECK(false, "Invalid mode: ", mode);
}

// NULL means "identity" to the library and an empty tensor has a NULL data pointer too: hand over
// another valid pointer, with zero occurrences it is never dereferenced.
const void* rev_ptr(const Tensor& rev, const Tensor& other) {
  return rev.numel() ? rev.data_ptr() : other.data_ptr();
}

Tensor opt_contig(const c10::optional<Tensor>& t, const char* name) {
  if (!t.has_value() || !t->defined()) return Tensor();
  require_gpu(*t, name);
  return t->contiguous();
}

}  // namespace

// ------------------------------------------------------------------------------------ pooling
Tensor segment_reduce_forward(Tensor unique_emb, c10::optional<Tensor> weight, Tensor reverse_indices,
                              Tensor offsets, std::string mode) {
  require_gpu(unique_emb, "unique_emb");
  require_gpu(reverse_indices, "reverse_indices");
  require_gpu(offsets, "offsets");
  TORCH_CHECK(unique_emb.dim() == 2, "unique_emb must be [U, D]");
  const int m = mode_code(mode);
  c10::DeviceGuard guard(unique_emb.device());
  unique_emb = unique_emb.contiguous();
  reverse_indices = reverse_indices.contiguous();
  offsets = offsets.contiguous();
  Tensor w = opt_contig(weight, "weight");
  const int64_t U = unique_emb.size(0), D = unique_emb.size(1);
  const int64_t S = offsets.numel() - 1, B = reverse_indices.numel();
  Tensor out = at::empty({m == RECIS_TILE ? B : S, D}, unique_emb.options());
  check(recis_segment_reduce_forward(
      unique_emb.data_ptr(), dtype_code(unique_emb.scalar_type()), w.defined() ? w.data_ptr() : nullptr,
      w.defined() ? dtype_code(w.scalar_type()) : 0, rev_ptr(reverse_indices, offsets),
      index_kind(reverse_indices, "reverse_indices"), offsets.data_ptr(), index_kind(offsets, "offsets"),
      out.data_ptr(), dtype_code(out.scalar_type()), nullptr, B, U, S, D, m, stream_of(out.device())));
  return out;
}

Tensor segment_reduce_backward(Tensor grad_output, c10::optional<Tensor> weight, Tensor reverse_indices,
                               Tensor offsets, int64_t unique_size, std::string mode) {
  require_gpu(grad_output, "grad_output");
  require_gpu(reverse_indices, "reverse_indices");
  require_gpu(offsets, "offsets");
  TORCH_CHECK(grad_output.dim() == 2, "grad_output must be 2-dim");
  const int m = mode_code(mode);
  TORCH_CHECK(m != RECIS_MAX, "the max combiner's backward needs the forward's argmax: use the C ABI");
  c10::DeviceGuard guard(grad_output.device());
  grad_output = grad_output.contiguous();
  reverse_indices = reverse_indices.contiguous();
  offsets = offsets.contiguous();
  Tensor w = opt_contig(weight, "weight");
  const int64_t D = grad_output.size(1), S = offsets.numel() - 1, B = reverse_indices.numel();
  {
    // reverse_indices as ids_partition handed them out, untouched since: the occurrence lists of that
    // dedup are still there, so the gradient of every unique id is a gather-reduce over its list (no
    // atomics), each row stored at its place in the sorted order of the unique ids
    BatchPlanPtr plan;
    Tensor rank;
    if ((m == RECIS_SUM || m == RECIS_MEAN) && known_partition(reverse_indices, &plan, &rank) &&
        plan->U() == unique_size && rank.numel() == unique_size) {
      auto sc = plan->SrcCoefForPool(offsets, w.defined() ? c10::optional<Tensor>(w) : c10::nullopt, m == RECIS_MEAN);
      Tensor coef = std::get<1>(sc).has_value() ? *std::get<1>(sc) : Tensor();
      Tensor out = csr_gather_reduce(grad_output, plan, std::get<0>(sc), coef, Tensor(), rank);
      return grad_output.scalar_type() == at::kFloat ? out : out.to(grad_output.scalar_type());
    }
  }
  // duplicates in reverse_indices are accumulated with fp32 atomics, whatever the gradient's type
  Tensor out = at::empty({unique_size, D}, grad_output.options().dtype(at::kFloat));
  check(recis_segment_reduce_backward(
      grad_output.data_ptr(), dtype_code(grad_output.scalar_type()), w.defined() ? w.data_ptr() : nullptr,
      w.defined() ? dtype_code(w.scalar_type()) : 0, rev_ptr(reverse_indices, offsets),
      index_kind(reverse_indices, "reverse_indices"), offsets.data_ptr(), index_kind(offsets, "offsets"), nullptr,
      out.data_ptr(), RECIS_F32, B, unique_size, S, D, m, 0, stream_of(out.device())));
  return grad_output.scalar_type() == at::kFloat ? out : out.to(grad_output.scalar_type());
}

Tensor merge_offsets(const TensorList& offsets, Tensor& max_value) {
  TORCH_CHECK(!offsets.empty(), "merge_offsets: empty list");
  require_gpu(offsets, "offsets");
  TensorList offs;
  for (const auto& o : offsets) {
    TORCH_CHECK(o.scalar_type() == offsets[0].scalar_type(), "offsets must share one integer dtype");
    offs.push_back(o.contiguous());
  }
  c10::DeviceGuard guard(offs[0].device());
  const int is64 = index_kind(offs[0], "offsets");
  std::vector<int64_t> mv = host_values(max_value);
  const int64_t n = static_cast<int64_t>(offs.size());
  TORCH_CHECK(static_cast<int64_t>(mv.size()) >= n, "max_value has ", mv.size(), " entries for ", n, " offsets");
  std::vector<int64_t> sizes = numels(offs);
  int64_t total = -(n - 1);
  for (int64_t s : sizes) total += s;
  Tensor out = at::empty({total}, offs[0].options());
  auto ptrs = host_ptrs<void>(offs);
  check(recis_merge_offsets(ptrs.data(), sizes.data(), mv.data(), n, is64, out.data_ptr(),
                            stream_of(out.device())));
  return out;
}

Tensor gen_segment_indices_by_offset(Tensor offset) {
  require_gpu(offset, "offset");
  c10::DeviceGuard guard(offset.device());
  offset = offset.contiguous();
  const int64_t S = offset.numel() - 1;
  // the reference reads the total back too (embedding_segment_reduce_kernel.cu:405)
  const int64_t total = S >= 0 ? offset[S].item<int64_t>() : 0;
  Tensor out = at::empty({total}, offset.options());
  check(recis_gen_segment_indices(offset.data_ptr(), index_kind(offset, "offset"), S, out.data_ptr(), total,
                                  stream_of(out.device())));
  return out;
}

Tensor segment_sum(Tensor data, c10::optional<Tensor> weight, Tensor indices, Tensor segment_ids,
                   at::Scalar num_segments) {
  require_gpu(data, "data");
  require_gpu(indices, "indices");
  require_gpu(segment_ids, "segment_ids");
  TORCH_CHECK(indices.scalar_type() == segment_ids.scalar_type(), "indices and segment_ids must share a dtype");
  TORCH_CHECK(data.dim() == 2, "data must be 2-dim");
  c10::DeviceGuard guard(data.device());
  data = data.contiguous();
  indices = indices.contiguous();
  segment_ids = segment_ids.contiguous();
  Tensor w = opt_contig(weight, "weight");
  const int64_t n_seg = num_segments.toLong(), D = data.size(1);
  Tensor out = at::empty({n_seg, D}, data.options().dtype(at::kFloat));
  check(recis_segment_sum(data.data_ptr(), dtype_code(data.scalar_type()), data.size(0),
                          w.defined() ? w.data_ptr() : nullptr, w.defined() ? dtype_code(w.scalar_type()) : 0,
                          w.defined() ? 1 : 0, indices.data_ptr(), segment_ids.data_ptr(),
                          index_kind(indices, "indices"), out.data_ptr<float>(), indices.numel(), n_seg, D,
                          stream_of(out.device())));
  return data.scalar_type() == at::kFloat ? out : out.to(data.scalar_type());
}

Tensor segment_mean(Tensor data, c10::optional<Tensor> weight, Tensor segment_ids, at::Scalar num_segments) {
  require_gpu(data, "data");
  require_gpu(segment_ids, "segment_ids");
  c10::DeviceGuard guard(data.device());
  segment_ids = segment_ids.contiguous();
  Tensor w = opt_contig(weight, "weight");
  const bool use_w = w.defined();
  w = use_w ? w.to(at::kFloat) : at::ones({1}, data.options().dtype(at::kFloat));
  const int64_t n_seg = num_segments.toLong(), n = segment_ids.numel();
  Tensor wsum = at::empty({n_seg}, w.options());
  Tensor wnorm = at::empty({n}, w.options());
  check(recis_segment_mean_weight(w.data_ptr<float>(), use_w ? 1 : 0, segment_ids.data_ptr(),
                                  index_kind(segment_ids, "segment_ids"), wsum.data_ptr<float>(),
                                  wnorm.data_ptr<float>(), n, n_seg, stream_of(w.device())));
  return data.scalar_type() == at::kFloat ? wnorm : wnorm.to(data.scalar_type());
}

// ------------------------------------------------------------------------------------ row blocks
Tensor gather(const Tensor ids, const Tensor emb) {
  require_gpu(ids, "ids");
  require_gpu(emb, "emb");
  c10::DeviceGuard guard(emb.device());
  Tensor i = ids.contiguous().view({-1}), e = emb.contiguous();
  std::vector<int64_t> shape = e.sizes().vec();
  TORCH_CHECK(!shape.empty(), "emb must have at least one dimension");
  shape[0] = i.numel();
  Tensor out = at::empty(shape, e.options());
  check(recis_gather(i.data_ptr(), index_kind(i, "ids"), e.data_ptr(), e.size(0), out.data_ptr(), i.numel(),
                     row_bytes(e), stream_of(e.device())));
  return out;
}

Tensor block_gather(const Tensor ids, TensorList emb_blocks, int64_t block_size, int64_t default_key,
                    bool readonly) {
  const Tensor& b0 = check_blocks(emb_blocks, block_size);
  c10::DeviceGuard guard(b0.device());
  Tensor i = flat_i64(ids, "ids");
  std::vector<int64_t> shape = b0.sizes().vec();
  shape[0] = i.numel();
  Tensor out = at::empty(shape, b0.options());
  Tensor tab = block_ptr_table(emb_blocks);
  check(recis_block_gather(i.data_ptr<int64_t>(), static_cast<void* const*>(tab.data_ptr()),
                           static_cast<int64_t>(emb_blocks.size()), block_size, row_pitch_bytes(b0), default_key,
                           readonly ? 1 : 0,
                           out.data_ptr(), i.numel(), row_bytes(b0), stream_of(b0.device())));
  return out;
}

namespace {
void block_insert_impl(const Tensor& ids, const Tensor& embedding, const Tensor* mask, TensorList& emb_blocks,
                       int64_t block_size) {
  const Tensor& b0 = check_blocks(emb_blocks, block_size);
  c10::DeviceGuard guard(b0.device());
  Tensor i = flat_i64(ids, "ids");
  require_gpu(embedding, "embedding");
  TORCH_CHECK(embedding.scalar_type() == b0.scalar_type(), "embedding dtype ", embedding.scalar_type(),
              " does not match the blocks (", b0.scalar_type(), ")");
  Tensor e = embedding.contiguous();
  TORCH_CHECK(e.dim() >= 1 && (e.size(0) == i.numel() || e.size(0) == 1),
              "ids batch_size must = embedding batch size or embedding batch size = 1");
  Tensor m;
  if (mask != nullptr) {
    require_gpu(*mask, "mask");
    TORCH_CHECK(mask->scalar_type() == at::kBool, "mask must be bool");
    m = mask->contiguous();
  }
  const int broadcast = (mask == nullptr && e.size(0) == 1 && i.numel() != 1) ? 1 : 0;
  Tensor tab = block_ptr_table(emb_blocks);
  check(recis_block_insert(i.data_ptr<int64_t>(), e.data_ptr(), broadcast,
                           m.defined() ? static_cast<const uint8_t*>(m.data_ptr()) : nullptr,
                           static_cast<void* const*>(tab.data_ptr()), static_cast<int64_t>(emb_blocks.size()),
                           block_size, row_pitch_bytes(b0), i.numel(), row_bytes(b0), stream_of(b0.device())));
}
}  // namespace

void block_insert(const Tensor ids, const Tensor embedding, TensorList emb_blocks, int64_t block_size) {
  block_insert_impl(ids, embedding, nullptr, emb_blocks, block_size);
}

void block_insert_with_mask(const Tensor ids, const Tensor embedding, const Tensor mask, TensorList emb_blocks,
                            int64_t block_size) {
  block_insert_impl(ids, embedding, &mask, emb_blocks, block_size);
}

Tensor block_filter(const Tensor ids, TensorList emb_blocks, int64_t block_size, int64_t step) {
  const Tensor& b0 = check_blocks(emb_blocks, block_size);
  TORCH_CHECK((b0.scalar_type() == at::kInt || b0.scalar_type() == at::kLong) &&
                  row_bytes(b0) == static_cast<int64_t>(b0.element_size()),
              "block_filter needs an int32/int64 slot of width 1");
  c10::DeviceGuard guard(b0.device());
  Tensor i = flat_i64(ids, "ids");
  Tensor out = at::empty({i.numel()}, b0.options().dtype(at::kBool));
  Tensor tab = block_ptr_table(emb_blocks);
  check(recis_block_filter(i.data_ptr<int64_t>(), static_cast<void* const*>(tab.data_ptr()),
                           static_cast<int64_t>(emb_blocks.size()), block_size, step,
                           b0.scalar_type() == at::kLong ? 1 : 0, static_cast<uint8_t*>(out.data_ptr()), i.numel(),
                           stream_of(b0.device())));
  return out;
}

// ------------------------------------------------------------------------------------ optimizers
void block_apply_adamw(const Tensor index, const Tensor grad, TensorList emb_blocks, Tensor beta1_t,
                       Tensor beta2_t, Tensor step, TensorList exp_avg, TensorList exp_avg_sq, double lr,
                       double beta1, double beta2, double weight_decay, double eps, int64_t block_size) {
  (void)step;  // accepted and left untouched, as in the reference (block_apply_adamw_op.cc:121)
  const Tensor& b0 = check_blocks(emb_blocks, block_size);
  check_blocks(exp_avg, block_size);
  check_blocks(exp_avg_sq, block_size);
  TORCH_CHECK(exp_avg.size() == emb_blocks.size() && exp_avg_sq.size() == emb_blocks.size(),
              "state slots must have as many blocks as the embedding slot");
  c10::DeviceGuard guard(b0.device());
  Tensor i = flat_i64(index, "index");
  require_gpu(grad, "grad");
  require_gpu(beta1_t, "beta1_t");
  require_gpu(beta2_t, "beta2_t");
  TORCH_CHECK(beta1_t.scalar_type() == beta2_t.scalar_type() &&
                  (beta1_t.scalar_type() == at::kFloat || beta1_t.scalar_type() == at::kDouble),
              "beta1_t / beta2_t must both be float32 or float64");
  Tensor g = grad.contiguous();
  const int64_t D = row_bytes(b0) / static_cast<int64_t>(b0.element_size());
  TORCH_CHECK(g.numel() == i.numel() * D, "grad has ", g.numel(), " elements, expected ", i.numel(), " x ", D);
  Tensor t0 = block_ptr_table(emb_blocks), t1 = block_ptr_table(exp_avg), t2 = block_ptr_table(exp_avg_sq);
  // rows of doubles (the reference's functor is dispatched for them too) go with gradients of doubles
  auto code = [&](at::ScalarType t) {
    return t == at::kDouble && b0.scalar_type() == at::kDouble ? RECIS_F64 : dtype_code(t);
  };
  check(recis_block_apply_adamw(i.data_ptr<int64_t>(), g.data_ptr(), code(g.scalar_type()),
                                static_cast<void* const*>(t0.data_ptr()), static_cast<void* const*>(t1.data_ptr()),
                                static_cast<void* const*>(t2.data_ptr()), static_cast<int64_t>(emb_blocks.size()),
                                block_size, shared_row_pitch_bytes({&b0, &exp_avg[0], &exp_avg_sq[0]}),
                                code(b0.scalar_type()), beta1_t.data_ptr(), beta2_t.data_ptr(),
                                beta1_t.scalar_type() == at::kDouble ? 1 : 0, lr, beta1, beta2, weight_decay, eps,
                                i.numel(), D, stream_of(b0.device())));
}

void block_apply_adagrad(const Tensor index, const Tensor grad, TensorList emb_blocks, TensorList accum,
                         double lr, double eps, int64_t block_size) {
  const Tensor& b0 = check_blocks(emb_blocks, block_size);
  check_blocks(accum, block_size);
  TORCH_CHECK(accum.size() == emb_blocks.size(), "state slot must have as many blocks as the embedding slot");
  c10::DeviceGuard guard(b0.device());
  Tensor i = flat_i64(index, "index");
  require_gpu(grad, "grad");
  Tensor g = grad.contiguous();
  const int64_t D = row_bytes(b0) / static_cast<int64_t>(b0.element_size());
  TORCH_CHECK(g.numel() == i.numel() * D, "grad has ", g.numel(), " elements, expected ", i.numel(), " x ", D);
  Tensor t0 = block_ptr_table(emb_blocks), t1 = block_ptr_table(accum);
  check(recis_block_apply_adagrad(i.data_ptr<int64_t>(), g.data_ptr(), dtype_code(g.scalar_type()),
                                  static_cast<void* const*>(t0.data_ptr()), static_cast<void* const*>(t1.data_ptr()),
                                  static_cast<int64_t>(emb_blocks.size()), block_size,
                                  shared_row_pitch_bytes({&b0, &accum[0]}), dtype_code(b0.scalar_type()), lr, eps,
                                  i.numel(), D, stream_of(b0.device())));
}

// ------------------------------------------------------------------------------------ allocator ops
Tensor generate_ids_op(const int64_t gen_num, TensorList free_blocks, const int64_t free_count,
                       const int64_t cur_count, const int64_t free_block_size) {
  TORCH_CHECK(!free_blocks.empty(), "generate_ids: empty free-block list");
  require_gpu(free_blocks, "free_blocks");
  c10::DeviceGuard guard(free_blocks[0].device());
  Tensor out = at::empty({gen_num}, free_blocks[0].options().dtype(at::kLong));
  Tensor tab = block_ptr_table(free_blocks);
  check(recis_generate_ids(gen_num, static_cast<const int64_t* const*>(tab.data_ptr()), free_count, cur_count,
                           free_block_size, out.data_ptr<int64_t>(), stream_of(out.device())));
  return out;
}

void free_ids_op(Tensor free_ids, TensorList free_blocks, const int64_t free_count,
                 const int64_t free_block_size) {
  TORCH_CHECK(!free_blocks.empty(), "free_ids: empty free-block list");
  require_gpu(free_blocks, "free_blocks");
  c10::DeviceGuard guard(free_blocks[0].device());
  Tensor i = flat_i64(free_ids, "free_ids");
  Tensor tab = block_ptr_table(free_blocks);
  check(recis_free_ids(i.data_ptr<int64_t>(), i.numel(), static_cast<int64_t* const*>(tab.data_ptr()), free_count,
                       free_block_size, stream_of(i.device())));
}

std::tuple<Tensor, Tensor> mask_key_index_op(Tensor in_keys, Tensor mask, Tensor out_index, int64_t out_size) {
  Tensor k = flat_i64(in_keys, "in_keys"), c = flat_i64(out_index, "in_out_index");
  require_gpu(mask, "mask");
  TORCH_CHECK(mask.scalar_type() == at::kBool, "mask must be bool");
  c10::DeviceGuard guard(k.device());
  Tensor m = mask.contiguous();
  Tensor out_keys = at::empty({out_size}, k.options());
  Tensor out_idx = at::empty({out_size}, k.options());
  check(recis_mask_key_index(k.data_ptr<int64_t>(), static_cast<const uint8_t*>(m.data_ptr()),
                             c.data_ptr<int64_t>(), k.numel(), out_size, out_keys.data_ptr<int64_t>(),
                             out_idx.data_ptr<int64_t>(), stream_of(k.device())));
  return std::make_tuple(out_keys, out_idx);
}

Tensor scatter_ids_with_mask_op(Tensor out_ids, Tensor in_ids, Tensor mask_index) {
  require_gpu(out_ids, "out_ids");
  TORCH_CHECK(out_ids.is_contiguous() && out_ids.scalar_type() == at::kLong, "out_ids must be contiguous int64");
  c10::DeviceGuard guard(out_ids.device());
  Tensor i = flat_i64(in_ids, "in_ids"), p = flat_i64(mask_index, "mask_index");
  check(recis_scatter_ids_with_mask(out_ids.data_ptr<int64_t>(), out_ids.numel(), i.data_ptr<int64_t>(),
                                    p.data_ptr<int64_t>(), i.numel(), stream_of(out_ids.device())));
  return out_ids;
}

// ------------------------------------------------------------------------------------ tagging / dedup
Tensor ids_encode(TensorList inputs, Tensor table_ids) {
  TORCH_CHECK(!inputs.empty(), "ids_encode: empty list");
  TensorList ids;
  for (const auto& t : inputs) ids.push_back(flat_i64(t, "ids"));
  c10::DeviceGuard guard(ids[0].device());
  std::vector<int64_t> tids = host_values(table_ids);
  TORCH_CHECK(tids.size() >= ids.size(), "table_ids has ", tids.size(), " entries for ", ids.size(), " tensors");
  std::vector<int64_t> sizes = numels(ids);
  int64_t total = 0;
  for (int64_t s : sizes) total += s;
  Tensor out = at::empty({total}, ids[0].options());
  auto ptrs = host_ptrs<int64_t>(ids);
  check(recis_ids_encode(ptrs.data(), sizes.data(), tids.data(), static_cast<int64_t>(ids.size()),
                         out.data_ptr<int64_t>(), stream_of(out.device())));
  return out;
}

// Device ordering of the reference (ids_partition_kernel.cu:36-55): unique ids ascending by
// rotr64(id, 16) taken as unsigned, i.e. by shard slot (id & 0xFFFF) first; counts per shard; int32
// inverse. The dedup is the library's hash kernel; only the unique set is sorted.
std::tuple<Tensor, Tensor, Tensor> ids_partition(const Tensor& ids, int64_t num_parts) {
  TORCH_CHECK(ids.dim() == 1, "ids must be 1-dim");
  TORCH_CHECK(num_parts >= 1, "num_parts must be positive");
  Tensor i = flat_i64(ids, "ids");
  c10::DeviceGuard guard(i.device());
  // the dedup is a batch plan: its occurrence lists are kept (see note_partition) so that the backward
  // over this call's inverse can be a gather-reduce per unique id instead of an atomic scatter
  BatchPlanPtr plan = BatchPlan::Make({i}, c10::nullopt, nullptr, /*wait=*/true, /*need_inverse=*/true,
                                      /*need_pos=*/false);
  const int64_t U = plan->U();
  Tensor u = plan->unique();
  Tensor inv = plan->inverse();
  // only the unique set is sorted: a radix sort of (rotated id, position) pairs
  Tensor sorted_u = at::empty({U}, u.options());
  Tensor order = at::empty({U}, u.options().dtype(at::kInt));
  Tensor rank = at::empty({U}, order.options());
  check(recis_partition_order(u.data_ptr<int64_t>(), U, sorted_u.data_ptr<int64_t>(), order.data_ptr<int32_t>(),
                              rank.data_ptr<int32_t>(), stream_of(i.device())));
  Tensor counts;
  if (num_parts == 1) {
    counts = at::full({1}, U, u.options());
  } else {
    const int64_t slice = 65536, m = slice / num_parts, r = slice % num_parts;
    Tensor slot = at::bitwise_and(sorted_u, slice - 1);
    Tensor part = m > 0 ? at::maximum(at::div(slot, m + 1, "floor"), at::div(slot - r, m, "trunc"))
                        : at::div(slot, m + 1, "floor");
    counts = at::bincount(part, {}, num_parts).to(at::kLong);
  }
  // inverse[i] = rank of the unique id of occurrence i: 4-byte rows out of the rank table, by the
  // library's own row gather (torch's index_select took 190 us for 2.6 M of them)
  Tensor inverse = at::empty({i.numel()}, rank.options());
  if (i.numel() > 0)
    check(recis_gather(inv.data_ptr(), index_kind(inv, "inverse"), rank.data_ptr(), U, inverse.data_ptr(), i.numel(),
                       sizeof(int32_t), stream_of(i.device())));
  note_unique(sorted_u);
  note_partition(inverse, plan, rank);
  return std::make_tuple(sorted_u, counts, inverse);
}

namespace {
struct NotedPartition {
  Tensor inverse;
  uint32_t version;
  BatchPlanPtr plan;
  Tensor rank;  // the plan's unique id -> its position in the sorted order
};
std::vector<NotedPartition> g_noted_partitions;  // the last few, newest last
}  // namespace

void note_partition(const Tensor& inverse, const BatchPlanPtr& plan, const Tensor& rank) {
  std::lock_guard<std::mutex> lock(g_unique_mu);
  if (g_noted_partitions.size() >= 2) g_noted_partitions.erase(g_noted_partitions.begin());
  g_noted_partitions.push_back({inverse, inverse._version(), plan, rank});
}

bool known_partition(const Tensor& inverse, BatchPlanPtr* plan, Tensor* rank) {
  if (!inverse.defined() || inverse.numel() == 0) return false;
  std::lock_guard<std::mutex> lock(g_unique_mu);
  for (const auto& e : g_noted_partitions) {
    if (e.inverse.data_ptr() == inverse.data_ptr() && e.inverse.numel() == inverse.numel() &&
        e.inverse.scalar_type() == inverse.scalar_type() && inverse.is_contiguous() &&
        e.version == inverse._version() && e.inverse._version() == e.version) {
      *plan = e.plan;
      *rank = e.rank;
      return true;
    }
  }
  return false;
}

namespace {
struct NotedUnique {
  Tensor t;
  uint32_t version;
};
std::vector<NotedUnique> g_noted_unique;  // the last few, newest last
}  // namespace

void note_unique(const Tensor& t) {
  std::lock_guard<std::mutex> lock(g_unique_mu);
  if (g_noted_unique.size() >= 4) g_noted_unique.erase(g_noted_unique.begin());
  g_noted_unique.push_back({t, t._version()});
}

bool known_unique(const Tensor& t) {
  if (!t.defined() || t.numel() == 0) return t.defined();
  std::lock_guard<std::mutex> lock(g_unique_mu);
  for (const auto& e : g_noted_unique) {
    if (e.t.data_ptr() == t.data_ptr() && e.t.numel() == t.numel() && e.t.scalar_type() == t.scalar_type() &&
        t.is_contiguous() && e.version == t._version() && e.t._version() == e.version) {
      return true;
    }
  }
  return false;
}

// ------------------------------------------------------------------------------------ over a batch plan
Tensor csr_gather_reduce(const Tensor& rows_in, const BatchPlanPtr& plan, const Tensor& src, const Tensor& coef,
                         const Tensor& cover, const Tensor& out_rows) {
  require_gpu(rows_in, "rows");
  require_gpu(src, "src");
  TORCH_CHECK(rows_in.dim() == 2, "gradient rows must be [rows, D]");
  c10::DeviceGuard guard(rows_in.device());
  Tensor rows = rows_in.contiguous();
  const int64_t D = rows.size(1), U = plan->U();
  Tensor out = at::empty({U, D}, rows.options().dtype(at::kFloat));
  const void* coef_p = coef.defined() ? coef.data_ptr() : nullptr;
  const int coef_dt = coef.defined() ? dtype_code(coef.scalar_type()) : 0;
  const void* cover_p = cover.defined() ? cover.data_ptr() : nullptr;
  const int cover64 = cover.defined() ? index_kind(cover, "offsets") : 0;
  const int64_t cover_S = cover.defined() ? cover.numel() - 1 : 0;
  if (out_rows.defined()) {
    require_gpu(out_rows, "out_rows");
    TORCH_CHECK(out_rows.scalar_type() == at::kInt && out_rows.is_contiguous() && out_rows.numel() >= U,
                "out_rows must be a contiguous int32 tensor with an entry per unique id");
    check(recis_csr_gather_reduce_mapped(
        rows.data_ptr(), dtype_code(rows.scalar_type()), rows.size(0), src.data_ptr<int32_t>(), coef_p, coef_dt,
        plan->row_start().data_ptr<int32_t>(), plan->hot_items().data_ptr<int32_t>(), plan->hot_cap(),
        plan->counts().data_ptr<int64_t>(), out.data_ptr(), RECIS_F32, U, D, 0, cover_p, cover64, cover_S,
        out_rows.data_ptr<int32_t>(), stream_of(rows.device())));
  } else {
    check(recis_csr_gather_reduce(
        rows.data_ptr(), dtype_code(rows.scalar_type()), rows.size(0), src.data_ptr<int32_t>(), coef_p, coef_dt,
        plan->row_start().data_ptr<int32_t>(), plan->hot_items().data_ptr<int32_t>(), plan->hot_cap(),
        plan->counts().data_ptr<int64_t>(), out.data_ptr(), RECIS_F32, U, D, 0, cover_p, cover64, cover_S,
        stream_of(rows.device())));
  }
  return out;
}

Tensor csr_gather_reduce_parts(const TensorList& parts_in, const BatchPlanPtr& plan, const Tensor& src) {
  TORCH_CHECK(!parts_in.empty() && parts_in.size() <= 8, "csr_gather_reduce_parts: 1 to 8 parts");
  require_gpu(parts_in, "parts");
  require_gpu(src, "src");
  TensorList parts;
  for (const auto& p : parts_in) {
    TORCH_CHECK(p.dim() == 2 && p.scalar_type() == parts_in[0].scalar_type() && p.size(1) == parts_in[0].size(1),
                "csr_gather_reduce_parts: the parts must be [rows, D] tensors of one dtype and row width");
    parts.push_back(p.contiguous());
  }
  c10::DeviceGuard guard(parts[0].device());
  const int64_t D = parts[0].size(1), U = plan->U();
  Tensor out = at::empty({U, D}, parts[0].options().dtype(at::kFloat));
  auto ptrs = host_ptrs<void>(parts);
  std::vector<int64_t> counts;
  for (const auto& p : parts) counts.push_back(p.size(0));
  check(recis_csr_gather_reduce_parts(ptrs.data(), counts.data(), static_cast<int>(parts.size()),
                                      dtype_code(parts[0].scalar_type()), src.data_ptr<int32_t>(),
                                      plan->row_start().data_ptr<int32_t>(), plan->hot_items().data_ptr<int32_t>(),
                                      plan->hot_cap(), plan->counts().data_ptr<int64_t>(), out.data_ptr(), U, D, 0,
                                      stream_of(parts[0].device())));
  return out;
}

// ------------------------------------------------------------------------------------ feature ops
TensorList fused_uint64_mod(TensorList inputs, Tensor mod_vec) {
  if (inputs.empty()) return {};
  TensorList in;
  for (const auto& t : inputs) in.push_back(flat_i64(t, "inputs"));
  c10::DeviceGuard guard(in[0].device());
  std::vector<int64_t> mods = host_values(mod_vec);
  TORCH_CHECK(mods.size() >= in.size(), "mod_vec has ", mods.size(), " entries for ", in.size(), " tensors");
  std::vector<int64_t> sizes = numels(in);
  int64_t total = 0;
  for (int64_t s : sizes) total += s;
  // one allocation for the whole list, one view per tensor
  TensorList outs = at::empty({total}, in[0].options()).split_with_sizes(sizes);
  for (size_t k = 0; k < outs.size(); ++k) outs[k] = outs[k].view(inputs[k].sizes());
  auto ip = host_ptrs<int64_t>(in);
  auto op = host_mut_ptrs<int64_t>(outs);
  check(recis_fused_uint64_mod(ip.data(), sizes.data(), mods.data(), op.data(), static_cast<int64_t>(in.size()),
                               stream_of(in[0].device())));
  return outs;
}

Tensor uint64_mod(Tensor inputs, at::Scalar num) {
  Tensor mod = at::empty({1}, at::TensorOptions().dtype(at::kLong));
  mod.data_ptr<int64_t>()[0] = num.toLong();
  return fused_uint64_mod({inputs}, mod)[0];
}

namespace {
TensorList bucketized_impl(const TensorList& inputs, const TensorList& boundaries, const std::vector<int64_t>* mods);
}

TensorList fused_bucketized(TensorList inputs, TensorList boundaries) {
  return bucketized_impl(inputs, boundaries, nullptr);
}

TensorList fused_bucketized_mod(TensorList inputs, TensorList boundaries, std::vector<int64_t> mods) {
  TORCH_CHECK(mods.size() == inputs.size(), "fused_bucketized_mod: ", mods.size(), " mods for ", inputs.size(), " tensors");
  return bucketized_impl(inputs, boundaries, &mods);
}

namespace {
TensorList bucketized_impl(const TensorList& inputs, const TensorList& boundaries, const std::vector<int64_t>* mods) {
  if (inputs.empty()) return {};
  TORCH_CHECK(inputs.size() == boundaries.size(), "fused_bucketized: one boundary tensor per input");
  require_gpu(inputs, "inputs");
  require_gpu(boundaries, "boundaries");
  TensorList in, bd;
  for (const auto& t : inputs) {
    TORCH_CHECK(t.scalar_type() == at::kFloat, "fused_bucketized takes float32 values and boundaries");
    in.push_back(t.contiguous().view({-1}));
  }
  for (const auto& b : boundaries) {
    TORCH_CHECK(b.scalar_type() == at::kFloat, "fused_bucketized takes float32 values and boundaries");
    bd.push_back(b.contiguous());
  }
  c10::DeviceGuard guard(in[0].device());
  std::vector<int64_t> sizes = numels(in), blens = numels(bd);
  int64_t total = 0;
  for (int64_t s : sizes) total += s;
  // the outputs are views of ONE buffer, as in the reference (fused_bucketized.cc:47-52)
  TensorList outs = at::empty({total}, in[0].options().dtype(at::kLong)).split_with_sizes(sizes);
  auto ip = host_ptrs<float>(in);
  auto bp = host_ptrs<float>(bd);
  auto op = host_mut_ptrs<int64_t>(outs);
  check(recis_fused_bucketized_mod(ip.data(), sizes.data(), bp.data(), blens.data(), mods ? mods->data() : nullptr,
                                   op.data(), static_cast<int64_t>(in.size()), stream_of(in[0].device())));
  return outs;
}
}  // namespace

Tensor bucketize_op(Tensor values, Tensor boundaries) {
  return fused_bucketized({values.to(at::kFloat)}, {boundaries.to(at::kFloat)})[0].view(values.sizes());
}

TensorList fused_multi_hash(TensorList inputs, TensorList muls, TensorList primes, TensorList bucket_num) {
  TORCH_CHECK(inputs.size() == muls.size() && inputs.size() == primes.size() && inputs.size() == bucket_num.size(),
              "fused_multi_hash: one muls / primes / bucket_num tensor per input");
  if (inputs.empty()) return {};
  TensorList jobs_in, jobs_out;
  std::vector<int64_t> sizes, m, p, b;
  for (size_t k = 0; k < inputs.size(); ++k) {
    Tensor t = flat_i64(inputs[k], "inputs");
    std::vector<int64_t> tm = host_values(muls[k]), tp = host_values(primes[k]), tb = host_values(bucket_num[k]);
    TORCH_CHECK(tm.size() == tp.size() && tm.size() == tb.size(), "muls / primes / bucket_num differ in length");
    for (size_t j = 0; j < tm.size(); ++j) {
      jobs_in.push_back(t);
      jobs_out.push_back(at::empty_like(t));
      sizes.push_back(t.numel());
      m.push_back(tm[j]);
      p.push_back(tp[j]);
      b.push_back(tb[j]);
    }
  }
  if (jobs_in.empty()) return {};
  c10::DeviceGuard guard(jobs_in[0].device());
  auto ip = host_ptrs<int64_t>(jobs_in);
  auto op = host_mut_ptrs<int64_t>(jobs_out);
  check(recis_fused_multi_hash(ip.data(), sizes.data(), m.data(), p.data(), b.data(), op.data(),
                               static_cast<int64_t>(jobs_in.size()), stream_of(jobs_in[0].device())));
  return jobs_out;
}

TensorList fused_hash(TensorList inputs, TensorList input_offsets, const std::string& hash_type) {
  TORCH_CHECK(hash_type == "farm" || hash_type == "murmur", "Unsupported hash type: ", hash_type);
  TORCH_CHECK(inputs.size() == input_offsets.size(), "fused_hash: one offsets tensor per input");
  if (inputs.empty()) return {};
  require_gpu(inputs, "inputs");
  require_gpu(input_offsets, "input_offsets");
  TensorList in, offs, outs;
  for (const auto& t : inputs) {
    TORCH_CHECK(t.scalar_type() == at::kChar || t.scalar_type() == at::kByte, "hash input must be int8 bytes");
    in.push_back(t.contiguous());
  }
  const int is64 = index_kind(input_offsets[0], "offsets");
  std::vector<int64_t> n_strings;
  for (const auto& o : input_offsets) {
    TORCH_CHECK(index_kind(o, "offsets") == is64, "offsets must share one integer dtype");
    offs.push_back(o.contiguous());
    n_strings.push_back(o.numel() - 1);
    outs.push_back(at::empty({o.numel() - 1}, o.options().dtype(at::kLong)));
  }
  c10::DeviceGuard guard(in[0].device());
  std::vector<int64_t> sizes = numels(in);
  auto ip = host_ptrs<int8_t>(in);
  auto fp = host_ptrs<void>(offs);
  auto op = host_mut_ptrs<int64_t>(outs);
  check(recis_fused_hash(ip.data(), sizes.data(), fp.data(), is64, n_strings.data(), op.data(),
                         static_cast<int64_t>(in.size()), hash_type == "farm" ? 0 : 1, stream_of(in[0].device())));
  return outs;
}

// ------------------------------------------------------------------------------------ padded gather
// batch_seq, the bookkeeping tensor the backward expects ([cumulative batch, cumulative batch * seq,
// seq] per feature after a leading zero triple), stays in host memory here: the backward reads it on
// the host, and a device copy would cost a wait for nothing.
TensorList ragged_tile(const std::vector<int64_t>& batch, const std::vector<int64_t>& seq, Tensor value,
                       Tensor offset, Tensor table) {
  TORCH_CHECK(batch.size() == seq.size(), "batch and seq differ in length");
  require_gpu(value, "value");
  require_gpu(offset, "offset");
  require_gpu(table, "table");
  TORCH_CHECK(table.dim() == 2, "table must be [rows, D]");
  c10::DeviceGuard guard(table.device());
  value = value.contiguous();
  offset = offset.contiguous();
  table = table.contiguous();
  const int64_t D = table.size(1), n = static_cast<int64_t>(batch.size());
  Tensor cum = at::zeros({3 * (n + 1)}, at::TensorOptions().dtype(at::kLong));
  int64_t* c = cum.data_ptr<int64_t>();
  int64_t rows = 0, ba = 0;
  for (int64_t f = 0; f < n; ++f) {
    ba += batch[f];
    rows += batch[f] * seq[f];
    c[3 * (f + 1)] = ba;
    c[3 * (f + 1) + 1] = rows;
    c[3 * (f + 1) + 2] = seq[f];
  }
  Tensor out = at::empty({rows, D}, table.options());
  check(recis_ragged_tile(batch.data(), seq.data(), n, value.data_ptr(), index_kind(value, "value"), value.numel(),
                          offset.data_ptr(), index_kind(offset, "offset"), table.data_ptr(), table.size(0),
                          dtype_code(table.scalar_type()), out.data_ptr(), D, stream_of(table.device())));
  return {out, cum};
}

Tensor ragged_tile_back(Tensor batch_seq, const std::vector<int64_t>& batch_info, Tensor value, Tensor offset,
                        Tensor dy) {
  TORCH_CHECK(batch_info.size() >= 2, "batch_info = [table_rows, n_features, batch_max, seq_min]");
  require_gpu(value, "value");
  require_gpu(offset, "offset");
  require_gpu(dy, "dy");
  TORCH_CHECK(dy.dim() == 2, "dy must be [rows, D]");
  c10::DeviceGuard guard(dy.device());
  value = value.contiguous();
  offset = offset.contiguous();
  dy = dy.contiguous();
  std::vector<int64_t> cum = host_values(batch_seq);
  const int64_t n = batch_info[1], table_rows = batch_info[0], D = dy.size(1);
  TORCH_CHECK(static_cast<int64_t>(cum.size()) >= 3 * (n + 1), "batch_seq is too short for ", n, " features");
  std::vector<int64_t> batch(n), seq(n);
  for (int64_t f = 0; f < n; ++f) {
    batch[f] = cum[3 * (f + 1)] - cum[3 * f];
    seq[f] = cum[3 * (f + 1) + 2];
  }
  Tensor out = at::empty({table_rows, D}, dy.options().dtype(at::kFloat));
  check(recis_ragged_tile_back(batch.data(), seq.data(), n, value.data_ptr(), index_kind(value, "value"),
                               value.numel(), offset.data_ptr(), index_kind(offset, "offset"), dy.data_ptr(),
                               dtype_code(dy.scalar_type()), out.data_ptr<float>(), table_rows, D,
                               stream_of(dy.device())));
  return dy.scalar_type() == at::kFloat ? out : out.to(dy.scalar_type());
}

// ------------------------------------------------------------------------------------ dense <-> ragged
namespace {
// The raw bytes of `value` converted to `dtype` (the fill value / the invalid value of a kernel).
std::vector<char> scalar_bytes(const at::Scalar& value, at::ScalarType dtype) {
  Tensor t = at::scalar_tensor(value, at::TensorOptions().dtype(dtype));
  std::vector<char> out(t.element_size());
  std::memcpy(out.data(), t.data_ptr(), out.size());
  return out;
}
}  // namespace

// The ragged tensor as a coalesced sparse COO tensor of shape [rows, longest row of level 0, ...,
// longest row of the last level]; coordinate k of a value is its position inside the row of level
// k - 1 that holds it (csrc/ops/ragged_to_sparse.cc:43-91; the reference has a CPU kernel only, this
// one is library calls on the device of its inputs, whichever that is).
Tensor ragged_to_sparse(Tensor values, TensorList offset_splits) {
  TORCH_CHECK(!offset_splits.empty(), "ragged_to_sparse: needs at least one level of offsets");
  for (const auto& o : offset_splits) {
    TORCH_CHECK(o.scalar_type() == offset_splits[0].scalar_type() &&
                    (o.scalar_type() == at::kInt || o.scalar_type() == at::kLong),
                "ragged_to_sparse: each offset_splits should be torch::kInt32 or torch::kInt64");
    TORCH_CHECK(o.device() == values.device(), "ragged_to_sparse: offset_splits and value should be all on cpu or cuda");
  }
  c10::DeviceGuard guard(values.device());
  TensorList splits;
  for (const auto& o : offset_splits) splits.push_back(o.to(at::kLong).contiguous());
  const Tensor& last = splits.back();
  const int64_t n = last.numel() ? last[last.numel() - 1].item<int64_t>() : 0;
  std::vector<int64_t> shape{splits[0].numel() - 1};
  for (const auto& o : splits) {
    shape.push_back(o.numel() > 1 ? (o.slice(0, 1) - o.slice(0, 0, o.numel() - 1)).max().item<int64_t>() : 0);
  }
  auto i64 = values.options().dtype(at::kLong);
  TensorList coords;
  Tensor child = at::arange(n, i64);  // index among the rows of the level below
  for (auto it = splits.rbegin(); it != splits.rend(); ++it) {
    Tensor parent = at::searchsorted(*it, child, /*out_int32=*/false, /*right=*/true) - 1;  // the row that holds `child`
    coords.push_back(child - it->index_select(0, parent));
    child = parent;
  }
  coords.push_back(child);
  std::reverse(coords.begin(), coords.end());
  Tensor indices = n ? at::stack(coords) : at::empty({static_cast<int64_t>(splits.size()) + 1, 0}, i64);
  for (int64_t d = 1; d < values.dim(); ++d) shape.push_back(values.size(d));
  return at::sparse_coo_tensor(indices, values.slice(0, 0, n), shape).coalesce();
}

Tensor ragged_to_dense(Tensor values, const TensorList& offsets, at::Scalar default_value) {
  require_gpu(values, "values");
  require_gpu(offsets, "offsets");
  TORCH_CHECK(values.dim() == 1, "values must dim == 1");
  TORCH_CHECK(!offsets.empty() && offsets.size() <= 5, "ragged_to_dense: 1 to 5 ragged levels");
  c10::DeviceGuard guard(values.device());
  values = values.contiguous();
  TensorList offs;
  const int is64 = index_kind(offsets[0], "offsets");
  std::vector<int64_t> shape{offsets[0].numel() - 1};
  for (const auto& o : offsets) {
    TORCH_CHECK(index_kind(o, "offsets") == is64, "ragged_to_dense: each offsets should be torch.int32 or torch.int64");
    offs.push_back(o.contiguous());
    // the longest row of the level, read back as the reference does (ragged_to_dense.cc:60-75)
    shape.push_back(o.numel() > 1 ? at::max(o.slice(0, 1) - o.slice(0, 0, o.numel() - 1)).item<int64_t>() : 0);
  }
  Tensor out = at::empty(shape, values.options());
  std::vector<char> fill = scalar_bytes(default_value, values.scalar_type());
  auto op = host_ptrs<void>(offs);
  std::vector<int64_t> sizes = numels(offs);
  check(recis_ragged_to_dense(values.data_ptr(), static_cast<int>(values.element_size()), values.numel(), op.data(),
                              sizes.data(), is64, shape.data() + 1, static_cast<int>(offs.size()), fill.data(),
                              out.data_ptr(), stream_of(values.device())));
  return out;
}

std::tuple<Tensor, Tensor> dense_to_ragged(const Tensor& data, bool check_invalid, const Tensor& invalid_value) {
  TORCH_CHECK(data.dim() == 2, "Input must be a 2D tensor");
  require_gpu(data, "data");
  c10::DeviceGuard guard(data.device());
  const int64_t rows = data.size(0), cols = data.size(1);
  if (!check_invalid) {
    Tensor offs = at::arange(0, rows * cols + 1, std::max<int64_t>(cols, 1), data.options().dtype(at::kInt));
    return std::make_tuple(data.reshape({-1}), offs.narrow(0, 0, rows + 1));
  }
  int kind;
  switch (data.scalar_type()) {
    case at::kFloat: kind = RECIS_SEQ_F32; break;
    case at::kDouble: kind = RECIS_SEQ_F64; break;
    case at::kInt: kind = RECIS_SEQ_I32; break;
    case at::kLong: kind = RECIS_SEQ_I64; break;
    default: TORCH_CHECK(false, "dense_to_ragged: float32, float64, int32 or int64 data, got ", data.scalar_type());
  }
  Tensor d = data.contiguous();
  TORCH_CHECK(invalid_value.numel() >= 1, "invalid_value must hold one element");
  std::vector<char> invalid = scalar_bytes(invalid_value.reshape({-1})[0].item(), d.scalar_type());
  Tensor offsets = at::empty({rows + 1}, d.options().dtype(at::kInt));
  Tensor src = at::empty({std::max<int64_t>(rows, 1)}, d.options().dtype(at::kLong));
  Tensor total = at::empty({1}, d.options().dtype(at::kLong));
  void* stream = stream_of(d.device());
  check(recis_dense_to_ragged_rows(d.data_ptr(), kind, rows, cols, invalid.data(), offsets.data_ptr<int32_t>(),
                                   src.data_ptr<int64_t>(), total.data_ptr<int64_t>(), stream));
  const int64_t n = total.item<int64_t>();
  Tensor values = at::empty({n}, d.options());
  if (n) {
    const void* vp = d.data_ptr();
    const void* fp = offsets.data_ptr();
    const int64_t* sp = src.data_ptr<int64_t>();
    void* outp = values.data_ptr();
    check(recis_ragged_cutoff_copy(&vp, static_cast<int>(d.element_size()), &fp, 0, &rows, &sp, &n, &outp, 1,
                                   stream));
  }
  return std::make_tuple(values, offsets);
}

// ------------------------------------------------------------------------------------ sequence truncation
namespace {

struct CutoffResult {
  TensorList values, offsets, drop_nums, pad_nums, outer;
};

CutoffResult ragged_cutoff(const TensorList& values_in, const TensorList& outer_in, const TensorList* inner_in,
                           const Tensor& keep_lengths, const Tensor& drop_sides, const Tensor& pad_sides) {
  const int64_t n = static_cast<int64_t>(values_in.size());
  TORCH_CHECK(static_cast<int64_t>(outer_in.size()) == n &&
                  (inner_in == nullptr || static_cast<int64_t>(inner_in->size()) == n),
              "offsets.numel() = ", outer_in.size(), " but is expected equals fea_num = ", n);
  require_gpu(values_in, "values");
  require_gpu(outer_in, "offsets");
  TensorList values, outer, inner;
  for (const auto& v : values_in) {
    TORCH_CHECK(v.scalar_type() == values_in[0].scalar_type(), "fused_ragged_cutoff: each value should be the same type");
    values.push_back(v.contiguous().reshape({-1}));
  }
  const int is64 = index_kind(outer_in[0], "offsets");
  for (const auto& o : outer_in) {
    TORCH_CHECK(index_kind(o, "offsets") == is64, "fused_ragged_cutoff: each offsets should be torch.int32 or torch.int64");
    outer.push_back(o.contiguous());
  }
  if (inner_in != nullptr) {
    require_gpu(*inner_in, "inner_offsets");
    for (const auto& o : *inner_in) {
      TORCH_CHECK(index_kind(o, "offsets") == is64, "fused_ragged_cutoff: each offsets should be torch.int32 or torch.int64");
      inner.push_back(o.contiguous());
    }
  }
  const bool three_d = inner_in != nullptr;
  std::vector<int64_t> keep = host_values(keep_lengths);
  std::vector<int64_t> drop = host_values(drop_sides.to(at::kLong)), pad = host_values(pad_sides.to(at::kLong));
  TORCH_CHECK(static_cast<int64_t>(keep.size()) == n, "keep_lengths.numel() = ", keep.size(),
              " but is expected equals fea_num = ", n);
  TORCH_CHECK(static_cast<int64_t>(drop.size()) == n, "drop_sides.numel() = ", drop.size(),
              " but is expected equals fea_num = ", n);
  TORCH_CHECK(static_cast<int64_t>(pad.size()) == n, "pad_sides.numel() = ", pad.size(),
              " but is expected equals fea_num = ", n);
  c10::DeviceGuard guard(values[0].device());
  auto iopt = outer[0].options();
  auto lopt = outer[0].options().dtype(at::kLong);
  std::vector<int64_t> rows(n), out_rows(n), n_inner(n), n_values = numels(values);
  int64_t sum_rows = 0, sum_out = 0;
  for (int64_t t = 0; t < n; ++t) {
    rows[t] = outer[t].numel() - 1;
    out_rows[t] = three_d ? rows[t] * keep[t] : rows[t];
    n_inner[t] = three_d ? inner[t].numel() - 1 : 0;
    sum_rows += rows[t];
    sum_out += out_rows[t];
  }
  // one allocation per kind of output, one view per tensor
  Tensor off_buf = at::empty({sum_out + n}, iopt);
  Tensor src_buf = at::empty({std::max<int64_t>(sum_out, 1)}, lopt);
  Tensor cnt_buf = at::empty({2 * sum_rows}, iopt);
  Tensor totals = at::empty({n}, lopt);
  Tensor outer_buf = three_d ? at::empty({sum_rows + n}, iopt) : Tensor();
  CutoffResult res;
  TensorList src;
  int64_t a = 0, b = 0;
  for (int64_t t = 0; t < n; ++t) {
    res.offsets.push_back(off_buf.narrow(0, a + t, out_rows[t] + 1));
    src.push_back(src_buf.narrow(0, out_rows[t] ? a : 0, out_rows[t]));
    res.drop_nums.push_back(cnt_buf.narrow(0, b, rows[t]));
    res.pad_nums.push_back(cnt_buf.narrow(0, sum_rows + b, rows[t]));
    if (three_d) res.outer.push_back(outer_buf.narrow(0, b + t, rows[t] + 1));
    a += out_rows[t];
    b += rows[t];
  }
  // an empty view has no address: any valid one will do, it is never dereferenced
  auto ptrs_or_dummy = [&](const TensorList& ts) {
    std::vector<void*> out(ts.size());
    for (size_t k = 0; k < ts.size(); ++k) out[k] = ts[k].numel() ? ts[k].data_ptr() : src_buf.data_ptr();
    return out;
  };
  std::vector<uint8_t> drop8(n), pad8(n);
  for (int64_t t = 0; t < n; ++t) {
    drop8[t] = drop[t] ? 1 : 0;
    pad8[t] = pad[t] ? 1 : 0;
  }
  void* stream = stream_of(values[0].device());
  auto outer_p = host_ptrs<void>(outer);
  auto inner_p = host_ptrs<void>(inner);
  auto out_off_p = host_mut_ptrs<void>(res.offsets);
  auto out_outer_p = host_mut_ptrs<void>(res.outer);
  auto drop_p = ptrs_or_dummy(res.drop_nums);
  auto pad_p = ptrs_or_dummy(res.pad_nums);
  auto src_p = ptrs_or_dummy(src);
  check(recis_ragged_cutoff_rows(outer_p.data(), three_d ? inner_p.data() : nullptr, is64, rows.data(),
                                 three_d ? n_inner.data() : nullptr, n_values.data(), keep.data(), drop8.data(),
                                 pad8.data(), n, out_off_p.data(), three_d ? out_outer_p.data() : nullptr,
                                 drop_p.data(), pad_p.data(), reinterpret_cast<int64_t* const*>(src_p.data()),
                                 totals.data_ptr<int64_t>(), stream));
  std::vector<int64_t> total_host = host_values(totals);  // the one wait of this op: the outputs are sized by it
  int64_t sum_total = 0;
  for (int64_t v : total_host) sum_total += v;
  Tensor val_buf = at::empty({sum_total}, values[0].options());
  a = 0;
  for (int64_t t = 0; t < n; ++t) {
    res.values.push_back(val_buf.narrow(0, a, total_host[t]));
    a += total_host[t];
  }
  auto val_p = ptrs_or_dummy(values);
  auto out_val_p = ptrs_or_dummy(res.values);
  check(recis_ragged_cutoff_copy(reinterpret_cast<const void* const*>(val_p.data()),
                                 static_cast<int>(values[0].element_size()),
                                 reinterpret_cast<const void* const*>(out_off_p.data()), is64, out_rows.data(),
                                 reinterpret_cast<const int64_t* const*>(src_p.data()), total_host.data(),
                                 out_val_p.data(), n, stream));
  return res;
}

}  // namespace

std::tuple<TensorList, TensorList, TensorList, TensorList, Tensor, Tensor> fused_ragged_cutoff(
    TensorList value, TensorList offset, Tensor keep_length, Tensor drop_sides, Tensor pad_sides) {
  if (value.empty()) return std::make_tuple(TensorList(), TensorList(), TensorList(), TensorList(), drop_sides, pad_sides);
  CutoffResult r = ragged_cutoff(value, offset, nullptr, keep_length, drop_sides, pad_sides);
  return std::make_tuple(r.values, r.offsets, r.drop_nums, r.pad_nums, drop_sides, pad_sides);
}

std::tuple<TensorList, TensorList, TensorList> fused_ragged_cutoff_3D(TensorList values, TensorList outer_offsets,
                                                                      TensorList inner_offsets,
                                                                      Tensor keep_lengths, Tensor drop_sides,
                                                                      Tensor pad_sides) {
  if (values.empty()) return std::make_tuple(TensorList(), TensorList(), TensorList());
  CutoffResult r = ragged_cutoff(values, outer_offsets, &inner_offsets, keep_lengths, drop_sides, pad_sides);
  return std::make_tuple(r.values, r.outer, r.offsets);
}

// ------------------------------------------------------------------------------------ feature cross
std::tuple<Tensor, Tensor, Tensor> feature_cross_ragged(const Tensor& x_value, const Tensor& x_offsets,
                                                        const Tensor& x_weight, const Tensor& y_value,
                                                        const Tensor& y_offsets, const Tensor& y_weight) {
  require_gpu(x_value, "x_value");
  require_gpu(x_offsets, "x_offsets");
  require_gpu(y_value, "y_value");
  require_gpu(y_offsets, "y_offsets");
  TORCH_CHECK(x_value.scalar_type() == at::kLong && y_value.scalar_type() == at::kLong,
              "feature_cross_ragged: ids for x and y must be torch.int64");
  const int is64 = index_kind(x_offsets, "x_offsets");
  TORCH_CHECK(index_kind(y_offsets, "y_offsets") == is64,
              "feature_cross_ragged: each offset should be torch.int32 or torch.int64");
  c10::DeviceGuard guard(x_value.device());
  Tensor xv = x_value.contiguous(), yv = y_value.contiguous(), xo = x_offsets.contiguous(), yo = y_offsets.contiguous();
  // an empty (or undefined) weight tensor means all ones
  Tensor xw = x_weight.defined() && x_weight.numel() ? x_weight.contiguous() : Tensor();
  Tensor yw = y_weight.defined() && y_weight.numel() ? y_weight.contiguous() : Tensor();
  at::ScalarType wdt = xw.defined() ? xw.scalar_type() : yw.defined() ? yw.scalar_type() : at::kFloat;
  TORCH_CHECK((wdt == at::kFloat || wdt == at::kDouble) && (!xw.defined() || xw.scalar_type() == wdt) &&
                  (!yw.defined() || yw.scalar_type() == wdt),
              "feature_cross_ragged: weights must share float32 or float64");
  if (xw.defined()) require_gpu(xw, "x_weight");
  if (yw.defined()) require_gpu(yw, "y_weight");
  const int64_t n_seg = std::min(xo.numel(), yo.numel()) - 1, nx = xv.numel(), ny = yv.numel();
  auto iopt = xv.options().dtype(at::kInt);
  Tensor x_rank = at::empty({std::max<int64_t>(nx, 1)}, iopt), y_rank = at::empty({std::max<int64_t>(ny, 1)}, iopt);
  Tensor y_count = at::empty({std::max<int64_t>(n_seg, 1)}, iopt);
  Tensor out_off = at::empty({n_seg + 1}, xo.options());
  Tensor total = at::empty({1}, xv.options());
  void* stream = stream_of(xv.device());
  check(recis_feature_cross_rows(xv.data_ptr<int64_t>(), xo.data_ptr(), nx, yv.data_ptr<int64_t>(), yo.data_ptr(), ny,
                                 is64, n_seg, x_rank.data_ptr<int32_t>(), y_rank.data_ptr<int32_t>(),
                                 y_count.data_ptr<int32_t>(), out_off.data_ptr(), total.data_ptr<int64_t>(), stream));
  const int64_t n = total.item<int64_t>();
  Tensor out_val = at::empty({n}, xv.options());
  Tensor out_w = at::empty({n}, xv.options().dtype(wdt));
  check(recis_feature_cross_emit(xv.data_ptr<int64_t>(), xo.data_ptr(), xw.defined() ? xw.data_ptr() : nullptr, nx,
                                 yv.data_ptr<int64_t>(), yo.data_ptr(), yw.defined() ? yw.data_ptr() : nullptr, ny,
                                 is64, wdt == at::kDouble ? 1 : 0, n_seg, x_rank.data_ptr<int32_t>(),
                                 y_rank.data_ptr<int32_t>(), y_count.data_ptr<int32_t>(), out_off.data_ptr(), n,
                                 out_val.data_ptr<int64_t>(), out_w.data_ptr(), stream));
  return std::make_tuple(out_val, out_off, out_w);
}

std::tuple<Tensor, Tensor> calc_ragged_index(Tensor drop_num, Tensor pad_num, Tensor drop_side, Tensor pad_side,
                                             Tensor offset, Tensor topk_index, Tensor indicator) {
  (void)pad_num;
  require_gpu(drop_num, "drop_num");
  require_gpu(offset, "offset");
  require_gpu(topk_index, "topk_index");
  require_gpu(indicator, "indicator");
  TORCH_CHECK(drop_side.scalar_type() == at::kBool && pad_side.scalar_type() == at::kBool,
              "drop_side and pad_side must be bool");
  const bool drop_left = drop_side.reshape({-1})[0].item<bool>(), pad_left = pad_side.reshape({-1})[0].item<bool>();
  TORCH_CHECK(drop_left && !pad_left, "drop ", drop_left ? "left" : "right", ", pad ", pad_left ? "left" : "right",
              " is not supported yet");
  TORCH_CHECK(topk_index.dim() == 2, "calc_ragged_index: topk_index must be [rows, cols]");
  const int64_t rows = topk_index.size(0), cols = topk_index.size(1), src_rows = offset.numel() - 1;
  TORCH_CHECK(indicator.numel() == rows, "indicator==row_num;indicator.numel(): ", indicator.numel(),
              "; row_num: ", rows);
  TORCH_CHECK(drop_num.numel() >= src_rows, "calc_ragged_index: drop_num is shorter than the rows of offset");
  c10::DeviceGuard guard(topk_index.device());
  Tensor d = drop_num.contiguous(), o = offset.contiguous(), t = topk_index.contiguous(), ind = indicator.contiguous();
  Tensor out_index = at::empty({std::max<int64_t>(rows * cols, 1)}, t.options());
  Tensor out_off = at::empty({rows + 1}, o.options());
  Tensor total = at::empty({1}, t.options().dtype(at::kLong));
  check(recis_ragged_topk_index(d.data_ptr(), index_kind(d, "drop_num"), o.data_ptr(), index_kind(o, "offset"),
                                src_rows, t.data_ptr(), index_kind(t, "topk_index"), ind.data_ptr(),
                                index_kind(ind, "indicator"), rows, cols, out_index.data_ptr(), out_off.data_ptr(),
                                total.data_ptr<int64_t>(), stream_of(t.device())));
  return std::make_tuple(out_index.narrow(0, 0, total.item<int64_t>()), out_off);
}

}  // namespace functional
}  // namespace recis
