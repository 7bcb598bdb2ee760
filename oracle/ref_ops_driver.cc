// Test infrastructure: runs the reference's OWN CPU implementations of the hot-path operators
// (compiled from /root/reference/csrc where they lie, see ref_build.sh) on inputs read from a
// file and writes their outputs to a file, so that the oracle (oracle/recis_oracle.c) can be
// checked against the real code. Nothing here is reference code: this file only moves tensors
// in and out and calls
//   recis::functional::block_apply_adamw            (csrc/ops/block_apply_adamw_op.cc:114-130)
//   recis::embedding::MakeCpuIdMap / CpuIdMap        (csrc/embedding/cpu_id_map.cc:73-190)
//   recis::embedding::IdAllocator                    (csrc/embedding/id_allocator.cc:17-60)
//   Hashtable (EmbeddingLookup, AcceptGrad, Delete, ids_map, slots) with SparseAdam / SparseAdamW /
//   SparseAdamWTF::step                              (csrc/embedding/hashtable.cc:46-278, adam*.cc)
//   recis::serialize::WriteBlock::MakeHTWriteBlock / MakeTensorWriteBlock + TableWriter (one data
//   file) and LoadBundle (directory index + file headers)  (csrc/serialize/write_block.cc:27-77,
//   table_writer.cc:48-88, load_bundle.cc:17-112). Saver/Loader themselves (save_bundle.cc,
//   load_internal.cc, read_block.cc) include CUDA headers and are not part of this build.
//   recis::functional::mask_key_index_op, scatter_ids_with_mask_op (csrc/ops/hashtable_ops.cc:150-214)
//   recis::functional::block_gather / block_insert / block_insert_with_mask / block_filter / gather
//                                                    (csrc/ops/block_ops.cc:270-397)
//   recis::functional::ids_partition_cpu, ids_encode_cpu, fused_uint64_mod, fused_bucketized,
//   fused_multi_hash, dense_to_ragged                (csrc/ops/*.cc)
// (segment_sum / segment_mean have no CPU implementation in the reference: segment_ops.cc only
// forwards to the CUDA functions.)
// The reference objects also refer to their CUDA counterparts (*_cuda, *_gpu); those symbols are
// left unresolved at link time (lazy binding) and are never reached: every tensor here is on the CPU.
//
// File format (little endian): int64 count, then per tensor: int32 dtype code, int32 ndim,
// int64 dims[ndim], raw bytes. dtype codes: 0 f32, 1 f64, 2 i64, 3 i32, 4 bool, 5 i8, 6 f16.
#include <torch/extension.h>

#include <chrono>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "embedding/adam.h"
#include "embedding/adamw.h"
#include "embedding/adamw_tf.h"
#include "embedding/hashtable.h"
#include "embedding/id_allocator.h"
#include "embedding/initializer.h"
#include "embedding/id_map.h"
#include "ops/block_apply_adamw_op.h"
#include "serialize/load_bundle.h"
#include "serialize/name.h"
#include "serialize/table_writer.h"
#include "serialize/write_block.h"
#include "ops/block_ops.h"
#include "ops/dense_to_ragged.h"
#include "ops/fused_bucketized.h"
#include "ops/fused_uint64_mod.h"
#include "ops/hashtable_ops.h"
#include "ops/ids_encode.h"
#include "ops/ids_partition.h"
#include "ops/multi_hash.h"

using torch::Tensor;

static at::ScalarType code_to_type(int c) {
  switch (c) {
    case 0: return at::kFloat;
    case 1: return at::kDouble;
    case 2: return at::kLong;
    case 3: return at::kInt;
    case 4: return at::kBool;
    case 5: return at::kChar;
    case 6: return at::kHalf;
  }
  TORCH_CHECK(false, "bad dtype code ", c);
}
static int type_to_code(at::ScalarType t) {
  switch (t) {
    case at::kFloat: return 0;
    case at::kDouble: return 1;
    case at::kLong: return 2;
    case at::kInt: return 3;
    case at::kBool: return 4;
    case at::kChar: return 5;
    case at::kHalf: return 6;
    default: TORCH_CHECK(false, "unsupported output dtype");
  }
}

static std::vector<Tensor> read_tensors(const char* path) {
  FILE* f = fopen(path, "rb");
  TORCH_CHECK(f, "cannot open ", path);
  int64_t n = 0;
  TORCH_CHECK(fread(&n, 8, 1, f) == 1, "short file");
  std::vector<Tensor> out;
  for (int64_t i = 0; i < n; ++i) {
    int32_t code = 0, ndim = 0;
    TORCH_CHECK(fread(&code, 4, 1, f) == 1 && fread(&ndim, 4, 1, f) == 1, "short file");
    std::vector<int64_t> dims(ndim);
    if (ndim) TORCH_CHECK(fread(dims.data(), 8, ndim, f) == static_cast<size_t>(ndim), "short file");
    Tensor t = torch::empty(dims, torch::TensorOptions().dtype(code_to_type(code)));
    const size_t bytes = t.numel() * t.element_size();
    if (bytes) TORCH_CHECK(fread(t.data_ptr(), 1, bytes, f) == bytes, "short file");
    out.push_back(t);
  }
  fclose(f);
  return out;
}

static void write_tensors(const char* path, const std::vector<Tensor>& ts) {
  FILE* f = fopen(path, "wb");
  TORCH_CHECK(f, "cannot open ", path);
  int64_t n = ts.size();
  fwrite(&n, 8, 1, f);
  for (const Tensor& t0 : ts) {
    Tensor t = t0.contiguous();
    int32_t code = type_to_code(t.scalar_type()), ndim = t.dim();
    fwrite(&code, 4, 1, f);
    fwrite(&ndim, 4, 1, f);
    for (int d = 0; d < ndim; ++d) {
      int64_t v = t.size(d);
      fwrite(&v, 8, 1, f);
    }
    const size_t bytes = t.numel() * t.element_size();
    if (bytes) fwrite(t.data_ptr(), 1, bytes, f);
  }
  fclose(f);
}

// a [rows, ...] tensor as the list of [block_size, ...] blocks the reference ops take (views)
static std::vector<Tensor> as_blocks(const Tensor& t, int64_t block_size) {
  std::vector<Tensor> b;
  for (int64_t r = 0; r + block_size <= t.size(0); r += block_size) b.push_back(t.narrow(0, r, block_size));
  return b;
}

static std::vector<Tensor> run(const std::string& op, std::vector<Tensor> in) {
  namespace F = recis::functional;
  if (op == "adamw") {
    // index [T, n] i64, grad [T, n, D], emb / exp_avg / exp_avg_sq [R, D], beta1_t, beta2_t [1],
    // scalars f64 [6] = lr, beta1, beta2, weight_decay, eps, block_size
    Tensor index = in[0], grad = in[1], emb = in[2], m = in[3], v = in[4], b1t = in[5], b2t = in[6];
    const double* s = in[7].data_ptr<double>();
    const int64_t bs = static_cast<int64_t>(s[5]);
    Tensor step = torch::zeros({1}, torch::kLong);
    for (int64_t t = 0; t < index.size(0); ++t)
      F::block_apply_adamw(index[t], grad[t], as_blocks(emb, bs), b1t, b2t, step, as_blocks(m, bs), as_blocks(v, bs),
                           s[0], s[1], s[2], s[3], s[4], bs);
    return {emb, m, v, b1t, b2t};
  }
  if (op == "idmap") {
    // codes i64 [K] (0 lookup, 1 lookup read-only, 2 delete), lens i64 [K], ids i64 [sum lens]
    auto map = recis::embedding::MakeCpuIdMap(torch::Device(torch::kCPU));
    const int64_t* codes = in[0].data_ptr<int64_t>();
    const int64_t* lens = in[1].data_ptr<int64_t>();
    std::vector<Tensor> res;
    int64_t at = 0;
    for (int64_t k = 0; k < in[0].numel(); ++k) {
      Tensor ids = in[2].narrow(0, at, lens[k]).clone();
      at += lens[k];
      if (codes[k] == 0) {
        res.push_back(map->Lookup(ids));
      } else if (codes[k] == 1) {
        res.push_back(map->LookupReadOnly(ids));
      } else {
        Tensor idx = map->LookupReadOnly(ids);
        map->DeleteIds(ids, idx);
        res.push_back(idx);
      }
    }
    auto snap = map->SnapShot();
    Tensor out = res.empty() ? torch::empty({0}, torch::kLong) : torch::cat(res);
    return {out, snap.first, snap.second, torch::tensor({map->GetIdNum()}, torch::kLong)};
  }
  if (op == "alloc") {
    // codes i64 [K] (0 gen, 1 free), lens i64 [K], ids to free i64 [sum of free lens], params i64 [2] = init, block
    const int64_t* codes = in[0].data_ptr<int64_t>();
    const int64_t* lens = in[1].data_ptr<int64_t>();
    const int64_t* prm = in[3].data_ptr<int64_t>();
    auto alloc = c10::make_intrusive<recis::embedding::IdAllocator>(torch::Device(torch::kCPU), prm[0],
                                                                    static_cast<size_t>(prm[1]));
    std::vector<Tensor> res;
    int64_t at = 0;
    for (int64_t k = 0; k < in[0].numel(); ++k) {
      if (codes[k] == 0) {
        res.push_back(alloc->GenIds(static_cast<size_t>(lens[k])));
      } else {
        alloc->FreeIds(in[2].narrow(0, at, lens[k]).clone());
        at += lens[k];
      }
    }
    Tensor out = res.empty() ? torch::empty({0}, torch::kLong) : torch::cat(res);
    return {out, torch::tensor({alloc->GetSize(), alloc->GetActiveSize()}, torch::kLong)};
  }
  if (op == "table_train") {
    // A script on one CPU Hashtable (constant initialiser) with one sparse optimizer.
    // params f64 [10] = block_size, D, optimizer (0 SparseAdam, 1 SparseAdamW, 2 SparseAdamWTF), lr,
    //                   beta1, beta2, eps, weight_decay, initial row value, grad accumulation steps
    // codes i64 [K]: 0 lookup + accept_grad, 1 optimizer step + zero_grad, 2 delete (ids must be
    //                present), 3 read-only lookup;  lens i64 [K];  ids i64 [sum of lens of codes 0/2/3];
    // grads f32 [sum of lens of code 0, D]
    const double* p = in[0].data_ptr<double>();
    const int64_t bs = static_cast<int64_t>(p[0]), D = static_cast<int64_t>(p[1]);
    const int kind = static_cast<int>(p[2]);
    auto gen = recis::embedding::MakeConstantGenerator({bs, D}, torch::kFloat, p[8]);
    auto table = Hashtable::Make(bs, {D}, torch::kFloat, torch::Device(torch::kCPU), true, {"t"}, gen, 0, 65536, 65536);
    // the optimizers are built from a plain map: the Dict overload (their static Make) needs the
    // custom-class registration of csrc/bind.cc, which is not part of this build
    std::unordered_map<std::string, HashTablePtr> tables{{"t", table}};
    c10::intrusive_ptr<recis::optim::SparseOptimizer> opt;
    std::string prefix;
    if (kind == 0) {
      recis::optim::SparseAdamOptions o;
      o.lr(p[3]).betas(std::make_tuple(p[4], p[5])).eps(p[6]).weight_decay(p[7]);
      opt = c10::make_intrusive<recis::optim::SparseAdam>(tables, o);
      prefix = "sparse_adam_";
    } else if (kind == 1) {
      recis::optim::SparseAdamWOptions o;
      o.lr(p[3]).betas(std::make_tuple(p[4], p[5])).eps(p[6]).weight_decay(p[7]);
      opt = c10::make_intrusive<recis::optim::SparseAdamW>(tables, o);
      prefix = "sparse_adamw_";
    } else {
      recis::optim::SparseAdamWTFOptions o;
      o.lr(p[3]).betas(std::make_tuple(p[4], p[5])).eps(p[6]).weight_decay(p[7]);
      opt = c10::make_intrusive<recis::optim::SparseAdamWTF>(tables, o);
      prefix = "sparse_adamw_tf_";
    }
    opt->set_grad_accum_steps(static_cast<int64_t>(p[9]));
    const int64_t* codes = in[1].data_ptr<int64_t>();
    const int64_t* lens = in[2].data_ptr<int64_t>();
    std::vector<Tensor> idx_out, emb_out;
    int64_t at_id = 0, at_grad = 0;
    for (int64_t k = 0; k < in[1].numel(); ++k) {
      if (codes[k] == 1) {
        opt->step();
        opt->zero_grad();
        continue;
      }
      Tensor ids = in[3].narrow(0, at_id, lens[k]).clone();
      at_id += lens[k];
      if (codes[k] == 0) {
        auto r = table->EmbeddingLookup(ids, false);
        idx_out.push_back(std::get<0>(r));
        emb_out.push_back(std::get<1>(r));
        table->AcceptGrad(std::get<0>(r), in[4].narrow(0, at_grad, lens[k]).clone());
        at_grad += lens[k];
      } else if (codes[k] == 3) {
        auto r = table->EmbeddingLookup(ids, true);
        idx_out.push_back(std::get<0>(r));
        emb_out.push_back(std::get<1>(r));
      } else {
        auto r = table->EmbeddingLookup(ids, true);
        table->Delete(ids, std::get<0>(r), "");
      }
    }
    auto snap = table->ids_map();
    return {idx_out.empty() ? torch::empty({0}, torch::kLong) : torch::cat(idx_out),
            emb_out.empty() ? torch::empty({0, D}) : torch::cat(emb_out),
            std::get<0>(snap), std::get<1>(snap),
            table->SlotGroup()->EmbSlot()->Value(),
            table->GetSlot(prefix + "exp_avg")->Value(),
            table->GetSlot(prefix + "exp_avg_sq")->Value()};
  }
  if (op == "table_step_time") {
    // Times one training step of the reference on one CPU Hashtable with SparseAdam:
    // ids_partition_cpu (dedup) + EmbeddingLookup + [pooling forward and backward] + AcceptGrad + step +
    // zero_grad. The reference has no CPU pooling OPERATOR (segment_ops.cc only forwards to CUDA); with
    // segment ids given (in[2]) the pooling runs as the reference's own "torch" backend does on CPU tensors
    // (recis/nn/functional/embedding_ops.py:59-66: data[indices] then index_add_ by segment id; backward
    // = the transpose, grad_out[segment_ids] index_add_-ed by unique row), on torch's CPU thread pool.
    // params f64 [9] = block_size, D, lr, beta1, beta2, eps, weight_decay, time budget in seconds,
    //                  threads;  ids i64 [n] = one step's ids (duplicates included);
    // optional segment_ids i64 [n] (sorted, last + 1 = number of segments).
    // Returns f64 [3] = seconds, steps timed, unique ids per step.
    const double* p = in[0].data_ptr<double>();
    const int64_t bs = static_cast<int64_t>(p[0]), D = static_cast<int64_t>(p[1]);
    at::set_num_threads(static_cast<int>(p[8]));
    auto gen = recis::embedding::MakeConstantGenerator({bs, D}, torch::kFloat, 0.01);
    auto table = Hashtable::Make(bs, {D}, torch::kFloat, torch::Device(torch::kCPU), true, {"t"}, gen, 0, 65536, 65536);
    std::unordered_map<std::string, HashTablePtr> tables{{"t", table}};
    recis::optim::SparseAdamOptions o;
    o.lr(p[2]).betas(std::make_tuple(p[3], p[4])).eps(p[5]).weight_decay(p[6]);
    auto opt = c10::make_intrusive<recis::optim::SparseAdam>(tables, o);
    const bool pool = in.size() > 2;
    Tensor seg, up;
    int64_t S = 0;
    if (pool) {
      seg = in[2];
      S = seg.numel() ? seg[seg.numel() - 1].item<int64_t>() + 1 : 0;
      up = torch::full({S, D}, 1e-3f);
    }
    int64_t uniq = 0, steps = 0;
    Tensor grad;
    auto one_step = [&]() {
      auto part = F::ids_partition_cpu(in[1], 1);
      Tensor u = std::get<0>(part);
      uniq = u.numel();
      auto r = table->EmbeddingLookup(u, false);
      if (pool) {
        Tensor inverse = std::get<2>(part).to(torch::kLong);
        Tensor pooled = torch::zeros({S, D}).index_add_(0, seg, std::get<1>(r).index_select(0, inverse));
        grad = torch::zeros({uniq, D}).index_add_(0, inverse, up.index_select(0, seg));
        (void)pooled;
      } else if (!grad.defined() || grad.size(0) != uniq) {
        grad = torch::full({uniq, D}, 1e-3f);
      }
      table->AcceptGrad(std::get<0>(r), grad);
      opt->step();
      opt->zero_grad();
    };
    one_step();  // admission of the ids: not timed
    const auto t0 = std::chrono::steady_clock::now();
    double dt = 0;
    do {
      one_step();
      ++steps;
      dt = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    } while (dt < p[7]);
    return {torch::tensor({dt, static_cast<double>(steps), static_cast<double>(uniq)}, torch::kDouble)};
  }
  if (op == "ckpt_write_file") {
    // Writes ONE data file with the reference's TableWriter from a CPU Hashtable and a dense tensor.
    // path i8 [len] = directory, params i64 [5] = block_size, coalesced (0/1), slice begin, end, size,
    // ids i64 [n] (already tagged when coalesced: two children "a" and "b"), rows f32 [n, D], dense f32 [...]
    std::string dir(reinterpret_cast<const char*>(in[0].data_ptr<int8_t>()), in[0].numel());
    const int64_t* p = in[1].data_ptr<int64_t>();
    const int64_t D = in[3].size(1);
    auto gen = recis::embedding::MakeConstantGenerator({p[0], D}, torch::kFloat, 0.0);
    std::vector<std::string> children = p[1] ? std::vector<std::string>{"a", "b"} : std::vector<std::string>{"a"};
    auto table = Hashtable::Make(p[0], {D}, torch::kFloat, torch::Device(torch::kCPU), p[1] != 0, children, gen,
                                 p[2], p[3], p[4]);
    table->AppendStepFilterSlot("step_filter", 7);
    table->Insert(in[2], in[3]);
    namespace S = recis::serialize;
    auto writer = S::TableWriter::Make(dir, "ref.safetensors", "ref.json");
    auto blocks = S::WriteBlock::MakeHTWriteBlock(table);
    blocks.push_back(S::WriteBlock::MakeTensorWriteBlock("dense_w", in[4]));
    for (auto& b : blocks) writer->AppendWriteBlock(b);
    writer->SequentialWrite();
    return {torch::tensor({static_cast<int64_t>(blocks.size())}, torch::kLong)};
  }
  if (op == "ckpt_inspect") {
    // Reads a checkpoint directory with the reference's LoadBundle. path i8 [len].
    // Returns names (i8, one per line: "<tensor>\t<c10::ScalarType number>\t<slice>"), then per line
    // shape row [4] (padded with -1) and the absolute byte range [2] of the block in its file.
    std::string dir(reinterpret_cast<const char*>(in[0].data_ptr<int8_t>()), in[0].numel());
    namespace S = recis::serialize;
    auto bundle = S::LoadBundle::Make(dir);
    auto names = bundle->ListTensor();
    std::sort(names.begin(), names.end());
    std::string text;
    std::vector<int64_t> shapes, ranges, total_shapes;
    for (const auto& name : names) {
      auto slices = bundle->SliceInfos(name);
      std::sort(slices.begin(), slices.end());
      auto total = bundle->TensorShape(name);
      for (const auto& sl : slices) {
        auto bn = S::BlockNameEncode(name, sl);
        auto info = bundle->GetBlockInfo(bn);
        text += name + "\t" + std::to_string(static_cast<int>(info->Dtype())) + "\t" + sl + "\n";
        auto shp = info->Shape();
        for (int d = 0; d < 4; ++d) shapes.push_back(d < static_cast<int>(shp.size()) ? shp[d] : -1);
        for (int d = 0; d < 4; ++d) total_shapes.push_back(d < static_cast<int>(total.size()) ? total[d] : -1);
        ranges.push_back(info->OffsetBeg());
        ranges.push_back(info->OffsetEnd());
      }
    }
    Tensor t = torch::empty({static_cast<int64_t>(text.size())}, torch::kChar);
    memcpy(t.data_ptr(), text.data(), text.size());
    const int64_t rows = static_cast<int64_t>(ranges.size() / 2);
    return {t, torch::tensor(shapes, torch::kLong).view({rows, 4}), torch::tensor(ranges, torch::kLong).view({rows, 2}),
            torch::tensor(total_shapes, torch::kLong).view({rows, 4})};
  }
  if (op == "dense_to_ragged") {  // data [rows, cols], invalid value [1] of the same dtype
    auto r = F::dense_to_ragged(in[0], true, in[1]);
    return {std::get<0>(r), std::get<1>(r)};
  }
  if (op == "mask_key_index") {  // keys, mask (bool), cumsum, out_size [1]
    auto r = F::mask_key_index_op(in[0], in[1], in[2], in[3].item<int64_t>());
    return {std::get<0>(r), std::get<1>(r)};
  }
  if (op == "scatter_ids_with_mask") return {F::scatter_ids_with_mask_op(in[0], in[1], in[2])};
  if (op == "block_gather") {  // ids, table [R, D], params i64 [3] = block_size, default_key, readonly
    const int64_t* p = in[2].data_ptr<int64_t>();
    return {F::block_gather(in[0], as_blocks(in[1], p[0]), p[0], p[1], p[2] != 0)};
  }
  if (op == "gather") return {F::gather(in[0], in[1])};
  if (op == "block_insert") {  // ids, rows, table, block_size [1]
    F::block_insert(in[0], in[1], as_blocks(in[2], in[3].item<int64_t>()), in[3].item<int64_t>());
    return {in[2]};
  }
  if (op == "block_insert_with_mask") {  // ids, rows, mask, table, block_size [1]
    F::block_insert_with_mask(in[0], in[1], in[2], as_blocks(in[3], in[4].item<int64_t>()), in[4].item<int64_t>());
    return {in[3]};
  }
  if (op == "block_filter") {  // ids, slot [R, 1], params i64 [2] = block_size, threshold
    const int64_t* p = in[2].data_ptr<int64_t>();
    return {F::block_filter(in[0], as_blocks(in[1], p[0]), p[0], p[1])};
  }
  if (op == "ids_partition") {  // ids, num_parts [1]
    auto r = F::ids_partition_cpu(in[0], in[1].item<int64_t>());
    return {std::get<0>(r), std::get<1>(r), std::get<2>(r)};
  }
  if (op == "ids_encode") {  // table_ids, tensors...
    std::vector<Tensor> l(in.begin() + 1, in.end());
    return {F::ids_encode_cpu(l, in[0])};
  }
  if (op == "fused_uint64_mod") {  // mods, tensors...
    std::vector<Tensor> l(in.begin() + 1, in.end());
    return F::fused_uint64_mod(l, in[0]);
  }
  if (op == "fused_bucketized") {  // k values then k boundaries
    const size_t k = in.size() / 2;
    std::vector<Tensor> v(in.begin(), in.begin() + k), b(in.begin() + k, in.end());
    return F::fused_bucketized(v, b);
  }
  if (op == "fused_multi_hash") {  // k inputs, k muls, k primes, k bucket counts
    const size_t k = in.size() / 4;
    std::vector<Tensor> a(in.begin(), in.begin() + k), m(in.begin() + k, in.begin() + 2 * k),
        p(in.begin() + 2 * k, in.begin() + 3 * k), b(in.begin() + 3 * k, in.end());
    return F::fused_multi_hash(a, m, p, b);
  }
  if (op == "generate") {
    // params f64 [10] = kind, rows, dim, seed, p0, p1, p2, p3, fan mode (0 in, 1 out), generate rows (0 = own shape).
    // kind: 0 constant(p0) 1 uniform(p0, p1) 2 normal(p0, p1) 3 xavier_uniform(gain p0) 4 xavier_normal(gain p0)
    // 5 kaiming_uniform(a p0) 6 kaiming_normal(a p0) 7 trunc_normal(mean p0, std p1, a p2, b p3); the
    // Kaiming generators with leaky_relu. Seeds torch's default generator, then calls the reference's
    // generator (csrc/embedding/initializer.cc:26-366) once.
    using namespace recis::embedding;
    const double* q = in[0].data_ptr<double>();
    const int kind = static_cast<int>(q[0]);
    const std::vector<int64_t> shape = {static_cast<int64_t>(q[1]), static_cast<int64_t>(q[2])};
    const std::string mode = q[8] != 0 ? "fan_out" : "fan_in";
    torch::intrusive_ptr<Generator> g;
    switch (kind) {
      case 0: g = MakeConstantGenerator(shape, at::kFloat, q[4]); break;
      case 1: g = MakeUniformGenerator(shape, at::kFloat, q[4], q[5], c10::nullopt); break;
      case 2: g = MakeNormalGenerator(shape, at::kFloat, q[4], q[5], c10::nullopt); break;
      case 3: g = MakeXavierUniFormGenerator(shape, at::kFloat, q[4], c10::nullopt); break;
      case 4: g = MakeXavierNormalGenerator(shape, at::kFloat, q[4], c10::nullopt); break;
      case 5: g = MakeKaimingUniformGenerator(shape, at::kFloat, q[4], mode, "leaky_relu", c10::nullopt); break;
      case 6: g = MakeKaimingNormalGenerator(shape, at::kFloat, q[4], mode, "leaky_relu", c10::nullopt); break;
      case 7: g = MakeTruncNormalGenerator(shape, at::kFloat, q[4], q[5], q[6], q[7], c10::nullopt); break;
      default: TORCH_CHECK(false, "bad generator kind ", kind);
    }
    torch::manual_seed(static_cast<uint64_t>(q[3]));
    if (q[9] != 0) return {g->Generate({static_cast<int64_t>(q[9]), shape[1]})};
    return {g->Generate()};
  }
  TORCH_CHECK(false, "unknown op ", op);
}

int main(int argc, char** argv) {
  if (argc != 4) {
    fprintf(stderr, "usage: %s <op> <in.bin> <out.bin>\n", argv[0]);
    return 2;
  }
  try {
    at::set_num_threads(1);  // the reference's id map assigns rows in thread order: one thread = input order
    write_tensors(argv[3], run(argv[1], read_tensors(argv[2])));
  } catch (const std::exception& e) {
    fprintf(stderr, "ref_ops %s: %s\n", argv[1], e.what());
    return 1;
  }
  return 0;
}
