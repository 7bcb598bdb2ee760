// The registration block the reference has at csrc/bind.cc:46-211: namespace `recis`, the same
// class and operator names, the reference's C++ signatures (torch infers the schemas from them).
// Loaded with torch.classes.load_library(<package>/lib/recis.so), as recis/__init__.py:8-16 does.
// Not registered: gauc_calc and adam_tf_apply (a metric and the dense optimizer: outside the
// sparse-embedding path this build covers).
#include <torch/custom_class.h>
#include <torch/library.h>

#include "ops.h"
#include "serialize.h"
#include "sparse_optim.h"
#include "table.h"

namespace {

template <typename Optim>
void def_optimizer(torch::Library& m, const char* name) {
  // the shared methods live in the base class: lambdas keep `self` typed as the registered class
  using Self = c10::intrusive_ptr<Optim>;
  using Tables = c10::Dict<std::string, HashTablePtr>;
  m.class_<Optim>(name)
      .def("step", [](const Self& self) { self->step(); })
      .def("add_parameters", [](const Self& self, const Tables& parameters) { self->add_parameters(parameters); })
      .def("zero_grad", [](const Self& self) { self->zero_grad(); })
      .def("state_dict", [](const Self& self) { return self->state_dict(); })
      .def("load_state_dict", [](const Self& self, Tables hashtables, c10::Dict<std::string, at::Tensor> steps) {
        self->load_state_dict(std::move(hashtables), std::move(steps));
      })
      .def("set_grad_accum_steps", [](const Self& self, int64_t steps) { self->set_grad_accum_steps(steps); })
      .def("set_lr", [](const Self& self, double lr) { self->set_lr(lr); })
      .def_static("make", &Optim::Make);
}

}  // namespace

TORCH_LIBRARY(recis, m) {
  using recis::embedding::ChildrenInfo;
  using recis::embedding::Generator;
  using recis::embedding::Slot;
  using recis::embedding::SlotGroup;

  m.class_<ChildrenInfo>("ChildrenInfo")
      .def("index_bits_num", &ChildrenInfo::IndexBitsNum)
      .def("id_bits_num", &ChildrenInfo::IdBitsNum)
      .def("index_mask", &ChildrenInfo::IndexMask)
      .def("id_mask", &ChildrenInfo::IdMask)
      .def("max_children_num", &ChildrenInfo::MaxChildrenNum)
      .def("encode_id", &ChildrenInfo::EncodeId)
      .def("children", &ChildrenInfo::Children)
      .def("child_index", &ChildrenInfo::ChildIndex)
      .def("has_child", &ChildrenInfo::HasChild)
      .def("child_at", &ChildrenInfo::ChildAt)
      .def("is_coalesce", &ChildrenInfo::IsCoalesce);

  // (classes are registered before the signatures that mention them)
  m.class_<Generator>("Generator")
      // additions: a tensor of another shape (Slot::GenVal, slot_group.cc:112-116; fan-dependent
      // initialisers take the fans from fan_shape when given), and the device the rows are drawn on
      .def(
          "gen",
          [](const c10::intrusive_ptr<Generator>& self, c10::optional<std::vector<int64_t>> shape,
             c10::optional<std::vector<int64_t>> fan_shape) {
            return self->Generate(shape.value_or(std::vector<int64_t>{}), fan_shape.value_or(std::vector<int64_t>{}));
          },
          "", {torch::arg("shape") = c10::nullopt, torch::arg("fan_shape") = c10::nullopt})
      .def("set_device", [](const c10::intrusive_ptr<Generator>& self, at::Device device) { self->set_device(device); })
      .def_static("generate", Generator::DoGenerator)
      .def_static("make_constant_generator", recis::embedding::MakeConstantGenerator)
      .def_static("make_uniform_generator", recis::embedding::MakeUniformGenerator)
      .def_static("make_normal_generator", recis::embedding::MakeNormalGenerator)
      .def_static("make_xavier_uniform_generator", recis::embedding::MakeXavierUniFormGenerator)
      .def_static("make_xavier_normal_generator", recis::embedding::MakeXavierNormalGenerator)
      .def_static("make_kaiming_uniform_generator", recis::embedding::MakeKaimingUniformGenerator)
      .def_static("make_kaiming_normal_generator", recis::embedding::MakeKaimingNormalGenerator)
      .def_static("make_trunc_normal_generator", recis::embedding::MakeTruncNormalGenerator)
      .def_static("make_tensor_generator", recis::embedding::MakeTensorGenerator);  // an addition

  using SlotSelf = c10::intrusive_ptr<Slot>;
  m.class_<Slot>("Slot")
      .def("block_size", &Slot::BlockSize)
      .def("name", &Slot::Name)
      .def("flat_size", &Slot::FlatSize)
      .def("value", &Slot::Value)
      .def("values", &Slot::ValuesDeref)
      // additions: what the reference reaches from C++ (csrc/serialize, the optimizers) and this
      // build's Python reaches through the binding
      .def("dtype", &Slot::Dtype)
      .def("row_shape", &Slot::RowShape)
      .def(
          "index_select",
          [](const SlotSelf& self, const at::Tensor& index, int64_t beg, int64_t end) {
            return self->IndexSelect(index, beg, end < 0 ? index.numel() : end);
          },
          "", {torch::arg("index"), torch::arg("beg") = 0, torch::arg("end") = -1})
      .def(
          "index_insert",
          [](const SlotSelf& self, const at::Tensor& index, at::Tensor value, c10::optional<at::Tensor> accept) {
            if (accept.has_value() && accept->defined()) {
              self->IndexInsert(index, std::move(value), *accept);
            } else {
              self->IndexInsert(index, std::move(value));
            }
          },
          "", {torch::arg("index"), torch::arg("value"), torch::arg("accept_indicator") = c10::nullopt})
      .def("gen_val", &Slot::GenVal)
      .def("kernel_blocks", [](const SlotSelf& self) { return std::make_tuple(self->Chunks(), self->ChunkRows()); });

  using GroupSelf = c10::intrusive_ptr<SlotGroup>;
  m.class_<SlotGroup>("SlotGroup")
      .def("slot_by_name", &SlotGroup::GetSlotByName)
      .def("slot_by_index", &SlotGroup::GetSlotByIndex)
      .def("slot_index", &SlotGroup::GetSlotByIndex)  // sic: the reference binds this name to GetSlotByIndex too
      .def("slots", &SlotGroup::Slots)
      // additions
      .def("emb_slot", &SlotGroup::EmbSlot)
      .def("get_slot_index", &SlotGroup::GetSlotIndex)
      .def("has_slot", &SlotGroup::HasSlot)
      .def("block_size", &SlotGroup::BlockSize)
      .def("block_num", &SlotGroup::BlockNum)
      .def("capacity_rows", &SlotGroup::CapacityRows)
      .def("chunk_rows", &SlotGroup::ChunkRows)
      .def("append_slot",
           [](const GroupSelf& self, const std::string& name, at::ScalarType dtype, std::vector<int64_t> partial_shape,
              c10::optional<c10::intrusive_ptr<Generator>> generator, double init_val) {
             if (generator.has_value() && generator->defined()) {
               return self->AppendSlot(name, dtype, partial_shape, *generator);
             }
             return self->AppendSlot(name, dtype, partial_shape, init_val);
           });

  using recis::BatchPlan;
  using PlanSelf = c10::intrusive_ptr<BatchPlan>;
  m.class_<BatchPlan>("BatchPlan")  // an addition: see plan.h
      .def_property("n", [](const PlanSelf& self) { return self->n(); })
      .def_property("serial", [](const PlanSelf& self) { return self->serial(); })
      .def_property("hot_cap", [](const PlanSelf& self) { return self->hot_cap(); })
      .def_property("U", [](const PlanSelf& self) { return self->U(); })
      .def_property("unique", [](const PlanSelf& self) { return self->unique(); })
      .def_property("unique_buf", [](const PlanSelf& self) { return self->unique_buf(); })
      .def_property("inverse", [](const PlanSelf& self) { return self->inverse(); })
      .def_property("pos", [](const PlanSelf& self) { return self->pos(); })
      .def_property("row_start", [](const PlanSelf& self) { return self->row_start(); })
      .def_property("occ", [](const PlanSelf& self) { return self->occ(); })
      .def_property("hot_items", [](const PlanSelf& self) { return self->hot_items(); })
      .def_property("counts", [](const PlanSelf& self) { return self->counts(); })
      .def_property("index_buf", [](const PlanSelf& self) { return self->index_buf(); })
      .def("U_bound", [](const PlanSelf& self) { return self->U_bound(); })
      .def("src_coef_for_pool", &BatchPlan::SrcCoefForPool, "",
           {torch::arg("offsets"), torch::arg("weight"), torch::arg("mean")})
      .def("src_for_tile", &BatchPlan::SrcForTile, "", {torch::arg("batch"), torch::arg("seq"), torch::arg("offsets")})
      .def("src_for_pool_and_tile", &BatchPlan::SrcForPoolAndTile, "",
           {torch::arg("offsets"), torch::arg("weight"), torch::arg("mean"), torch::arg("batch"), torch::arg("seq")});

  m.class_<Hashtable>("HashtableImpl")
      .def("accept_grad", &Hashtable::AcceptGrad)
      .def("grad", &Hashtable::grad)
      .def("clear_grad", &Hashtable::ClearGrad)
      .def("embedding_lookup", &Hashtable::EmbeddingLookup)
      .def("insert", &Hashtable::Insert)
      .def("clear", &Hashtable::Clear)
      .def("clear_id", &Hashtable::ClearId)
      .def("ids", &Hashtable::ids)
      .def("slot_group", &Hashtable::SlotGroup)
      .def("children_info", &Hashtable::ChildrenInfo)
      .def("append_filter_slot", &Hashtable::AppendFilterSlot)
      .def("append_step_filter_slot", &Hashtable::AppendStepFilterSlot)
      .def("update_slot", &Hashtable::UpdateSlot)
      .def("get_slot", &Hashtable::GetSlot)
      .def("delete", &Hashtable::Delete)
      .def("ids_map", &Hashtable::ids_map)
      .def_readonly("hashtable_tag", &Hashtable::kNullIndex)
      // additions (no counterpart in the reference's binding): what its C++ reaches directly
      // (csrc/serialize: InsertLookupIndexWithIndicator, ids_num, SliceInfo) and the batch-plan path
      .def("ids_num", &Hashtable::ids_num)
      .def("slice_info", &Hashtable::SliceInfo)
      .def("embedding_shape", &Hashtable::EmbeddingShape)
      .def("device", [](const HashTablePtr& self) { return self->device(); })
      .def("dtype", [](const HashTablePtr& self) { return self->dtype(); })
      .def("has_grad", &Hashtable::has_grad)
      .def("grad_pairs", &Hashtable::GradPairs)
      .def("insert_lookup_index", &Hashtable::InsertLookupIndex)
      .def("insert_lookup_index_with_indicator", &Hashtable::InsertLookupIndexWithIndicator)
      .def("lookup_index_readonly", &Hashtable::LookupIndexReadOnly)
      .def("lookup_index", &Hashtable::LookupIndex)
      .def("reserve", &Hashtable::Reserve)
      .def("emb_blocks",
           [](const HashTablePtr& self) {
             auto emb = self->RawSlotGroup()->EmbSlot();
             return std::make_tuple(emb->Chunks(), emb->ChunkRows());
           })
      .def("slot_blocks",
           [](const HashTablePtr& self, const std::string& name) {
             return self->RawSlotGroup()->GetSlotByName(name)->Chunks();
           })
      .def("plan_lookup", &Hashtable::PlanLookup)
      .def("plan_index", &Hashtable::PlanIndex)
      .def("lookup_index_counted", &Hashtable::LookupIndexCounted)
      .def("settle_count", &Hashtable::SettleCount)
      .def("settle_lookup", &Hashtable::SettleLookup)
      .def("expand_rows", &Hashtable::ExpandRows)
      .def("dense_lookup_expand", &Hashtable::DenseLookupExpand)
      .def("accept_split_grad", &Hashtable::AcceptSplitGrad)
      .def("accept_grad_ex", &Hashtable::AcceptGradEx)
      .def("accept_planned_grad", &Hashtable::AcceptPlannedGrad)
      .def("evict_older", &Hashtable::EvictOlder)
      .def("id_map_stats", &Hashtable::IdMapStats)
      .def("pending_grads", &Hashtable::PendingGrads)
      .def("id_map_handle", [](const HashTablePtr& self) { return reinterpret_cast<int64_t>(self->id_map()); });

  def_optimizer<recis::optim::SparseAdamW>(m, "SparseAdamW");
  def_optimizer<recis::optim::SparseAdam>(m, "SparseAdam");
  def_optimizer<recis::optim::SparseAdamWTF>(m, "SparseAdamWTF");
  def_optimizer<recis::optim::SparseAdagrad>(m, "SparseAdagrad");  // an addition

  m.def("make_hashtable", Hashtable::Make);

  // ---- checkpoints (csrc/bind.cc:147-170)
  using namespace recis::serialize;
  m.class_<WriteBlock>("WriteBlock")
      .def("tensor_name", [](const WriteBlockPtr& self) { return self->TensorName(); })
      .def("slice_info", [](const WriteBlockPtr& self) { return self->SliceInfo(); })
      .def("is_dense", [](const WriteBlockPtr& self) { return self->IsDense(); })  // an addition
      // additions: blocks made from tensors the caller holds (tools, tests)
      .def_static("make_tensor", MakeTensorWriteBlock)
      .def_static("make_array", MakeArrayWriteBlock);
  m.class_<Saver>("Saver")
      .def(torch::init<int64_t, int64_t, int64_t, const std::string>())
      .def("make_write_blocks", &Saver::MakeWriteBlocks)
      .def("save", &Saver::Save);
  m.class_<Loader>("Loader")
      .def(torch::init<const std::string, int64_t, c10::Dict<std::string, HashTablePtr>,
                       c10::Dict<std::string, at::Tensor>>())
      .def("default_load_info", &Loader::DefaultLoadInfo)
      .def("load", &Loader::Load);
  m.class_<CheckpointReader>("CheckpointReader")
      .def(torch::init<std::string>())
      .def("init", &CheckpointReader::Init)
      .def("list_tensor_names", &CheckpointReader::ListTensors)
      .def("read_tensor", &CheckpointReader::LoadTensor)
      .def("tensor_shape", &CheckpointReader::TensorShape)
      .def("tensor_dtype", &CheckpointReader::TensorType);
  // additions: the directory writer by itself (the reference reaches it from C++ only) and two
  // helpers for tools that read or write single data files
  m.class_<SaveBundle>("SaveBundle")
      .def(torch::init<std::string, int64_t, int64_t, int64_t, double>())
      .def("add_block", &SaveBundle::AddBlock)
      .def("save", &SaveBundle::Save)
      .def("merge_meta_info", &SaveBundle::MergeMetaInfo);
  m.def("write_data_file", [](const std::string& path, const std::string& json_path, std::vector<WriteBlockPtr> blocks) {
    WriteDataFile(path, json_path, blocks);
  });
  // per block of the file, in file order: (name, dtype string, shape, first byte, end byte)
  m.def("read_data_file_header", [](const std::string& path) {
    std::vector<std::tuple<std::string, std::string, std::vector<int64_t>, int64_t, int64_t>> out;
    for (const auto& kv : ReadDataFileHeader(path, nullptr)) {
      out.emplace_back(kv.first, DtypeToString(kv.second.dtype), kv.second.shape, kv.second.offset_beg,
                       kv.second.offset_end);
    }
    return out;
  });
  m.def("unique_plan", recis::unique_plan);  // an addition: see plan.h
  // an addition: the integer a ScalarType crosses the binding as (Slot.dtype(), HashtableImpl.dtype())
  m.def("scalar_type_code", [](const at::Tensor& t) { return t.scalar_type(); });

  m.def("ragged_to_dense", recis::functional::ragged_to_dense);
  m.def("ragged_to_sparse", recis::functional::ragged_to_sparse);
  m.def("uint64_mod", recis::functional::uint64_mod);
  m.def("bucketize_op", recis::functional::bucketize_op);
  m.def("fused_multi_hash", recis::functional::fused_multi_hash);
  m.def("segment_mean", recis::functional::segment_mean);
  m.def("segment_sum", recis::functional::segment_sum);

  m.def("block_insert", recis::functional::block_insert);
  m.def("block_insert_with_mask", recis::functional::block_insert_with_mask);
  m.def("block_gather", recis::functional::block_gather);
  m.def("block_filter", recis::functional::block_filter);
  m.def("gather", recis::functional::gather);
  m.def("block_apply_adamw", recis::functional::block_apply_adamw);
  m.def("block_apply_adagrad", recis::functional::block_apply_adagrad);  // an addition
  m.def("fused_bucketized_mod", recis::functional::fused_bucketized_mod);  // an addition

  m.def("generate_ids", recis::functional::generate_ids_op);
  m.def("free_ids", recis::functional::free_ids_op);
  m.def("mask_key_index", recis::functional::mask_key_index_op);
  m.def("scatter_ids_with_mask", recis::functional::scatter_ids_with_mask_op);

  m.def("ids_encode", recis::functional::ids_encode);
  m.def("merge_offsets", recis::functional::merge_offsets);
  m.def("ids_partition", recis::functional::ids_partition);
  m.def("segment_reduce_forward", recis::functional::segment_reduce_forward);
  m.def("segment_reduce_backward", recis::functional::segment_reduce_backward);
  m.def("gen_segment_indices_by_offset", recis::functional::gen_segment_indices_by_offset);
  m.def("dense_to_ragged", recis::functional::dense_to_ragged);
  m.def("fused_uint64_mod", recis::functional::fused_uint64_mod);
  m.def("fused_bucketized", recis::functional::fused_bucketized);
  m.def("fused_hash", recis::functional::fused_hash);
  m.def("fused_ragged_cutoff", recis::functional::fused_ragged_cutoff);
  m.def("fused_ragged_cutoff_3D", recis::functional::fused_ragged_cutoff_3D);
  m.def("feature_cross_ragged", recis::functional::feature_cross_ragged);
  m.def("ragged_tile", recis::functional::ragged_tile);
  m.def("ragged_tile_back", recis::functional::ragged_tile_back);
  m.def("calc_ragged_index", recis::functional::calc_ragged_index);
}
