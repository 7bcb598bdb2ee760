// The registration block the reference has at csrc/bind.cc:46-211: namespace `recis`, the same
// class and operator names, the reference's C++ signatures (torch infers the schemas from them).
// Loaded with torch.classes.load_library(<package>/lib/recis.so), as recis/__init__.py:8-16 does.
// Not registered: gauc_calc, adam_tf_apply, ragged_to_sparse and the Saver / Loader /
// CheckpointReader / WriteBlock classes (metrics, the dense optimizer and a CPU-only op are outside
// this build; checkpoints are written and read by the Python package recis_amd.serialize).
#include <torch/custom_class.h>
#include <torch/library.h>

#include "ops.h"
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

  m.class_<Slot>("Slot")
      .def("block_size", &Slot::BlockSize)
      .def("name", &Slot::Name)
      .def("flat_size", &Slot::FlatSize)
      .def("value", &Slot::Value)
      .def("values", &Slot::ValuesDeref);

  m.class_<SlotGroup>("SlotGroup")
      .def("slot_by_name", &SlotGroup::GetSlotByName)
      .def("slot_by_index", &SlotGroup::GetSlotByIndex)
      .def("slot_index", &SlotGroup::GetSlotByIndex)  // sic: the reference binds this name to GetSlotByIndex too
      .def("slots", &SlotGroup::Slots);

  m.class_<Generator>("Generator")
      .def_static("generate", Generator::DoGenerator)
      .def_static("make_constant_generator", recis::embedding::MakeConstantGenerator)
      .def_static("make_uniform_generator", recis::embedding::MakeUniformGenerator)
      .def_static("make_normal_generator", recis::embedding::MakeNormalGenerator)
      .def_static("make_xavier_uniform_generator", recis::embedding::MakeXavierUniFormGenerator)
      .def_static("make_xavier_normal_generator", recis::embedding::MakeXavierNormalGenerator)
      .def_static("make_kaiming_uniform_generator", recis::embedding::MakeKaimingUniformGenerator)
      .def_static("make_kaiming_normal_generator", recis::embedding::MakeKaimingNormalGenerator)
      .def_static("make_trunc_normal_generator", recis::embedding::MakeTruncNormalGenerator);

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
      .def_readonly("hashtable_tag", &Hashtable::kNullIndex);

  def_optimizer<recis::optim::SparseAdamW>(m, "SparseAdamW");
  def_optimizer<recis::optim::SparseAdam>(m, "SparseAdam");
  def_optimizer<recis::optim::SparseAdamWTF>(m, "SparseAdamWTF");
  def_optimizer<recis::optim::SparseAdagrad>(m, "SparseAdagrad");  // an addition

  m.def("make_hashtable", Hashtable::Make);

  m.def("ragged_to_dense", recis::functional::ragged_to_dense);
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
