"""The ``TORCH_LIBRARY(recis)`` registration (recis_amd/lib/recis.so), CPU side: the library loads,
every operator the reference registers on this path exists with the schema torch infers from the
reference's C++ signature (csrc/bind.cc:145-210, csrc/ops/*.h), the custom classes exist with the
reference's method names (bind.cc:47-143), and the host-only classes (Generator, ChildrenInfo)
behave like the Python mirrors that are pinned against the reference's compiled generators."""
import json
import os

import pytest
import torch

from recis_amd import torch_library
from recis_amd.nn import initializers

torch_library.load()

H = "__torch__.torch.classes.recis."
SCHEMAS = {
    "make_hashtable": "recis::make_hashtable(int _0, int[] _1, ScalarType _2, Device _3, bool _4, str[] _5, "
                      + H + "Generator _6, int _7, int _8, int _9) -> " + H + "HashtableImpl _0",
    "gather": "recis::gather(Tensor _0, Tensor _1) -> Tensor _0",
    "block_gather": "recis::block_gather(Tensor _0, Tensor[] _1, int _2, int _3, bool _4) -> Tensor _0",
    "block_insert": "recis::block_insert(Tensor _0, Tensor _1, Tensor[] _2, int _3) -> ()",
    "block_insert_with_mask": "recis::block_insert_with_mask(Tensor _0, Tensor _1, Tensor _2, Tensor[] _3, int _4) -> ()",
    "block_filter": "recis::block_filter(Tensor _0, Tensor[] _1, int _2, int _3) -> Tensor _0",
    "block_apply_adamw": "recis::block_apply_adamw(Tensor _0, Tensor _1, Tensor[] _2, Tensor _3, Tensor _4, Tensor _5, "
                         "Tensor[] _6, Tensor[] _7, float _8, float _9, float _10, float _11, float _12, int _13) -> ()",
    "generate_ids": "recis::generate_ids(int _0, Tensor[] _1, int _2, int _3, int _4) -> Tensor _0",
    "free_ids": "recis::free_ids(Tensor _0, Tensor[] _1, int _2, int _3) -> ()",
    "mask_key_index": "recis::mask_key_index(Tensor _0, Tensor _1, Tensor _2, int _3) -> (Tensor _0, Tensor _1)",
    "scatter_ids_with_mask": "recis::scatter_ids_with_mask(Tensor _0, Tensor _1, Tensor _2) -> Tensor _0",
    "ids_encode": "recis::ids_encode(Tensor[] _0, Tensor _1) -> Tensor _0",
    "merge_offsets": "recis::merge_offsets(Tensor[] _0, Tensor _1) -> Tensor _0",
    "ids_partition": "recis::ids_partition(Tensor _0, int _1) -> (Tensor _0, Tensor _1, Tensor _2)",
    "segment_reduce_forward": "recis::segment_reduce_forward(Tensor _0, Tensor? _1, Tensor _2, Tensor _3, str _4) -> Tensor _0",
    "segment_reduce_backward": "recis::segment_reduce_backward(Tensor _0, Tensor? _1, Tensor _2, Tensor _3, int _4, str _5) -> Tensor _0",
    "gen_segment_indices_by_offset": "recis::gen_segment_indices_by_offset(Tensor _0) -> Tensor _0",
    "segment_sum": "recis::segment_sum(Tensor _0, Tensor? _1, Tensor _2, Tensor _3, Scalar _4) -> Tensor _0",
    "segment_mean": "recis::segment_mean(Tensor _0, Tensor? _1, Tensor _2, Scalar _3) -> Tensor _0",
    "uint64_mod": "recis::uint64_mod(Tensor _0, Scalar _1) -> Tensor _0",
    "bucketize_op": "recis::bucketize_op(Tensor _0, Tensor _1) -> Tensor _0",
    "fused_uint64_mod": "recis::fused_uint64_mod(Tensor[] _0, Tensor _1) -> Tensor[] _0",
    "fused_bucketized": "recis::fused_bucketized(Tensor[] _0, Tensor[] _1) -> Tensor[] _0",
    "fused_hash": "recis::fused_hash(Tensor[] _0, Tensor[] _1, str _2) -> Tensor[] _0",
    "fused_multi_hash": "recis::fused_multi_hash(Tensor[] _0, Tensor[] _1, Tensor[] _2, Tensor[] _3) -> Tensor[] _0",
    "ragged_tile": "recis::ragged_tile(int[] _0, int[] _1, Tensor _2, Tensor _3, Tensor _4) -> Tensor[] _0",
    "ragged_tile_back": "recis::ragged_tile_back(Tensor _0, int[] _1, Tensor _2, Tensor _3, Tensor _4) -> Tensor _0",
    "ragged_to_dense": "recis::ragged_to_dense(Tensor _0, Tensor[] _1, Scalar _2) -> Tensor _0",
    "dense_to_ragged": "recis::dense_to_ragged(Tensor _0, bool _1, Tensor _2) -> (Tensor _0, Tensor _1)",
    "fused_ragged_cutoff": "recis::fused_ragged_cutoff(Tensor[] _0, Tensor[] _1, Tensor _2, Tensor _3, Tensor _4) -> "
                           "(Tensor[] _0, Tensor[] _1, Tensor[] _2, Tensor[] _3, Tensor _4, Tensor _5)",
    "fused_ragged_cutoff_3D": "recis::fused_ragged_cutoff_3D(Tensor[] _0, Tensor[] _1, Tensor[] _2, Tensor _3, Tensor _4, "
                              "Tensor _5) -> (Tensor[] _0, Tensor[] _1, Tensor[] _2)",
    "feature_cross_ragged": "recis::feature_cross_ragged(Tensor _0, Tensor _1, Tensor _2, Tensor _3, Tensor _4, Tensor _5) "
                            "-> (Tensor _0, Tensor _1, Tensor _2)",
    "calc_ragged_index": "recis::calc_ragged_index(Tensor _0, Tensor _1, Tensor _2, Tensor _3, Tensor _4, Tensor _5, "
                         "Tensor _6) -> (Tensor _0, Tensor _1)",
}

CLASS_METHODS = {
    "ChildrenInfo": ["index_bits_num", "id_bits_num", "index_mask", "id_mask", "max_children_num", "encode_id",
                     "children", "child_index", "has_child", "child_at", "is_coalesce"],
    "Slot": ["block_size", "name", "flat_size", "value", "values"],
    "SlotGroup": ["slot_by_name", "slot_by_index", "slot_index", "slots"],
    "HashtableImpl": ["accept_grad", "grad", "clear_grad", "embedding_lookup", "insert", "clear", "clear_id", "ids",
                      "slot_group", "children_info", "append_filter_slot", "append_step_filter_slot", "update_slot",
                      "get_slot", "delete", "ids_map"],
    "SparseAdam": ["step", "add_parameters", "zero_grad", "state_dict", "load_state_dict", "set_grad_accum_steps",
                   "set_lr", "make"],
    "SparseAdamW": ["step", "add_parameters", "zero_grad", "state_dict", "load_state_dict", "set_grad_accum_steps",
                    "set_lr", "make"],
    "SparseAdamWTF": ["step", "add_parameters", "zero_grad", "state_dict", "load_state_dict", "set_grad_accum_steps",
                      "set_lr", "make"],
    "Generator": ["generate", "make_constant_generator", "make_uniform_generator", "make_normal_generator",
                  "make_xavier_uniform_generator", "make_xavier_normal_generator", "make_kaiming_uniform_generator",
                  "make_kaiming_normal_generator", "make_trunc_normal_generator"],
}


@pytest.mark.parametrize("name", sorted(SCHEMAS))
def test_operator_schema(name):
    assert str(getattr(torch.ops.recis, name).default._schema) == SCHEMAS[name]


def _bound_methods():
    """class name -> names of the methods registered for it (static ones are attributes of the class)."""
    out = {}
    for schema in torch._C._jit_get_custom_class_schemas():
        if schema.arguments and (H in str(schema.arguments[0].type)):
            out.setdefault(str(schema.arguments[0].type).split(".")[-1], set()).add(schema.name)
    return out


@pytest.mark.parametrize("cls", sorted(CLASS_METHODS))
def test_class_methods(cls):
    c = getattr(torch.classes.recis, cls)
    bound = _bound_methods().get(cls, set())
    for m in CLASS_METHODS[cls]:
        assert m in bound or hasattr(c, m), "%s.%s" % (cls, m)


def _gen(kind, shape, dtype, *args):
    return getattr(torch.classes.recis.Generator, "make_%s_generator" % kind)(shape, dtype, *args)


GEN_CASES = [
    ("constant", (0.25,), initializers.ConstantInitializer(0.25)),
    ("uniform", (-0.3, 0.7, None), initializers.UniformInitializer(-0.3, 0.7)),
    ("normal", (0.1, 0.02, None), initializers.NormalInitializer(0.1, 0.02)),
    ("xavier_uniform", (1.3, None), initializers.XavierUniformInitializer(1.3)),
    ("xavier_normal", (0.7, None), initializers.XavierNormalInitializer(0.7)),
    ("kaiming_uniform", (0.2, "fan_out", "leaky_relu", None),
     initializers.KaimingUniformInitializer(0.2, "fan_out", "leaky_relu")),
    ("trunc_normal", (0.1, 0.5, -0.4, 0.9, None), initializers.TruncNormalInitializer(0.1, 0.5, -0.4, 0.9)),
]


@pytest.mark.parametrize("kind,args,py", GEN_CASES, ids=[c[0] for c in GEN_CASES])
def test_python_initializers_build_the_registered_generators(kind, args, py):
    """recis_amd.nn.initializers builds torch.classes.recis.Generator objects with the arguments of the
    registered factories (the rows they draw are pinned bit for bit against the reference's own generators,
    csrc/embedding/initializer.cc:26-366, in tests/test_initializers.py)."""
    shape = [64, 16]
    py.set_shape(shape)
    py.set_dtype(torch.float32)
    py.build()
    torch.manual_seed(7)
    want = py.generate()
    g = _gen(kind, shape, torch.float32, *args)
    torch.manual_seed(7)
    got = torch.classes.recis.Generator.generate(g)
    assert got.shape == (64, 16) and torch.equal(got, want)
    torch.manual_seed(7)
    assert torch.equal(g.gen(), want) and g.gen([5, 16]).shape == (5, 16)


def test_kaiming_normal_generator_moments():
    """make_kaiming_normal_generator draws normals (the reference's Python class of that name builds
    the uniform generator, recis/nn/initializers.py:585, so the Python mirror has no twin to compare
    with): std = gain / sqrt(fan_in), torch::nn::init::kaiming_normal_."""
    g = _gen("kaiming_normal", [4096, 64], torch.float32, 0.0, "fan_in", "relu", None)
    torch.manual_seed(3)
    t = torch.classes.recis.Generator.generate(g)
    torch.manual_seed(3)
    want = torch.empty(4096, 64).normal_(0, (2.0 ** 0.5) / 64 ** 0.5)
    assert torch.equal(t, want)


def test_generator_rejects_bad_names():
    with pytest.raises(RuntimeError, match="fan_in, fan_out"):
        _gen("kaiming_uniform", [4, 4], torch.float32, 0.0, "fan_avg", "relu", None)
    with pytest.raises(RuntimeError, match="not in"):
        _gen("kaiming_uniform", [4, 4], torch.float32, 0.0, "fan_in", "gelu", None)


def test_gpu_only_ops_refuse_cpu_tensors():
    """There is no CPU path behind this registration: a CPU tensor is an error, never a fallback."""
    with pytest.raises(RuntimeError, match="GPU tensor"):
        torch.ops.recis.gather(torch.arange(3), torch.zeros(4, 2))
    with pytest.raises(RuntimeError, match="GPU"):
        g = _gen("constant", [4, 2], torch.float32, 0.0)
        torch.ops.recis.make_hashtable(4, [2], torch.float32, torch.device("cpu"), False, ["t"], g, 0, 65536, 65536)


def test_scalar_type_numbers_of_the_binding():
    """Methods that return a ScalarType (Slot.dtype(), HashtableImpl.dtype()) hand Python its number."""
    from recis_amd import _lib
    for code, dtype in _lib.SCALAR_TYPE_DTYPES.items():
        assert torch.ops.recis.scalar_type_code(torch.empty(0, dtype=dtype)) == code


# What the reference registers and this library leaves out, each with its reason.
NOT_REGISTERED = {
    "gauc_calc": "a metric (recis/metrics): not on the sparse-embedding path",
    "adam_tf_apply": "the dense TF-style Adam (recis/optim/adamw_tf.py): not on the sparse-embedding path",
}


def test_every_name_the_reference_registers_is_registered():
    """tests/golden/registered_names.json lists the operators and the class methods of the reference's
    TORCH_LIBRARY(recis) block (written by tests/golden/make_registered_names.py from csrc/bind.cc:46-211)."""
    golden = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "registered_names.json")))
    missing = [op for op in golden["ops"] if op not in NOT_REGISTERED and not hasattr(torch.ops.recis, op)]
    assert not missing, missing
    bound = _bound_methods()
    for cls, methods in golden["classes"].items():
        c = getattr(torch.classes.recis, cls)
        lost = [m for m in methods if m not in bound.get(cls, set()) and not hasattr(c, m)]
        assert not lost, (cls, lost)
    # (read-only attributes need an instance: tests/test_gpu_torch_library.py reads HashtableImpl.hashtable_tag)
    assert golden["readonly_attributes"] == {"HashtableImpl": ["hashtable_tag"]}


def test_children_are_validated_as_in_the_reference():
    """csrc/embedding/children_info.cc:38-48: no children, too many, more than one without coalescing and
    duplicate names are refused (before anything touches a device)."""
    gen = torch.classes.recis.Generator.make_constant_generator([4, 2], torch.float32, 0.0)

    def make(coalesce, children):
        return torch.ops.recis.make_hashtable(4, [2], torch.float32, torch.device("cpu"), coalesce, children, gen, 0,
                                              65536, 65536)
    with pytest.raises(RuntimeError, match="empty children"):
        make(True, [])
    with pytest.raises(RuntimeError, match="exceeds max children size"):
        make(True, ["c%d" % i for i in range(4095)])
    with pytest.raises(RuntimeError, match="non coalesce has more than one child"):
        make(False, ["a", "b"])
    with pytest.raises(RuntimeError, match="duplicate child"):
        make(True, ["a", "b", "a"])
    with pytest.raises(RuntimeError, match="tables live in GPU memory"):   # valid names: the device is looked at next
        make(True, ["c%d" % i for i in range(4094)])
