"""The nine row initialisers (recis_amd/nn/initializers.py) on the CPU.

Pins, strongest first:
* against the reference's own generators (csrc/embedding/initializer.cc:26-366, compiled into
  oracle/_ref and driven with torch's default generator seeded the same way): bit for bit, for
  every kind, for a block of the generator's own shape and for a differently sized tensor
  (``Slot::GenVal``, whose fan-out is the number of rows asked for);
* closed forms: support, mean and variance of every distribution, the fan arithmetic against
  ``torch.nn.init`` on a ``[block_size, D]`` tensor, the truncated normal's moments against scipy.
"""
import math

import numpy as np
import pytest
import torch

from oracle import ref_ops
from recis_amd.nn import initializers as I

BS, D = 1024, 24


def _built(init, shape=(BS, D)):
    init.set_shape(list(shape))
    init.set_dtype(torch.float32)
    return init.build().impl()


CASES = [
    # name, initialiser, reference kind + params (p0..p3, fan mode)
    ("constant", lambda: I.ConstantInitializer(0.3), (0, 0.3, 0, 0, 0, 0)),
    ("uniform", lambda: I.UniformInitializer(-0.7, 0.1), (1, -0.7, 0.1, 0, 0, 0)),
    ("normal", lambda: I.NormalInitializer(0.1, 0.01), (2, 0.1, 0.01, 0, 0, 0)),
    ("xavier_uniform", lambda: I.XavierUniformInitializer(1.7), (3, 1.7, 0, 0, 0, 0)),
    ("xavier_normal", lambda: I.XavierNormalInitializer(0.6), (4, 0.6, 0, 0, 0, 0)),
    ("kaiming_uniform_in", lambda: I.KaimingUniformInitializer(0.2, "fan_in"), (5, 0.2, 0, 0, 0, 0)),
    ("kaiming_uniform_out", lambda: I.KaimingUniformInitializer(0.0, "fan_out"), (5, 0.0, 0, 0, 0, 1)),
    # the reference's Python class for "kaiming normal" builds the uniform generator too
    ("kaiming_normal_is_uniform", lambda: I.KaimingNormalInitializer(0.2, "fan_in"), (5, 0.2, 0, 0, 0, 0)),
    ("trunc_normal", lambda: I.TruncNormalInitializer(0.05, 0.3, -0.2, 0.6), (7, 0.05, 0.3, -0.2, 0.6, 0)),
    ("trunc_normal_default", lambda: I.TruncNormalInitializer(), (7, 0.0, 1.0, -2.0, 2.0, 0)),
]


@pytest.mark.skipif(not ref_ops.available(), reason="the reference build (oracle/_ref) is absent")
@pytest.mark.parametrize("name,make,ref", CASES, ids=[c[0] for c in CASES])
@pytest.mark.parametrize("rows", [0, 37])
def test_bit_exact_against_the_reference_generators(name, make, ref, rows):
    kind, p0, p1, p2, p3, mode = ref
    seed = 20 + kind
    params = np.array([kind, BS, D, seed, p0, p1, p2, p3, mode, rows], np.float64)
    exp = ref_ops.run("generate", [params])[0]
    g = _built(make())
    torch.manual_seed(seed)
    got = g.gen([rows, D]) if rows else g.gen()
    assert got.dtype == torch.float32 and list(got.shape) == [rows or BS, D]
    np.testing.assert_array_equal(got.numpy(), exp)


def _moments(t):
    x = t.double().flatten()
    return float(x.mean()), float(x.var()), float(x.min()), float(x.max())


def test_uniform_and_normal_moments():
    torch.manual_seed(1)
    m, v, lo, hi = _moments(_built(I.UniformInitializer(-0.7, 0.1), (4096, 64)).gen())
    assert -0.7 <= lo and hi < 0.1 + 1e-7
    assert abs(m - (-0.3)) < 2e-3 and abs(v - 0.8 ** 2 / 12) < 5e-4
    m, v, _, _ = _moments(_built(I.NormalInitializer(0.1, 0.5), (4096, 64)).gen())
    assert abs(m - 0.1) < 4e-3 and abs(v - 0.25) < 3e-3


@pytest.mark.parametrize("gain", [1.0, 2.5])
def test_xavier_fans_match_torch_nn_init(gain):
    """Same seed, same tensor shape: torch.nn.init's own fan computation gives the same values."""
    for ours, theirs in ((I.XavierUniformInitializer, torch.nn.init.xavier_uniform_),
                         (I.XavierNormalInitializer, torch.nn.init.xavier_normal_)):
        torch.manual_seed(3)
        got = _built(ours(gain)).gen()
        torch.manual_seed(3)
        exp = theirs(torch.empty(BS, D), gain=gain)
        assert torch.equal(got, exp)
    bound = gain * math.sqrt(6.0 / (BS + D))
    m, v, lo, hi = _moments(_built(I.XavierUniformInitializer(gain), (BS, D)).gen())
    assert -bound <= lo and hi <= bound and abs(v - bound ** 2 / 3) < 0.05 * bound ** 2


@pytest.mark.parametrize("mode", ["fan_in", "fan_out"])
@pytest.mark.parametrize("a", [0.0, 0.3])
def test_kaiming_fans_match_torch_nn_init(mode, a):
    torch.manual_seed(5)
    got = _built(I.KaimingUniformInitializer(a, mode)).gen()
    torch.manual_seed(5)
    exp = torch.nn.init.kaiming_uniform_(torch.empty(BS, D), a=float(np.float32(a)), mode=mode, nonlinearity="leaky_relu")
    assert torch.equal(got, exp)
    fan = D if mode == "fan_in" else BS
    bound = math.sqrt(3.0) * math.sqrt(2.0 / (1 + a * a)) / math.sqrt(fan)
    _, v, lo, hi = _moments(got)
    assert -bound * (1 + 1e-6) <= lo and hi <= bound * (1 + 1e-6) and abs(v - bound ** 2 / 3) < 0.05 * bound ** 2
    with pytest.raises(ValueError):
        _built(I.KaimingUniformInitializer(a, "fan_avg"))


def test_fans_of_a_chunk_of_several_blocks_are_those_of_one_block():
    """Row storage allocates several [block_size, D] blocks as one tensor; the values must be drawn
    as for one block (fan_out = block_size), whatever the chunk size."""
    g = _built(I.XavierUniformInitializer(1.0), (BS, D))
    torch.manual_seed(9)
    chunk = g.gen([4 * BS, D], [BS, D])
    bound = math.sqrt(6.0 / (BS + D))
    assert float(chunk.abs().max()) <= bound
    assert float(chunk.abs().max()) > 0.99 * bound
    torch.manual_seed(9)
    rows = g.gen([7, D])            # Slot::GenVal of 7 rows: fans of a [7, D] tensor, as in the reference
    assert float(rows.abs().max()) > bound


def test_trunc_normal_support_and_moments():
    from scipy.stats import truncnorm

    mean, std, a, b = 0.05, 0.3, -0.2, 0.6
    torch.manual_seed(7)
    x = _built(I.TruncNormalInitializer(mean, std, a, b), (4096, 64)).gen()
    m, v, lo, hi = _moments(x)
    assert np.float32(a) <= lo and hi <= np.float32(b)
    dist = truncnorm((a - mean) / std, (b - mean) / std, loc=mean, scale=std)
    assert abs(m - dist.mean()) < 2e-3 and abs(v - dist.var()) < 2e-3
    # the inverse-CDF construction against a quantile of the exact law
    assert abs(float(x.double().flatten().quantile(0.9)) - dist.ppf(0.9)) < 5e-3


def test_half_precision_rows_and_integer_constant_rows():
    torch.manual_seed(11)
    init = I.NormalInitializer(0.0, 1.0)
    init.set_shape([BS, D])
    init.set_dtype(torch.bfloat16)
    assert init.build().impl().gen().dtype == torch.bfloat16
    c = I.ConstantInitializer(3)
    c.set_shape([8, 1])
    c.set_dtype(torch.int64)
    assert c.build().impl().gen().tolist() == [[3]] * 8


def test_an_initializer_is_built_once_and_needs_building():
    init = I.NormalInitializer()
    with pytest.raises(RuntimeError):
        init.impl()
    init.set_shape([4, 2])
    assert init.build().impl() is init.build().impl()


def test_generator_of_another_device_is_refused():
    g = _built(I.UniformInitializer(generator=torch.Generator(device="cpu")))
    g.set_device(torch.device("cpu"))
    with pytest.raises(RuntimeError, match="lives on"):
        g.set_device(torch.device("cuda"))
