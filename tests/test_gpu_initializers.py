"""Every row initialiser drawing on the GPU (torch's device RNG) and feeding a table: support and
moments of the rows a lookup returns. The arithmetic of each initialiser is pinned bit for bit
against the reference's generators on the CPU (tests/test_initializers.py); here the same code
runs with device tensors."""
import math

import pytest
import torch

from recis_amd.nn import initializers as I
from recis_amd.nn.modules.hashtable import HashtableImpl

pytestmark = pytest.mark.gpu

BS, D = 2048, 32
XB = math.sqrt(6.0 / (BS + D))
KB = math.sqrt(3.0) * math.sqrt(2.0) / math.sqrt(D)
CASES = [
    ("constant", lambda: I.ConstantInitializer(0.25), 0.25, 0.25, 0.25, 0.0),
    ("uniform", lambda: I.UniformInitializer(-1.0, 3.0), -1.0, 3.0, 1.0, 16 / 12),
    ("normal", lambda: I.NormalInitializer(0.5, 0.1), -math.inf, math.inf, 0.5, 0.01),
    ("xavier_uniform", lambda: I.XavierUniformInitializer(), -XB, XB, 0.0, XB * XB / 3),
    ("xavier_normal", lambda: I.XavierNormalInitializer(), -math.inf, math.inf, 0.0, 2.0 / (BS + D)),
    ("kaiming_uniform", lambda: I.KaimingUniformInitializer(), -KB, KB, 0.0, KB * KB / 3),
    ("kaiming_normal", lambda: I.KaimingNormalInitializer(), -KB, KB, 0.0, KB * KB / 3),
    ("trunc_normal", lambda: I.TruncNormalInitializer(0.0, 1.0, -2.0, 2.0), -2.0, 2.0, 0.0, 0.774),
]


@pytest.mark.parametrize("name,make,lo,hi,mean,var", CASES, ids=[c[0] for c in CASES])
def test_rows_of_a_table_follow_the_initialiser(name, make, lo, hi, mean, var):
    torch.manual_seed(0)
    init = make()
    init.set_shape([BS, D])
    init.set_dtype(torch.float32)
    table = HashtableImpl(BS, [D], torch.float32, torch.device("cuda"), False, [name], init.build().impl())
    ids = torch.arange(5 * BS + 3, device="cuda") * 7919
    index, rows = table.embedding_lookup(ids, False)
    assert rows.shape == (ids.numel(), D) and rows.is_cuda
    x = rows.double()
    assert float(x.min()) >= lo - 1e-6 and float(x.max()) <= hi + 1e-6
    assert abs(float(x.mean()) - mean) < 0.02 * max(1.0, abs(mean)) + 3 * math.sqrt(var / x.numel()) + 1e-9
    assert abs(float(x.var()) - var) <= 0.03 * var + 1e-12
    # evicted rows are drawn again from the same law (Slot::GenVal)
    fresh = table.slot_group().emb_slot().gen_val(4096)
    assert fresh.shape == (4096, D) and fresh.is_cuda
    if not name.startswith(("xavier", "kaiming")):   # those take their fans from the 4096 rows asked for
        assert float(fresh.min()) >= lo - 1e-6 and float(fresh.max()) <= hi + 1e-6


def test_a_cpu_generator_is_refused_for_a_gpu_table():
    init = I.UniformInitializer(generator=torch.Generator(device="cpu"))
    init.set_shape([BS, D])
    with pytest.raises(RuntimeError, match="lives on"):
        HashtableImpl(BS, [D], torch.float32, torch.device("cuda"), False, ["t"], init.build().impl())
