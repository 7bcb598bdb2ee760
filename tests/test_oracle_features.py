"""Pins the tagging / dedup / feature-op part of the CPU oracle.

Sources of truth: reference known-answer vectors (hashes, Mod, IDMultiHash),
golden vectors produced from the reference's own CPU hash sources
(tests/golden/hash_vectors.json), the pure-torch reference implementations the
reference tests carry (ids_encode, ids_partition), numpy / torch library
routines (uint64 %, torch.bucketize) and explicit edge cases from the code.
"""
import ctypes
import json
import os

import numpy as np
import pytest
import torch

import oracle

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
REF_HASH = os.path.join(os.path.dirname(GOLDEN), "..", "oracle", "_ref", "libref_hash.so")


def test_hash_kats_from_reference_tests():
    # tests/ops/fused_hash_test.py:20-21,37-38; tests/feature_engine/op_test.py:115-116
    off = [0, 3, 6]
    a = np.array([0, 1, 2, 1, 2, 3], np.int8)
    b = np.array([0, 5, 5, 5, 6, 7], np.int8)
    assert oracle.hash_strings(a, off, "farm").tolist() == [-7736835464683084646, -5546720800891377920]
    assert oracle.hash_strings(b, off, "farm").tolist() == [-4442022684725028445, -909183002746659612]
    assert oracle.hash_strings(a, off, "murmur").tolist() == [-4003751876240412087, -1042754718167355375]
    assert oracle.hash_strings(b, off, "murmur").tolist() == [-5541886947548579749, 4434088491466393040]


def test_hash_golden_vectors_all_length_classes():
    with open(os.path.join(GOLDEN, "hash_vectors.json")) as f:
        vec = json.load(f)["vectors"]
    data = b"".join(bytes.fromhex(v["hex"]) for v in vec)
    off = np.concatenate([[0], np.cumsum([len(v["hex"]) // 2 for v in vec])])
    arr = np.frombuffer(data, dtype=np.uint8)
    assert oracle.hash_strings(arr, off, "farm").tolist() == [v["farm"] for v in vec]
    assert oracle.hash_strings(arr, off, "murmur").tolist() == [v["murmur"] for v in vec]


@pytest.mark.skipif(not os.path.exists(REF_HASH), reason="oracle/_ref not built (no reference tree)")
def test_hash_against_compiled_reference(rng):
    ref = ctypes.CDLL(REF_HASH)
    ref.ref_farm_fingerprint64.restype = ctypes.c_uint64
    ref.ref_murmur64.restype = ctypes.c_uint64
    lens = rng.integers(0, 300, size=400)
    data = rng.integers(0, 256, size=int(lens.sum()), dtype=np.uint8)
    off = np.concatenate([[0], np.cumsum(lens)])
    farm = oracle.hash_strings(data, off, "farm")
    mur = oracle.hash_strings(data, off, "murmur")
    for i, n in enumerate(lens.tolist()):
        s = data[off[i]:off[i + 1]].tobytes()
        assert np.int64(np.uint64(ref.ref_farm_fingerprint64(s, ctypes.c_size_t(n)))) == farm[i]
        assert np.int64(np.uint64(ref.ref_murmur64(s, ctypes.c_size_t(n), ctypes.c_uint64(0)))) == mur[i]


def test_uint64_mod(rng):
    # tests/feature_engine/op_test.py:17-24 and tests/ops/fused_uint64_mod_test.py:19-26
    assert oracle.uint64_mod([1001, 1002, 1003], 1000).tolist() == [1, 2, 3]
    x = rng.integers(-2**63, 2**63 - 1, size=1000, dtype=np.int64)
    for mod in (1, 7, 1000000, 2**40 + 3):
        exp = (x.astype(np.uint64) % np.uint64(mod)).astype(np.int64)
        np.testing.assert_array_equal(oracle.uint64_mod(x, mod), exp)
    assert oracle.uint64_mod([-1], 10)[0] == (2**64 - 1) % 10


def test_bucketize_vs_torch_and_edges(rng):
    b = np.sort(rng.standard_normal(64)).astype(np.float32)
    v = rng.standard_normal(5000).astype(np.float32) * 2
    v[:64] = b  # exact ties
    exp = torch.bucketize(torch.tensor(v), torch.tensor(b), right=True).numpy()
    np.testing.assert_array_equal(oracle.bucketize(v, b), exp)
    # tests/feature_engine/op_test.py:27-36 uses right=False on tie-free data: same there
    edge = np.array([np.nan, np.inf, -np.inf, b[0], b[-1]], np.float32)
    assert oracle.bucketize(edge, b).tolist() == [64, 64, 0, 1, 64]
    assert oracle.bucketize(np.array([1.0], np.float32), np.zeros(0, np.float32)).tolist() == [0]


def test_multi_hash_kat_and_negative():
    # tests/feature_engine/op_test.py:95-110: IDMultiHash([1000]*4) on 1001..1003
    def largest_prime_le(n):
        def is_p(k):
            return k > 1 and all(k % d for d in range(2, int(k ** 0.5) + 1))
        while not is_p(n):
            n -= 1
        return n
    muls, mods = [1, 3, 5, 7], [29, 47, 67, 83]
    primes = [largest_prime_le(m * 1000) for m in mods]
    outs = oracle.multi_hash([1001, 1002, 1003], muls, primes, [1000] * 4)
    assert [o.tolist() for o in outs] == [[1, 2, 3], [3, 6, 9], [5, 10, 15], [7, 14, 21]]
    # C semantics for negatives and wrap-around (python ints as the model)
    x = np.array([-5, -2**62, 2**62 + 12345, -1], np.int64)
    for mul, p, bkt in ((3, 46993, 1000), (7, 82997, 37)):
        exp = []
        for xi in x.tolist():
            t = (xi * mul + 2**63) % 2**64 - 2**63  # wrap to int64
            r = abs(t) % p * (1 if t >= 0 else -1)  # C remainder truncates toward zero
            exp.append(((r + p) % p) % bkt)
        assert oracle.multi_hash(x, [mul], [p], [bkt])[0].tolist() == exp


def test_ids_encode_vs_reference_torch_impl(rng):
    # tests/ops/ids_encode_test.py:8-18
    ids = [rng.integers(-2**62, 2**62, size=n, dtype=np.int64) for n in (10, 100, 7)]
    tids = [0, 5, 4094]
    exp = []
    for i, t in zip(ids, tids):  # the torch formulation of the reference test (int64 wrap-around)
        mask = torch.bitwise_left_shift(torch.ones(len(i), dtype=torch.int64), 52) - 1
        off = torch.bitwise_left_shift(torch.tensor(t, dtype=torch.int64), 52)
        exp.append((torch.bitwise_and(torch.tensor(i), mask) + off).numpy())
    exp = np.concatenate(exp)
    np.testing.assert_array_equal(oracle.ids_encode(ids, tids), exp)


def _ids_partition_torch(ids, world):
    """The pure-torch reference of tests/ops/ids_partition_test.py:8-25."""
    ids, rev = torch.unique(ids, return_inverse=True)
    mod = torch.bitwise_and(ids, torch.tensor(65535))
    arg = torch.argsort(mod, stable=True)
    mod_sorted = mod[arg]
    m, n = divmod(65536, world)
    parts = [m + (i < n) for i in range(world)]
    bnd = torch.cumsum(torch.tensor(parts), 0)
    bi = torch.cat((torch.tensor([0]), torch.searchsorted(mod_sorted, bnd)))
    return ids[arg], bi[1:] - bi[:-1], torch.argsort(arg)[rev]


def test_ids_partition_vs_reference_torch_impl(rng):
    for n, world in ((10, 1), (1000, 128), (20000, 256), (5000, 3)):
        ids = rng.integers(0, n * 100, size=n)
        u, c, inv = oracle.ids_partition(ids, world)
        eu, ec, einv = _ids_partition_torch(torch.tensor(ids), world)
        np.testing.assert_array_equal(u, eu.numpy())
        np.testing.assert_array_equal(c, ec.numpy())
        np.testing.assert_array_equal(inv, einv.numpy())
        np.testing.assert_array_equal(u[inv], ids)


def test_ids_partition_negative_ids_unsigned_order():
    # ids_partition_kernel.cu:36-43: the rotated key is compared as unsigned
    ids = np.array([-1, 1 << 16, 0, -(1 << 16), 5], np.int64)
    u, c, inv = oracle.ids_partition(ids, 1)
    np.testing.assert_array_equal(u[inv], ids)
    assert u.tolist() == [0, 1 << 16, -(1 << 16), 5, -1]
    assert c.tolist() == [5]
