"""Checkpoint directory layout (host side): what the writer produces is read back by the
safetensors library and by the reference's own LoadBundle, the side files satisfy the rules of the
reference's save/load test (tests/serialize/save_load_test.py:86-139), and a data file written by
the reference's TableWriter is reproduced byte for byte."""
import json
import os

import numpy as np
import pytest
import torch
from safetensors import safe_open

from oracle import ref_ops
from recis_amd.serialize import format as fmt

needs_ref = pytest.mark.skipif(not ref_ops.available(), reason="oracle/_ref/ref_ops not built")


def _path_arg(p):
    return np.frombuffer(p.encode(), dtype=np.int8).copy()


def _make_blocks(rng, shard=(0, 65536, 65536)):
    sl = fmt.slice_to_string(*shard)
    data = {}
    blocks = []
    for child, n in (("user", 1000), ("item", 37), ("empty", 0)):
        ids = torch.from_numpy(rng.integers(0, 1 << 50, n))
        emb = torch.from_numpy(rng.standard_normal((n, 8)).astype(np.float32))
        m = torch.from_numpy(rng.standard_normal((n, 8)).astype(np.float32)).to(torch.bfloat16)
        stamp = torch.from_numpy(rng.integers(0, 100, (n, 1)))
        for slot, t in (("id", ids), ("embedding", emb), ("sparse_adam_exp_avg", m), ("step_filter", stamp)):
            blocks.append(fmt.ArrayWriteBlock("%s@%s" % (child, slot), sl, t))
            data["%s@%s" % (child, slot)] = t
    dense = {"tower.0.weight": torch.from_numpy(rng.standard_normal((5, 3)).astype(np.float32)),
             "tower.0.bias": torch.from_numpy(rng.standard_normal(3)), "step": torch.tensor(17)}
    for k, v in dense.items():
        blocks.append(fmt.TensorWriteBlock(k, v))
        data[k] = v
    return blocks, data


def _save(path, blocks, parallel, shard_index=0, shard_num=1):
    b = fmt.SaveBundle(path, parallel, shard_index, shard_num, merge_timeout=5.0)
    for blk in blocks:
        b.add_block(blk)
    b.save()
    b.merge_meta_info()


@pytest.mark.parametrize("parallel", [1, 4, 32])
def test_written_directory_reads_back(tmp_path, parallel):
    rng = np.random.default_rng(parallel)
    blocks, data = _make_blocks(rng)
    path = str(tmp_path)
    _save(path, blocks, parallel)
    left = sorted(os.listdir(path))
    assert not [f for f in left if "tmp" in f or f.startswith("ckpt-") or f[0].isdigit()], left

    # the safetensors library reads every data file (the reference test's check, :166-186)
    index = json.load(open(os.path.join(path, "index")))
    names = json.load(open(os.path.join(path, "tensorkey.json")))
    seen = {}
    for fname in index["file_index"]:
        assert os.path.getsize(os.path.join(path, fname)) > 8
        with safe_open(os.path.join(path, fname), "pt") as f:
            for k in f.keys():
                seen[k] = f.get_tensor(k)
    assert len(seen) == len(data)
    for k, t in seen.items():
        if k in names:
            assert k.endswith("/part_0_1") and "@" not in k
            model_name, sl = names[k].split("^")
            assert sl == "00000@65536@65536"
        else:
            model_name, sl = k.split("^")
            assert sl == " "
        assert torch.equal(t, data[model_name]) and t.dtype == data[model_name].dtype
        assert index["block_index"][k] == index["file_index"][
            [fn for fn in index["file_index"] if k in safe_open(os.path.join(path, fn), "pt").keys()][0]]

    # rules of the reference test for the description file (:86-139)
    rank = json.load(open(os.path.join(path, fmt.RANK_JSON_FILE)))
    assert len(rank) == len(data) and set(names) <= set(rank)
    for k, v in rank.items():
        if ".embedding" in k:
            for sub in ("dimension", "dtype", "name", "dense", "hashmap_key", "hashmap_key_dtype", "hashmap_value",
                        "is_hashmap"):
                assert sub in v
            assert v["is_hashmap"] and ".id" in v["hashmap_key"] and v["hashmap_key"] in rank and v["dimension"] == 8
        elif v["dense"]:
            assert v["dimension"] == 0 and not v["is_hashmap"] and v["name"] == k
    assert all(0 <= v < len(index["file_index"]) for v in index["block_index"].values())

    # the reader of this package
    r = fmt.CheckpointReader(path)
    assert sorted(r.tensor_names()) == sorted(data)
    for k, t in data.items():
        got = r.read_tensor(k)
        assert got.dtype == t.dtype == r.tensor_dtype(k) and r.tensor_shape(k) == list(t.shape)
        assert torch.equal(got, t)


def test_two_shards_merge(tmp_path):
    rng = np.random.default_rng(7)
    path = str(tmp_path)
    b1, d1 = _make_blocks(rng, (32768, 65536, 65536))
    b0, d0 = _make_blocks(rng, (0, 32768, 65536))
    _save(path, [b for b in b1 if not b.is_dense()], 2, shard_index=1, shard_num=2)   # a non-zero shard saves no dense tensors
    _save(path, b0, 2, shard_index=0, shard_num=2)
    assert sorted(f for f in os.listdir(path) if f.endswith(".safetensors")) == [
        "model-%06d-of-000004.safetensors" % i for i in range(4)]
    r = fmt.CheckpointReader(path)
    got = r.read_tensor("user@embedding")  # slices in ascending order: shard 0 first
    assert torch.equal(got, torch.cat([d0["user@embedding"], d1["user@embedding"]]))
    assert r.tensor_shape("user@id") == [2000]
    assert torch.equal(r.read_tensor("tower.0.weight"), d0["tower.0.weight"])
    index = json.load(open(os.path.join(path, "index")))
    assert sorted(index["file_index"].values()) == [0, 1, 2, 3]


def test_slice_strings_and_intersection():
    assert fmt.slice_to_string(0, 65536, 65536) == "00000@65536@65536"
    assert fmt.slice_to_string(8192, 16384, 65536) == "08192@16384@65536"
    assert fmt.slice_from_string("08192@16384@65536") == (8192, 16384, 65536)
    assert fmt.slices_intersect((0, 32768, 65536), (16384, 49152, 65536))
    assert fmt.slices_intersect((0, 65536, 65536), (16384, 49152, 65536))
    assert not fmt.slices_intersect((0, 32768, 65536), (32768, 65536, 65536))
    assert not fmt.slices_intersect((0, 32768, 65536), (0, 32768, 1024))


@needs_ref
@pytest.mark.parametrize("parallel", [1, 3])
def test_reference_load_bundle_reads_the_directory(tmp_path, parallel):
    # csrc/serialize/load_bundle.cc:17-112 on a directory written here
    rng = np.random.default_rng(11)
    blocks, data = _make_blocks(rng)
    path = str(tmp_path)
    _save(path, blocks, parallel)
    text, shapes, ranges, totals = ref_ops.run("ckpt_inspect", [_path_arg(path)])
    lines = text.tobytes().decode().strip().split("\n")
    assert len(lines) == len(data)
    codes = {torch.float32: 6, torch.float64: 7, torch.int64: 4, torch.bfloat16: 15}  # c10::ScalarType
    index = json.load(open(os.path.join(path, "index")))
    names = {v: k for k, v in json.load(open(os.path.join(path, "tensorkey.json"))).items()}
    for line, shp, rng_, tot in zip(lines, shapes, ranges, totals):
        name, code, sl = line.split("\t")
        t = data[name]
        assert int(code) == codes[t.dtype]
        assert [int(x) for x in shp if x >= 0] == list(t.shape) == [int(x) for x in tot if x >= 0]
        assert sl == ("00000@65536@65536" if "@" in name else " ")
        disk_name = names.get(name + "^" + sl, name + "^" + sl)
        fname = [f for f, i in index["file_index"].items() if i == index["block_index"][disk_name]][0]
        with open(os.path.join(path, fname), "rb") as f:
            f.seek(int(rng_[0]))
            raw = f.read(int(rng_[1] - rng_[0]))
        assert raw == (t.contiguous().reshape(-1).view(torch.uint8).numpy().tobytes() if t.numel() else b"")


@needs_ref
@pytest.mark.parametrize("coalesced", [0, 1])
def test_data_file_of_reference_table_writer_is_reproduced(tmp_path, coalesced):
    # csrc/serialize/write_block.cc:33-199 + table_writer.cc:48-88 on a reference CPU Hashtable
    rng = np.random.default_rng(13 + coalesced)
    n, D, bs = 3000, 6, 256
    ids = rng.choice(1 << 40, n, replace=False).astype(np.int64)
    tag = rng.integers(0, 2, n) if coalesced else np.zeros(n, np.int64)
    rows = rng.standard_normal((n, D)).astype(np.float32)
    dense = rng.standard_normal((4, 5)).astype(np.float32)
    path = str(tmp_path)
    (count,) = ref_ops.run("ckpt_write_file", [_path_arg(path), np.asarray([bs, coalesced, 0, 65536, 65536], np.int64),
                                                 ids | (tag << 52), rows, dense])
    ref_file = os.path.join(path, "ref.safetensors")
    header = fmt.read_data_file_header(ref_file)
    children = ["a", "b"] if coalesced else ["a"]
    assert int(count[0]) == 3 * len(children) + 1 == len(header)
    sl = "00000@65536@65536"
    by_id = {int(i): r for i, r in zip(ids, rows)}
    blocks = []
    for c, child in enumerate(children):
        b_id = header["%s@id^%s" % (child, sl)]
        got_ids = b_id.read().view(np.int64)
        assert sorted(got_ids.tolist()) == sorted(ids[tag == c].tolist())   # stored without the tag
        got_rows = header["%s@embedding^%s" % (child, sl)].read().view(np.float32).reshape(-1, D)
        np.testing.assert_array_equal(got_rows, np.stack([by_id[int(i)] for i in got_ids]) if len(got_ids) else
                                      np.empty((0, D), np.float32))
        stamp = header["%s@step_filter^%s" % (child, sl)]
        assert stamp.shape == [len(got_ids), 1] and stamp.dtype == torch.int64
        assert (stamp.read().view(np.int64) == 7).all()
        blocks.append(fmt.ArrayWriteBlock(child + "@id", sl, got_ids))
        blocks.append(fmt.ArrayWriteBlock(child + "@embedding", sl, got_rows))
        blocks.append(fmt.ArrayWriteBlock(child + "@step_filter", sl, np.full((len(got_ids), 1), 7, np.int64)))
    np.testing.assert_array_equal(header["dense_w^ "].read().view(np.float32).reshape(4, 5), dense)
    blocks.append(fmt.TensorWriteBlock("dense_w", torch.from_numpy(dense)))
    mine = os.path.join(path, "mine.safetensors")
    fmt._write_data_file(mine, os.path.join(path, "mine.json"), blocks)
    assert open(mine, "rb").read() == open(ref_file, "rb").read()
    assert open(os.path.join(path, "mine.json")).read() == open(os.path.join(path, "ref.json")).read()
