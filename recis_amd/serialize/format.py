"""On-disk layout of a table checkpoint, host side only (no device code in this file).

A checkpoint directory holds (csrc/serialize/name.cc:15-62, save_bundle.cc:56-330):

* ``model-XXXXXX-of-YYYYYY.safetensors`` data files, XXXXXX = shard_index * parallel + writer,
  YYYYYY = parallel * shard_num. Each file is ``u64 header_size | header | raw blocks``; the
  header is compact JSON ``{name: {"dtype", "shape", "data_offsets"}}`` in block order, padded with
  1..8 spaces to a multiple of 8 (table_writer.cc:60-82), offsets relative to the end of the header;
* ``index``: ``{"block_index": {block name: file number}, "file_index": {file name: number}}``
  (index_info.cc:18-27,93-105);
* ``tensorkey.json``: on-disk name -> model block name for table blocks (save_bundle.cc:84-105);
* ``torch_rank_weights_embs_table_multi_shard.json``: a description of every block for
  downstream tools (save_bundle.cc:277-318).

Names. A table block is ``<child>@<slot>`` (slot ``id`` for the keys) with the slice string
``begin@end@size`` (zero padded to the width of ``size``, slice_info.cc:38-48); its model block
name is ``<child>@<slot>^<slice>`` and its on-disk name ``<child>.<slot>/part_<shard>_<shards>``.
A dense tensor keeps its name with the slice ``" "``: block name ``<name>^ `` on disk and in the index.
"""
import json
import os
import struct
import threading
import time

import numpy as np
import torch

INTER_SEP = "^"  # serialize/string_sep.cc:5
INTRA_SEP = "@"  # serialize/string_sep.cc:6
PART = "/part_"
EMPTY_SLICE = " "
ID_SLOT = "id"
INDEX_FILE = "index"
TENSORKEY_FILE = "tensorkey.json"
RANK_JSON_FILE = "torch_rank_weights_embs_table_multi_shard.json"

# dtype_serialize.cc:4-66 (it writes "bool" but only reads "BOOL": both are read here)
_DTYPE_TO_STR = {torch.bool: "bool", torch.int8: "I8", torch.uint8: "U8", torch.int16: "I16", torch.int32: "I32",
                 torch.int64: "I64", torch.float16: "F16", torch.bfloat16: "BF16", torch.float32: "F32",
                 torch.float64: "F64"}
_STR_TO_DTYPE = {v: k for k, v in _DTYPE_TO_STR.items()}
_STR_TO_DTYPE["BOOL"] = torch.bool
# save_bundle.cc:40-54
_TYPE_MAP = {"F64": "float64", "F32": "float32", "F16": "float16", "BF16": "bfloat16", "I64": "int64",
             "U64": "uint64", "I32": "int32", "U32": "uint32", "I16": "int16", "U16": "uint16", "I8": "int8",
             "U8": "uint8", "BOOL": "bool"}


def block_write_size():
    return int(os.environ.get("RECIS_BLOCK_WRITE_SIZE", 1 << 20))  # name.cc:135-142


def block_read_size():
    return int(os.environ.get("RECIS_BLOCK_READ_SIZE", 1 << 20))  # name.cc:144-151


def dtype_to_str(dtype):
    try:
        return _DTYPE_TO_STR[dtype]
    except KeyError:
        raise RuntimeError("Dtype: %s not supported!" % dtype)


def str_to_dtype(s):
    try:
        return _STR_TO_DTYPE[s]
    except KeyError:
        raise RuntimeError("dtype: %s is invalid" % s)


def slice_to_string(begin, end, size):
    width = len(str(size))
    return "%s@%s@%s" % (str(begin).zfill(width), str(end).zfill(width), size)


def slice_from_string(msg):
    tokens = msg.split(INTRA_SEP)
    if len(tokens) != 3:
        raise RuntimeError("SliceInfo::FromString failed, msg: %s" % msg)
    return tuple(int(t) for t in tokens)


def slices_intersect(a, b):
    """slice_info.h:22-37: same slice_size and overlapping [begin, end) ranges."""
    def one_way(l, r):
        return (l[0] <= r[0] < l[1]) or (l[0] < r[1] <= l[1])
    return a[2] == b[2] and (one_way(a, b) or one_way(b, a))


def data_file_name(file_index, file_count):
    return "model-%06d-of-%06d.safetensors" % (file_index, file_count)


def block_name(tensor_name, slice_info, sep=INTER_SEP):
    return "%s%s%s" % (tensor_name, sep, slice_info)


def _compact(obj):
    return json.dumps(obj, separators=(",", ":"), ensure_ascii=False)


class WriteBlock:
    """One named block of a data file. ``chunks()`` yields C-contiguous host buffers
    (anything ``file.write`` takes) whose sizes add up to ``nbytes``."""

    def __init__(self, tensor_name, slice_info, dense, dtype, shape):
        self.tensor_name, self.slice_info, self.dense = tensor_name, slice_info, dense
        self.dtype, self.shape = dtype, [int(s) for s in shape]
        n = 1
        for s in self.shape:
            n *= s
        self.nbytes = n * torch.empty((), dtype=dtype).element_size()

    def chunks(self):
        raise NotImplementedError

    def meta_key(self):
        # write_block.cc:117-121: a renamed table block carries no slice suffix
        if PART in self.tensor_name:
            return self.tensor_name
        return block_name(self.tensor_name, self.slice_info)


class TensorWriteBlock(WriteBlock):
    """A dense tensor, copied to the host when the block is made (write_block.cc:88-97)."""

    def __init__(self, tensor_name, tensor):
        t = tensor.detach().cpu().contiguous()
        super().__init__(tensor_name, EMPTY_SLICE, True, t.dtype, t.shape)
        self._t = t

    def chunks(self):
        if self.nbytes:
            yield self._t.reshape(-1).view(torch.uint8).numpy()


class ArrayWriteBlock(WriteBlock):
    """A table block whose rows are already in host memory (ids, or tests)."""

    def __init__(self, tensor_name, slice_info, array):
        t = torch.as_tensor(array).contiguous()
        super().__init__(tensor_name, slice_info, False, t.dtype, t.shape)
        self._t = t

    def chunks(self):
        if self.nbytes:
            yield self._t.reshape(-1).view(torch.uint8).numpy()


def _write_data_file(path, json_path, blocks):
    """table_writer.cc:48-88: header (offsets in block order), then the blocks."""
    meta, offset = {}, 0
    for b in blocks:
        meta[b.meta_key()] = {"dtype": dtype_to_str(b.dtype), "shape": b.shape,
                              "data_offsets": [offset, offset + b.nbytes], "dense": b.dense}
        offset += b.nbytes
    with open(json_path, "w") as f:
        f.write(_compact(meta))
    for v in meta.values():
        del v["dense"]
    header = _compact(meta).encode()
    header += b" " * (8 - len(header) % 8)
    with open(path, "wb", buffering=8 << 20) as f:
        f.write(struct.pack("<Q", len(header)))
        f.write(header)
        for b in blocks:
            written = 0
            for c in b.chunks():
                f.write(c)
                written += memoryview(c).nbytes
            if written != b.nbytes:
                raise RuntimeError("block %s wrote %d bytes, header says %d" % (b.tensor_name, written, b.nbytes))


class IndexInfo:
    """index_info.cc: block name -> file number, file name -> number."""

    def __init__(self):
        self.file_index, self.block_index = {}, {}

    def append(self, name, file_name):
        if file_name not in self.file_index:
            self.file_index[file_name] = len(self.file_index)
        self.block_index[name] = self.file_index[file_name]

    def merge_from(self, other):
        base = len(self.file_index)
        for k, v in other.file_index.items():
            self.file_index[k] = base + v
        for k, v in other.block_index.items():
            self.block_index[k] = base + v

    def serialize(self):
        return _compact({"block_index": dict(sorted(self.block_index.items())),
                         "file_index": dict(sorted(self.file_index.items()))})

    @classmethod
    def deserialize(cls, text, name_map=None):
        obj, info = cls(), json.loads(text)
        obj.file_index = dict(info["file_index"])
        for k, v in info["block_index"].items():
            obj.block_index[(name_map or {}).get(k, k)] = v
        return obj


def _wait_for(paths, what, timeout):
    deadline = time.monotonic() + timeout
    while True:
        missing = [p for p in paths if not os.path.exists(p)]
        if not missing:
            return
        if time.monotonic() > deadline:
            raise RuntimeError("timed out waiting for %s of other shards: %s" % (what, missing))
        time.sleep(0.1)


class SaveBundle:
    """save_bundle.cc:56-330. Blocks go to ``parallel`` data files round robin in the order they are
    added; every file is written by its own thread. Shard 0 merges the per-shard side files; it
    waits (up to ``merge_timeout`` seconds) for those of the other shards."""

    def __init__(self, path, parallel, shard_index, shard_num, merge_timeout=3600.0):
        if parallel <= 0:
            raise RuntimeError("parallel must > 0")
        if shard_index < 0 or shard_num <= shard_index:
            raise RuntimeError("shard_num must > shard_index")
        self.path, self.parallel, self.shard_index, self.shard_num = path, parallel, shard_index, shard_num
        self.merge_timeout = merge_timeout
        self._writers = [[] for _ in range(parallel)]
        self._file_names = [data_file_name(shard_index * parallel + i, parallel * shard_num)
                            for i in range(parallel)]
        self._next = 0
        self._index = IndexInfo()
        self._name_map = {}

    def _tmp(self, kind, writer=None, shard=None):
        shard = self.shard_index if shard is None else shard
        if kind == "data":
            return os.path.join(self.path, "ckpt-%07d-%07d.data.tmp" % (shard, writer))
        if kind == "json":
            return os.path.join(self.path, "ckpt-%07d-%07d.json.tmp" % (shard, writer))
        if kind == "index":
            return os.path.join(self.path, "ckpt-%07d.index" % shard)
        return os.path.join(self.path, "%dtensorkey.json" % shard)

    def add_block(self, block):
        w = self._next
        self._next = (self._next + 1) % self.parallel
        self._writers[w].append(block)
        if not block.dense:
            new_name = block.tensor_name.replace(INTRA_SEP, ".") + "%s%d_%d" % (PART, self.shard_index,
                                                                                  self.shard_num)
            if new_name not in self._name_map:
                self._name_map[new_name] = block_name(block.tensor_name, block.slice_info)
            block.tensor_name = new_name
            self._index.append(new_name, self._file_names[w])
        else:
            self._index.append(block_name(block.tensor_name, block.slice_info), self._file_names[w])

    def save(self):
        """Index first, data files next, the shard's name map last: shard 0 takes the name map of
        another shard as the sign that all of that shard's files are complete."""
        os.makedirs(self.path, exist_ok=True)
        tmp = self._tmp("index") + ".tmp"
        with open(tmp, "w") as f:
            f.write(self._index.serialize())
        os.replace(tmp, self._tmp("index"))
        errors = []

        def run(i):
            try:
                _write_data_file(self._tmp("data", i), self._tmp("json", i), self._writers[i])
            except BaseException as e:  # noqa: BLE001 - re-raised on the calling thread
                errors.append(e)

        threads = [threading.Thread(target=run, args=(i,)) for i in range(self.parallel) if self._writers[i]]
        for t in threads:
            t.start()
        for t in threads:
            t.join()
        if errors:
            raise errors[0]
        for i in range(self.parallel):
            if self._writers[i]:
                os.replace(self._tmp("data", i), os.path.join(self.path, self._file_names[i]))
        tmp = self._tmp("tensorkey") + ".tmp"
        with open(tmp, "w") as f:
            f.write(json.dumps(dict(sorted(self._name_map.items())), indent=4))
        os.replace(tmp, self._tmp("tensorkey"))
        if self.shard_index == 0:
            _wait_for([self._tmp("tensorkey", shard=s) for s in range(self.shard_num)], "files",
                      self.merge_timeout)
            self._merge_rank_json()
            self._merge_tensorkey_json()

    def _merge_rank_json(self):
        # save_bundle.cc:277-318. A writer with no blocks leaves no side file.
        files = [self._tmp("json", w, s) for s in range(self.shard_num) for w in range(self.parallel)]
        sub = {}
        for f in files:
            if not os.path.exists(f):
                continue
            with open(f) as fh:
                sub.update(json.load(fh))
            os.remove(f)
        combined = {}
        for k in sorted(sub):
            v = sub[k]
            if v["dense"]:
                v.pop("data_offsets")
                v.update(name=k, dtype=_TYPE_MAP.get(v["dtype"], ""), dimension=0, is_hashmap=False)
            elif ".embedding" in k:
                v.pop("data_offsets")
                v.update(name=k, dtype=_TYPE_MAP.get(v["dtype"], ""), dimension=int(v["shape"][-1]),
                         hashmap_key=k.replace(".embedding", ".id"), hashmap_key_dtype="int64", hashmap_value=k,
                         is_hashmap=True)
            combined[k] = dict(sorted(v.items()))
        with open(os.path.join(self.path, RANK_JSON_FILE), "w") as f:
            f.write(json.dumps(combined, indent=4))

    def _merge_tensorkey_json(self):
        files = [self._tmp("tensorkey", shard=s) for s in range(self.shard_num)]
        combined = {}
        for f in files:
            with open(f) as fh:
                combined.update(json.load(fh))
            os.remove(f)
        with open(os.path.join(self.path, TENSORKEY_FILE), "w") as f:
            f.write(json.dumps(dict(sorted(combined.items())), indent=4))

    def merge_meta_info(self):
        """save_bundle.cc:124-171: shard 0 folds every shard's index into ``index``."""
        if self.shard_index != 0:
            return
        files = [self._tmp("index", shard=s) for s in range(self.shard_num)]
        _wait_for(files, "indexes", self.merge_timeout)
        merged = IndexInfo()
        for f in sorted(files):
            with open(f) as fh:
                merged.merge_from(IndexInfo.deserialize(fh.read()))
            os.remove(f)
        tmp = os.path.join(self.path, INDEX_FILE + ".tmp")
        with open(tmp, "w") as f:
            f.write(merged.serialize())
        os.replace(tmp, os.path.join(self.path, INDEX_FILE))


class BlockInfo:
    def __init__(self, dtype, shape, beg, end, path):
        self.dtype, self.shape, self.offset_beg, self.offset_end, self.path = dtype, shape, beg, end, path

    @property
    def size(self):
        return self.offset_end - self.offset_beg

    def read(self, byte_offset=0, nbytes=None):
        """Bytes [byte_offset, byte_offset + nbytes) of the block as a uint8 array."""
        nbytes = self.size - byte_offset if nbytes is None else nbytes
        with open(self.path, "rb") as f:
            f.seek(self.offset_beg + byte_offset)
            buf = np.empty(nbytes, np.uint8)
            got = f.readinto(memoryview(buf))
        if got != nbytes:
            raise RuntimeError("short read in %s" % self.path)
        return buf

    def read_into(self, out, byte_offset=0):
        """Fills the uint8 array ``out`` with the block's bytes from ``byte_offset`` on."""
        with open(self.path, "rb", buffering=0) as f:
            f.seek(self.offset_beg + byte_offset)
            view, got = memoryview(out), 0
            while got < len(view):
                n = f.readinto(view[got:])
                if not n:
                    raise RuntimeError("short read in %s" % self.path)
                got += n

    def read_tensor(self):
        if self.size == 0:
            return torch.empty(self.shape, dtype=self.dtype)
        return torch.from_numpy(self.read()).view(self.dtype).reshape(self.shape)


def read_data_file_header(path, name_map=None):
    """table_reader.cc:34-60: block name -> BlockInfo with absolute file offsets."""
    with open(path, "rb") as f:
        (meta_size,) = struct.unpack("<Q", f.read(8))
        meta = json.loads(f.read(meta_size).decode())
    base = 8 + meta_size
    out = {}
    for k, v in meta.items():
        if k == "__metadata__":
            continue
        for key in ("dtype", "shape", "data_offsets"):
            if key not in v:
                raise RuntimeError("BlockInfo::DecodeFromJson %s failed, json: %s" % (key, v))
        beg, end = v["data_offsets"]
        out[(name_map or {}).get(k, k)] = BlockInfo(str_to_dtype(v["dtype"]), [int(s) for s in v["shape"]],
                                                    beg + base, end + base, path)
    return out


class LoadBundle:
    """load_bundle.cc:17-112: the index and name map of a checkpoint directory; file headers are
    parsed on first use."""

    def __init__(self, path):
        self.path = path
        with open(os.path.join(path, TENSORKEY_FILE)) as f:
            self._name_map = json.load(f)
        index_file = os.path.join(path, INDEX_FILE)
        if not os.path.exists(index_file):
            raise RuntimeError("[%s] not found" % index_file)
        with open(index_file) as f:
            self._index = IndexInfo.deserialize(f.read(), self._name_map)
        self._file_by_number = {v: k for k, v in self._index.file_index.items()}
        self._headers = {}

    def _header(self, number):
        if number not in self._headers:
            self._headers[number] = read_data_file_header(os.path.join(self.path, self._file_by_number[number]),
                                                          self._name_map)
        return self._headers[number]

    def has_tensor(self, tensor_name):
        prefix = tensor_name  # index_info.cc:58-66: prefix match on the bare tensor name
        return any(k.startswith(prefix) for k in self._index.block_index)

    def list_tensor(self):
        names = set()
        for k in self._index.block_index:
            tokens = k.split(INTER_SEP)
            if len(tokens) != 2:
                raise RuntimeError("block_name: %s, type error" % k)
            names.add(tokens[0])
        return sorted(names)

    def slice_infos(self, tensor_name):
        out = []
        for k in self._index.block_index:
            if k.startswith(tensor_name):
                tokens = k.split(INTER_SEP)
                if len(tokens) != 2:
                    raise RuntimeError("block_name: %s, type error" % k)
                out.append(tokens[1])
        return out

    def block_info(self, name):
        return self._header(self._index.block_index[name])[name]

    def tensor_shape(self, tensor_name):
        shape = []
        for s in self.slice_infos(tensor_name):
            b = self.block_info(block_name(tensor_name, s))
            if not shape:
                shape = list(b.shape)
            else:
                shape[0] += b.shape[0]
        return shape

    def tensor_type(self, tensor_name):
        return self.block_info(block_name(tensor_name, self.slice_infos(tensor_name)[0])).dtype


class CheckpointReader:
    """recis/serialize/checkpoint_reader.py over csrc/serialize/checkpoint_reader.cc:14-66: reads
    whole tensors (table blocks of all shards concatenated in slice order) into host memory."""

    def __init__(self, path):
        self._bundle = LoadBundle(path)

    def tensor_names(self):
        return self._bundle.list_tensor()

    def read_tensor(self, name):
        if not self._bundle.has_tensor(name):
            raise RuntimeError("%s not found" % name)
        parts = []
        for s in sorted(self._bundle.slice_infos(name)):
            b = self._bundle.block_info(block_name(name, s))
            parts.append(b.read_tensor())
        return parts[0] if len(parts) == 1 else torch.cat(parts, 0)

    def tensor_shape(self, name):
        if not self._bundle.has_tensor(name):
            raise RuntimeError("%s not found" % name)
        return self._bundle.tensor_shape(name)

    def tensor_dtype(self, name):
        if not self._bundle.has_tensor(name):
            raise RuntimeError("%s not found" % name)
        return self._bundle.tensor_type(name)
