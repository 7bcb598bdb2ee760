"""On-disk layout of a table checkpoint: the Python face of the writer and reader of recis.so
(recis_amd/csrc/torch/serialize.cc, the counterpart of csrc/serialize/*), for tools and tests that
work on single blocks, files or directories.

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
import numpy as np
import torch

from .. import _lib

INTER_SEP = "^"  # serialize/string_sep.cc:5
INTRA_SEP = "@"  # serialize/string_sep.cc:6
EMPTY_SLICE = " "
ID_SLOT = "id"
INDEX_FILE = "index"
TENSORKEY_FILE = "tensorkey.json"
RANK_JSON_FILE = "torch_rank_weights_embs_table_multi_shard.json"

# dtype_serialize.cc:4-66 (it writes "bool" but only reads "BOOL": both are read)
_STR_TO_DTYPE = {"bool": torch.bool, "BOOL": torch.bool, "I8": torch.int8, "U8": torch.uint8, "I16": torch.int16,
                 "I32": torch.int32, "I64": torch.int64, "F16": torch.float16, "BF16": torch.bfloat16,
                 "F32": torch.float32, "F64": torch.float64}


def _classes():
    from .. import torch_library
    torch_library.load()
    return torch.classes.recis


def _ops():
    from .. import torch_library
    torch_library.load()
    return torch.ops.recis


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


def block_name(tensor_name, slice_info, sep=INTER_SEP):
    return "%s%s%s" % (tensor_name, sep, slice_info)


def TensorWriteBlock(tensor_name, tensor):
    """A dense tensor as a ``torch.classes.recis.WriteBlock``, copied to the host when the block is
    made (write_block.cc:88-97)."""
    return _classes().WriteBlock.make_tensor(tensor_name, tensor)


def ArrayWriteBlock(tensor_name, slice_info, array):
    """A table block whose rows are already in host memory, as a ``torch.classes.recis.WriteBlock``."""
    return _classes().WriteBlock.make_array(tensor_name, slice_info, torch.as_tensor(array))


def SaveBundle(path, parallel, shard_index, shard_num, merge_timeout=3600.0):
    """save_bundle.cc:56-330 (``torch.classes.recis.SaveBundle``): ``add_block``, ``save``,
    ``merge_meta_info``. Blocks go to ``parallel`` data files round robin in the order they are added;
    every file is written by its own thread. Shard 0 merges the per-shard side files; it waits (up to
    ``merge_timeout`` seconds) for those of the other shards."""
    return _classes().SaveBundle(path, parallel, shard_index, shard_num, float(merge_timeout))


def _write_data_file(path, json_path, blocks):
    """table_writer.cc:48-88: header (offsets in block order), then the blocks."""
    _ops().write_data_file(path, json_path, list(blocks))


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


def read_data_file_header(path):
    """table_reader.cc:34-60: block name -> BlockInfo with absolute file offsets."""
    return {name: BlockInfo(_STR_TO_DTYPE[dtype], list(shape), beg, end, path)
            for name, dtype, shape, beg, end in _ops().read_data_file_header(path)}


class CheckpointReader:
    """recis/serialize/checkpoint_reader.py over ``torch.classes.recis.CheckpointReader``
    (csrc/serialize/checkpoint_reader.cc:14-66): reads whole tensors (table blocks of all shards
    concatenated in slice order) into host memory."""

    def __init__(self, path):
        self.reader = _classes().CheckpointReader(path)
        self.reader.init()

    def tensor_names(self):
        return self.reader.list_tensor_names()

    def read_tensor(self, name):
        return self.reader.read_tensor(name)

    def tensor_shape(self, name):
        return self.reader.tensor_shape(name)

    def tensor_dtype(self, name):
        return self.reader.tensor_dtype(name).dtype


def raise_device_errors():
    _lib.raise_device_errors()
