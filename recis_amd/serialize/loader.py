"""Loader: fills tables and dense tensors from a checkpoint directory
(recis/serialize/loader.py:7-76 over csrc/serialize/{loader,load_info,load_internal,read_block,
ht_read_collection}.cc)."""
import json
from concurrent.futures import ThreadPoolExecutor

import torch

from . import format as fmt
from .. import _lib


def default_load_info(hashtables, tensors):
    """load_info.cc:17-33: {destination: {source: [slot names]}}; a dense tensor has no slots."""
    info = {}
    for ht in hashtables.values():
        impl = getattr(ht, "_hashtable_impl", ht)
        slots = [fmt.ID_SLOT] + [s.name() for s in impl.slot_group().slots()]
        for child in impl.children_info().children():
            info.setdefault(child, {})[child] = list(slots)
    for name in tensors:
        info.setdefault(name, {})[name] = []
    return info


def _accept_mask(ids, slice_info):
    """read_block.cc:52-65: a key belongs to this table when (uint64)key % slice_size is in
    [slice_begin, slice_end)."""
    slice_begin, slice_end, slice_size = slice_info
    if slice_size & (slice_size - 1) == 0:
        mod = ids & (slice_size - 1)
    else:
        mod = torch.from_numpy(ids.numpy().view("uint64") % slice_size).to(torch.int64)
    return (mod >= slice_begin) & (mod < slice_end)


def _load_table_blocks(ht, child, id_block, slot_blocks, parallel=1):
    """One (child, slice) group: keys first, then every slot in pieces of RECIS_BLOCK_READ_SIZE
    rows (read_block.cc:67-79,94-109,125-163)."""
    ids = id_block.read_tensor().reshape(-1)
    accept = _accept_mask(ids, ht.slice_info())
    info = ht.children_info()
    if info.is_coalesce():
        tagged = (ids & info.id_mask()) | (info.child_index(child) << info.id_bits_num())
        ids = torch.where(accept, tagged, ids)
    device = ht.device()
    accept_dev = accept.to(device)
    index = ht.insert_lookup_index_with_indicator(ids.to(device), accept_dev)
    step = fmt.block_read_size()
    pieces = []
    for slot, b in slot_blocks:
        want = [b.shape[0]] + slot.row_shape()
        if want != b.shape:
            raise RuntimeError("shape not match")
        if _lib.as_dtype(slot.dtype()) != b.dtype:
            raise RuntimeError("dtype not match")
        pieces += [(slot, b, beg, min(beg + step, b.shape[0])) for beg in range(0, b.shape[0], step)]
    if not pieces:
        return
    # File reads run on ``parallel`` threads into a ring of pinned buffers; this thread copies each
    # piece to the device and scatters it into the slot, in order.
    ring = max(2, min(parallel, len(pieces)) + 1)
    biggest = max((end - beg) * (b.size // b.shape[0]) for _, b, beg, end in pieces)
    bufs = [torch.empty(biggest, dtype=torch.uint8, pin_memory=True) for _ in range(ring)]
    done = [None] * ring

    def read(k):
        slot, b, beg, end = pieces[k]
        row_bytes = b.size // b.shape[0]
        if done[k % ring] is not None:
            done[k % ring].synchronize()      # the copy that last used this buffer has finished
        view = bufs[k % ring][: (end - beg) * row_bytes]
        b.read_into(view.numpy(), beg * row_bytes)
        return view

    with ThreadPoolExecutor(max_workers=max(1, min(parallel, ring - 1))) as pool, torch.cuda.device(device):
        futures = {}
        issued = 0
        for k in range(len(pieces)):
            while issued < len(pieces) and issued < k + ring - 1:
                futures[issued] = pool.submit(read, issued)
                issued += 1
            view = futures.pop(k).result()
            slot, b, beg, end = pieces[k]
            rows = view.to(device, non_blocking=True).view(b.dtype).reshape([end - beg] + b.shape[1:])
            ev = torch.cuda.Event()
            ev.record()
            done[k % ring] = ev
            slot.index_insert(index[beg:end], rows, accept_dev[beg:end])


class Loader:
    def __init__(self, checkpoint_path, hashtables=None, tensors=None, parallel=16, filter_func=lambda x: x):
        self._path = checkpoint_path
        self._hashtables = hashtables if hashtables is not None else {}
        self._tensors = tensors if tensors is not None else {}
        self._parallel = parallel
        self._filter_func = filter_func

    def default_load_info(self):
        return json.dumps(default_load_info(self._hashtables, self._tensors))

    def load(self):
        info = self._filter_func(json.loads(self.default_load_info()))
        self._load(info)

    def _load(self, info):
        bundle = fmt.LoadBundle(self._path)
        name_to_ht = {}
        for ht in self._hashtables.values():
            impl = getattr(ht, "_hashtable_impl", ht)
            for child in impl.children_info().children():
                name_to_ht[child] = impl
        # load_internal.cc:96-146
        for shared_name, entries in info.items():
            if shared_name not in name_to_ht:
                continue
            ht = name_to_ht[shared_name]
            mine = tuple(ht.slice_info())
            for load_shared_name, slot_names in entries.items():
                groups = {}
                for slot_name in slot_names:
                    tensor_name = shared_name + fmt.INTRA_SEP + slot_name
                    if not bundle.has_tensor(tensor_name):
                        continue
                    for slice_str in bundle.slice_infos(tensor_name):
                        if not fmt.slices_intersect(fmt.slice_from_string(slice_str), mine):
                            continue
                        g = groups.setdefault(slice_str, {"id": None, "slots": []})
                        b = bundle.block_info(fmt.block_name(tensor_name, slice_str))
                        if slot_name == fmt.ID_SLOT:
                            g["id"] = b
                        else:
                            g["slots"].append((ht.slot_group().slot_by_name(slot_name), b))
                for g in groups.values():
                    if g["id"] is None or not g["slots"]:
                        raise RuntimeError("%s, invalid" % load_shared_name)
                    _load_table_blocks(ht, load_shared_name, g["id"], g["slots"], self._parallel)
        # load_internal.cc:149-175
        for tensor_name, entries in info.items():
            if tensor_name not in self._tensors:
                continue
            target = self._tensors[tensor_name]
            if len(entries) != 1:
                raise RuntimeError("currently only support one tensor")
            for load_name in entries:
                if not bundle.has_tensor(load_name):
                    continue
                b = bundle.block_info(fmt.block_name(load_name, fmt.EMPTY_SLICE))
                if b.dtype != target.dtype:
                    raise RuntimeError("dtype not match")
                if b.shape != list(target.shape):
                    raise RuntimeError("shape not match")
                with torch.no_grad():
                    target.copy_(b.read_tensor())
        if torch.cuda.is_available():
            _lib.raise_device_errors()   # rows the inserts had to skip would be missing silently
