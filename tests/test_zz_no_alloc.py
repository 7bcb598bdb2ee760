"""recis_unique_plan_noalloc (the entry point for callers that cannot allocate) against
recis_unique_plan, through the C ABI: bit for bit on everything recis_unique_plan specifies (unique
ids, inverse, row_start, counts, hot-item set), and the occurrence lists equal as sets per id with
pos consistent; two calls in a row on the device's one built-in scratch array, the second with a
smaller input; then the size limit."""
import ctypes

import numpy as np
import pytest
import torch

from recis_amd import _lib
from recis_amd._lib import check, i64, ptr, stream_ptr

pytestmark = pytest.mark.gpu

HOT_LEN, HOT_CHUNK = 64, 2048
MAX_IDS = 262144


def _run(entry, ids):
    n = ids.numel()
    dev = ids.device
    hot_cap = n // HOT_LEN + n // HOT_CHUNK + 2
    out = {
        "unique": torch.full((n,), -77, dtype=torch.int64, device=dev),
        "inverse": torch.full((n,), -77, dtype=torch.int32, device=dev),
        "row_start": torch.full((n + 1,), -77, dtype=torch.int32, device=dev),
        "occ": torch.full((n,), -77, dtype=torch.int32, device=dev),
        "pos": torch.full((n,), -77, dtype=torch.int32, device=dev),
        "hot": torch.full((2 * hot_cap,), -77, dtype=torch.int32, device=dev),
        "counts": torch.full((2,), -77, dtype=torch.int64, device=dev),
    }
    lib = _lib.lib()
    args = [ptr(ids), i64(n), ptr(out["unique"]), ptr(out["inverse"]), ptr(out["row_start"]), ptr(out["occ"]),
            ptr(out["pos"]), ptr(out["hot"]), i64(hot_cap), ptr(out["counts"])]
    if entry == "noalloc":
        rc = lib.recis_unique_plan_noalloc(*args, stream_ptr(dev))
    else:
        count = ctypes.c_int64(0)
        rc = lib.recis_unique_plan(*args, ctypes.byref(count), 0, stream_ptr(dev))
    check(rc)
    torch.cuda.synchronize()
    return {k: v.cpu().numpy() for k, v in out.items()}


def _same(a, b, ids):
    n = len(ids)
    U, n_hot = int(a["counts"][0]), int(a["counts"][1])
    assert (U, n_hot) == (int(b["counts"][0]), int(b["counts"][1]))
    assert U == len(np.unique(ids))
    np.testing.assert_array_equal(a["unique"][:U], b["unique"][:U])
    np.testing.assert_array_equal(a["inverse"], b["inverse"])
    np.testing.assert_array_equal(a["row_start"], b["row_start"])
    np.testing.assert_array_equal(a["unique"][:U][a["inverse"]], ids)
    for r in (a, b):   # list entries may come in any order inside one id's list
        np.testing.assert_array_equal(r["occ"][r["pos"]], np.arange(n))
        np.testing.assert_array_equal(np.repeat(np.arange(U), np.diff(r["row_start"][: U + 1])), r["inverse"][r["occ"]])
    items = lambda r: sorted(map(tuple, r["hot"][: 2 * n_hot].reshape(-1, 2)))
    assert items(a) == items(b)


def _ids(rng, n, hot_frac):
    hot = rng.integers(0, 37, size=n)
    cold = rng.integers(-(1 << 60), 1 << 60, size=n)
    ids = np.where(rng.random(n) < hot_frac, hot, cold)
    if n > 3:
        ids[2] = -1
    return ids


def test_noalloc_plan_matches_the_allocating_plan_twice_in_a_row(rng):
    first = _ids(rng, 200_000, 0.5)
    second = _ids(rng, 33_333, 0.2)      # smaller: leaves most of the scratch holding the first call's data
    for ids in (first, second, np.zeros(0, np.int64), _ids(rng, MAX_IDS, 0.9)):
        t = torch.from_numpy(ids).cuda()
        got = _run("noalloc", t)
        ref = _run("plan", t)
        _same(got, ref, ids)
    assert _lib.poll_device_errors() == 0


def test_noalloc_plan_rejects_what_does_not_fit():
    n = MAX_IDS + 1
    t = torch.zeros(n, dtype=torch.int64, device="cuda")
    with pytest.raises(_lib.RecisHipError, match="at most"):
        _run("noalloc", t)


def test_noalloc_plan_allocates_nothing(rng):
    """Free device memory as the runtime reports it (hipMemGetInfo) is the same before and after a call:
    the outputs are the caller's, the scratch is the library's static array. (The first call on a device
    looks the array's address up; the one measured is a later one.)"""
    ids = torch.from_numpy(_ids(rng, 100_000, 0.3)).cuda()
    n, dev = ids.numel(), ids.device
    hot_cap = n // 64 + n // 2048 + 2
    i32 = lambda k: torch.empty(k, dtype=torch.int32, device=dev)
    outs = (torch.empty(n, dtype=torch.int64, device=dev), i32(n), i32(n + 1), i32(n), i32(n), i32(2 * hot_cap),
            torch.empty(2, dtype=torch.int64, device=dev))
    lib = _lib.lib()

    def call():
        check(lib.recis_unique_plan_noalloc(ptr(ids), i64(n), ptr(outs[0]), ptr(outs[1]), ptr(outs[2]), ptr(outs[3]),
                                            ptr(outs[4]), ptr(outs[5]), i64(hot_cap), ptr(outs[6]), stream_ptr(dev)))
        torch.cuda.synchronize()

    call()
    free_before = torch.cuda.mem_get_info()[0]
    for _ in range(3):
        call()
    assert torch.cuda.mem_get_info()[0] == free_before
    assert int(outs[6][0]) == len(np.unique(ids.cpu().numpy()))
