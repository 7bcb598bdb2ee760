"""ctypes loader for ``librecis_hip.so`` (the C-ABI HIP library).

The product path never falls back to a CPU implementation: if the library is
missing it is built once (hipcc cross-compiles without a GPU); if that fails,
or a call returns an error, a ``RuntimeError`` is raised.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "librecis_hip.so")
HEADER_PATH = os.path.join(_HERE, "..", "include", "recis_hip.h")

_lib = None

ABI_VERSION = 2  # RECIS_HIP_ABI_VERSION of include/recis_hip.h
F32, BF16, F16 = 0, 1, 2
F64 = 3   # rows and gradients of block_apply_adamw only
SUM, MEAN, TILE, MAX = 0, 1, 2, 3
FLAG_REV_UNIQUE = 1

DEVERR_INDEX_RANGE = 1
DEVERR_OFFSETS = 2
DEVERR_TABLE_FULL = 4
DEVERR_PLAN_OVERFLOW = 8

_DTYPES = {torch.float32: F32, torch.bfloat16: BF16, torch.float16: F16}
MODES = {"sum": SUM, "mean": MEAN, "tile": TILE, "max": MAX}


class RecisHipError(RuntimeError):
    pass


# A ScalarType that a method of a torch.classes.recis object returns crosses the binding as its
# c10::ScalarType number (tests/test_torch_library.py checks the table against the library).
SCALAR_TYPE_DTYPES = {0: torch.uint8, 1: torch.int8, 2: torch.int16, 3: torch.int32, 4: torch.int64,
                      5: torch.float16, 6: torch.float32, 7: torch.float64, 11: torch.bool, 15: torch.bfloat16}


def as_dtype(code):
    """torch.dtype of a ScalarType number (a torch.dtype passes through)."""
    return code if isinstance(code, torch.dtype) else SCALAR_TYPE_DTYPES[int(code)]


def lib():
    """The loaded library (built first if no binary is present)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            from . import build as _build

            _build.build(verbose=False)
        _lib = ctypes.CDLL(LIB_PATH)
        _lib.recis_hip_last_error.restype = ctypes.c_char_p
        abi = _lib.recis_hip_abi_version()
        if abi != ABI_VERSION:
            raise RecisHipError("librecis_hip.so ABI %d, expected %d: rebuild with "
                                "python -m recis_amd.build" % (abi, ABI_VERSION))
    return _lib


def check(rc):
    if rc != 0:
        raise RecisHipError("librecis_hip: %s (code %d)" %
                            (lib().recis_hip_last_error().decode(), rc))


def dtype_code(dt):
    try:
        return _DTYPES[dt]
    except KeyError:
        raise TypeError("unsupported row dtype %s (float32, bfloat16, float16)" % dt)


def ptr(t):
    """Device pointer of a tensor as a ctypes void pointer (None -> NULL)."""
    if t is None:
        return ctypes.c_void_p(0)
    return ctypes.c_void_p(t.data_ptr())


def i64(x):
    return ctypes.c_int64(int(x))


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_ptr(device=None):
    """The current HIP stream of ``device`` as a void pointer (called once or more per op: the
    raw getter is several times cheaper than building a ``torch.cuda.Stream`` object)."""
    if _raw_stream is not None:
        if device is None:
            idx = torch.cuda.current_device()
        else:
            idx = device.index if isinstance(device, torch.device) else torch.device(device).index
            if idx is None:
                idx = torch.cuda.current_device()
        return ctypes.c_void_p(_raw_stream(idx))
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def require_cuda(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RecisHipError("expected a GPU tensor, got one on %s" % t.device)


def poll_device_errors():
    """Synchronises the device and returns (and clears) the soft-error bits."""
    bits = ctypes.c_int(0)
    check(lib().recis_hip_poll_device_errors(ctypes.byref(bits)))
    return bits.value


DEVERR_TEXT = ((DEVERR_INDEX_RANGE, "an index outside the rows / blocks the caller passed"),
               (DEVERR_OFFSETS, "offsets not monotone or out of range"),
               (DEVERR_TABLE_FULL, "the id map found no free slot"),
               (DEVERR_PLAN_OVERFLOW, "batch plan: too many distinct ids in one hash bucket"))


def describe_device_errors(bits):
    return "; ".join(t for b, t in DEVERR_TEXT if bits & b) + " (bits %d)" % bits


def raise_device_errors(extra_bits=0):
    """Waits for the device, clears the soft-error word and raises if any kernel since the last
    poll skipped a faulty access (bad row index, full id map, ...). For host code that waits for
    the device anyway: table statistics, checkpoint save / load."""
    bits = poll_device_errors() | extra_bits
    if bits:
        raise RecisHipError("device-side errors in earlier kernels: " + describe_device_errors(bits))
