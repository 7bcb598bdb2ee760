"""Test infrastructure: runs the reference's own CPU operators, compiled from the reference
tree into ``oracle/_ref/ref_ops`` (see ``ref_build.sh`` / ``ref_ops_driver.cc``), on numpy
inputs. Used by the tests to check the oracle against the real code; never by the product."""
import os
import struct
import subprocess
import tempfile

import numpy as np

BINARY = os.path.join(os.path.dirname(os.path.abspath(__file__)), "_ref", "ref_ops")
_CODES = {np.dtype(np.float32): 0, np.dtype(np.float64): 1, np.dtype(np.int64): 2, np.dtype(np.int32): 3,
          np.dtype(np.bool_): 4, np.dtype(np.int8): 5, np.dtype(np.float16): 6}
_TYPES = {v: k for k, v in _CODES.items()}


def available():
    return os.path.exists(BINARY)


def _write(path, arrays):
    with open(path, "wb") as f:
        f.write(struct.pack("<q", len(arrays)))
        for a in arrays:
            a = np.ascontiguousarray(a)
            f.write(struct.pack("<ii", _CODES[a.dtype], a.ndim))
            f.write(struct.pack("<%dq" % a.ndim, *a.shape))
            f.write(a.tobytes())


def _read(path):
    out = []
    with open(path, "rb") as f:
        (n,) = struct.unpack("<q", f.read(8))
        for _ in range(n):
            code, ndim = struct.unpack("<ii", f.read(8))
            dims = struct.unpack("<%dq" % ndim, f.read(8 * ndim)) if ndim else ()
            dt = _TYPES[code]
            count = int(np.prod(dims)) if ndim else 1
            out.append(np.frombuffer(f.read(count * dt.itemsize), dtype=dt).reshape(dims).copy())
    return out


def run(op, arrays, threads=1, timeout=300):
    """Outputs (list of numpy arrays) of reference operator ``op`` on ``arrays``."""
    with tempfile.TemporaryDirectory() as d:
        fin, fout = os.path.join(d, "in.bin"), os.path.join(d, "out.bin")
        _write(fin, arrays)
        env = dict(os.environ, OMP_NUM_THREADS=str(threads))
        r = subprocess.run([BINARY, op, fin, fout], capture_output=True, text=True, env=env, timeout=timeout)
        if r.returncode != 0:
            raise RuntimeError("ref_ops %s failed (%d): %s" % (op, r.returncode, r.stderr[-2000:]))
        return _read(fout)
