"""Writes tests/golden/hash_vectors.json from the reference's own CPU hash code.

Needs oracle/_ref/libref_hash.so (built by oracle/ref_build.sh from the reference
tree's third_party/column-io/cc/column-io/dataset/{farmhash,hash_utils}.cc).
The vectors cover every length class of FarmHash64 (0, 1-3, 4-7, 8-16, 17-32,
33-64, >64 with one and several 64-byte rounds) and of MurmurHash64A (tails 0-7).
"""
import ctypes
import json
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))


def main():
    ref = ctypes.CDLL(os.path.join(ROOT, "oracle", "_ref", "libref_hash.so"))
    ref.ref_farm_fingerprint64.restype = ctypes.c_uint64
    ref.ref_murmur64.restype = ctypes.c_uint64
    rng = np.random.default_rng(20240607)
    lengths = list(range(0, 40)) + [47, 48, 63, 64, 65, 66, 96, 127, 128, 129, 191, 192, 193, 255, 256, 257, 300, 1000]
    vectors = []
    for n in lengths:
        b = rng.integers(0, 256, size=n, dtype=np.uint8).tobytes()
        farm = ref.ref_farm_fingerprint64(b, ctypes.c_size_t(n))
        mur = ref.ref_murmur64(b, ctypes.c_size_t(n), ctypes.c_uint64(0))
        vectors.append({"hex": b.hex(), "farm": int(np.int64(np.uint64(farm))),
                        "murmur": int(np.int64(np.uint64(mur)))})
    with open(os.path.join(HERE, "hash_vectors.json"), "w") as f:
        json.dump({"source": "third_party/column-io/cc/column-io/dataset/farmhash.cc (util::Fingerprint64), "
                             "hash_utils.cc (MurMurHash64, seed 0)", "vectors": vectors}, f, indent=0)
    print("wrote", len(vectors), "vectors")


if __name__ == "__main__":
    main()
