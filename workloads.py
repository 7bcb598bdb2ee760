"""Seeded synthetic inputs for the BASELINE configurations.

Used by ``bench.py`` and the tests; every generator is deterministic in its
seed (numpy ``PCG64``) and returns torch tensors on the requested device.
"""
import numpy as np
import torch


def _rng(seed):
    return np.random.Generator(np.random.PCG64(seed))


def bounded_zipf(rng, n, alpha, num_keys):
    """n ranks in [0, num_keys) with P(rank r) proportional to (r+1)^-alpha.

    Inverse-CDF sampling on the exact cumulative table (numpy's ``zipf`` is
    unbounded and only defined for alpha > 1)."""
    p = np.arange(1, num_keys + 1, dtype=np.float64) ** (-alpha)
    cdf = np.cumsum(p)
    cdf /= cdf[-1]
    return np.minimum(np.searchsorted(cdf, rng.random(n), side="left"), num_keys - 1).astype(np.int64)


def splitmix64(x):
    """Bijective 64-bit mix (numpy uint64 arrays), used to turn ranks into random keys."""
    x = (x.astype(np.uint64) + np.uint64(0x9E3779B97F4A7C15))
    x = (x ^ (x >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
    x = (x ^ (x >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
    return x ^ (x >> np.uint64(31))


def config2(device="cuda", seed=1, features=32, batch=16384, dim=64, mean_len=30, max_len=200):
    """Standalone ragged segment_reduce on pre-materialised rows (BASELINE config 2)."""
    rng = _rng(seed)
    S = features * batch
    lens = np.clip(rng.poisson(mean_len, size=S), 1, max_len).astype(np.int64)
    off = np.zeros(S + 1, np.int64)
    np.cumsum(lens, out=off[1:])
    N = int(off[-1])
    g = torch.Generator(device=device).manual_seed(seed)
    values = torch.randn((N, dim), dtype=torch.float32, device=device, generator=g)
    grad = torch.randn((S, dim), dtype=torch.float32, device=device, generator=g)
    return {
        "values": values,
        "grad": grad,
        "offsets": torch.from_numpy(off.astype(np.int32)).to(device),
        "reverse_indices": None,
        "num_segments": S,
        "num_ids": N,
        "dim": dim,
    }


def config1_step(step, seed=0, batch=4096, num_keys=1_000_000, alpha=1.05, max_len=20, dim=16, _cache={}):
    """One batch of BASELINE config 1 as numpy arrays: (ids int64 [N], offsets int64 [batch+1],
    upstream gradient float32 [batch, dim]). Deterministic in (seed, step)."""
    key = (num_keys, alpha)
    if key not in _cache:
        p = np.arange(1, num_keys + 1, dtype=np.float64) ** (-alpha)
        cdf = np.cumsum(p)
        _cache[key] = cdf / cdf[-1]
    rng = _rng([seed, step])
    lens = rng.integers(1, max_len + 1, size=batch)
    off = np.zeros(batch + 1, np.int64)
    np.cumsum(lens, out=off[1:])
    n = int(off[-1])
    ids = np.minimum(np.searchsorted(_cache[key], rng.random(n), side="left"), num_keys - 1).astype(np.int64)
    grad = rng.standard_normal((batch, dim)).astype(np.float32)
    return ids, off, grad


def seeded_block(seed, block_index, block_size, dim, std=0.01):
    """Initial rows of one storage block, identical on the CPU and the GPU side."""
    return (std * _rng([seed, 7919, block_index]).standard_normal((block_size, dim))).astype(np.float32)


def config4(device="cuda", seed=4, batch=65536, n_sparse=26, n_dense=13, n_boundaries=64, mod=1_000_000):
    """Click-through-style merged table (BASELINE config 4): 26 int64 id fields with log-uniform
    cardinalities in 10..1e7, 13 lognormal(0, 2) dense fields bucketized against 64 sorted
    boundaries and taken mod 1e6; one id per field per sample."""
    rng = _rng(seed)
    cards = np.floor(10 ** rng.uniform(1, 7, size=n_sparse)).astype(np.int64)
    sparse = [torch.from_numpy(rng.integers(0, c, size=batch, dtype=np.int64)).to(device) for c in cards]
    dense = [torch.from_numpy(rng.lognormal(0.0, 2.0, size=batch).astype(np.float32)).to(device)
             for _ in range(n_dense)]
    # boundaries: 64 quantile-like points of lognormal(0, 2)
    q = (np.arange(1, n_boundaries + 1) - 0.5) / n_boundaries
    from scipy.special import erfinv
    z = np.sqrt(2.0) * erfinv(2 * q - 1)
    bnd = torch.from_numpy(np.exp(2.0 * z).astype(np.float32)).to(device)
    return {"sparse": sparse, "dense": dense, "boundaries": [bnd] * n_dense, "mod": mod,
            "cardinalities": cards, "batch": batch, "num_ids": batch * (n_sparse + n_dense)}
