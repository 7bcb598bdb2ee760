"""Seeded synthetic inputs for the benchmark configurations.

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
    """Standalone ragged segment_reduce on pre-materialised rows (benchmark config 2)."""
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
    """One batch of benchmark config 1 as numpy arrays: (ids int64 [N], offsets int64 [batch+1],
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


def config4(device="cuda", seed=4, batch=65536, n_sparse=26, n_dense=13, n_boundaries=64, mod=1_000_000,
            data_seed=None):
    """Click-through-style merged table (benchmark config 4): 26 int64 id fields with log-uniform
    cardinalities in 10..1e7, 13 lognormal(0, 2) dense fields bucketized against 64 sorted
    boundaries and taken mod 1e6; one id per field per sample. ``data_seed`` draws another batch
    of the same fields (same cardinalities and boundaries)."""
    rng = _rng(seed)
    cards = np.floor(10 ** rng.uniform(1, 7, size=n_sparse)).astype(np.int64)
    if data_seed is not None:
        rng = np.random.Generator(np.random.PCG64([seed, data_seed]))
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


# ---------------------------------------------------------------- GPU-side helpers (config 3 / 5)
_M64 = (1 << 64) - 1


def _lsr(x, k):
    """Logical right shift of int64 tensors (torch shifts int64 arithmetically)."""
    return torch.bitwise_and(torch.bitwise_right_shift(x, k), (1 << (64 - k)) - 1)


def _i64(v):
    v &= _M64
    return v - (1 << 64) if v >= (1 << 63) else v


def splitmix64_torch(x):
    """The same bijective mix as ``splitmix64`` on int64 tensors (wrapping arithmetic)."""
    x = x + _i64(0x9E3779B97F4A7C15)
    x = torch.bitwise_xor(x, _lsr(x, 30)) * _i64(0xBF58476D1CE4E5B9)
    x = torch.bitwise_xor(x, _lsr(x, 27)) * _i64(0x94D049BB133111EB)
    return torch.bitwise_xor(x, _lsr(x, 31))


def zipf_cdf_torch(num_keys, alpha, device="cuda"):
    """Cumulative table of the bounded Zipf(alpha) law over ranks 1..num_keys (float64)."""
    cdf = torch.arange(1, num_keys + 1, dtype=torch.float64, device=device).pow_(-alpha).cumsum_(0)
    return cdf.div_(cdf[-1].clone())


def zipf_ranks_torch(cdf, n, generator):
    u = torch.rand(n, dtype=torch.float64, device=cdf.device, generator=generator)
    return torch.searchsorted(cdf, u).clamp_(max=cdf.numel() - 1)


class Config3Lookups:
    """benchmark config 3 lookups: step k draws `ids_per_step` keys, Zipf(alpha) over the `resident`
    pre-populated keys (key of rank r = splitmix64(r)), with a fraction `new_frac` of the positions
    replaced by keys never seen before: ranks resident + k * n_new + arange(n_new), beyond the
    resident set and distinct for every step. Deterministic in (seed, k) whatever the order of the
    calls."""

    def __init__(self, resident, ids_per_step=2_000_000, alpha=1.1, new_frac=0.1, seed=3, device="cuda"):
        self.resident, self.n, self.seed, self.device = resident, ids_per_step, seed, device
        self.n_new = int(ids_per_step * new_frac)
        self.cdf = zipf_cdf_torch(resident, alpha, device)

    def batch(self, k):
        g = torch.Generator(device=self.device).manual_seed(self.seed * 1_000_003 + k)
        ranks = zipf_ranks_torch(self.cdf, self.n, g)
        pos = torch.randperm(self.n, device=self.device, generator=g)[: self.n_new]
        ranks[pos] = self.resident + k * self.n_new + torch.arange(self.n_new, device=self.device)
        return splitmix64_torch(ranks)


def config3_batches(n_batches, resident, ids_per_step=2_000_000, alpha=1.1, new_frac=0.1, seed=3,
                    device="cuda"):
    """The lookups of the first `n_batches` steps of benchmark config 3 (see Config3Lookups)."""
    gen = Config3Lookups(resident, ids_per_step, alpha, new_frac, seed, device)
    return [gen.batch(k) for k in range(n_batches)]


def config5(device="cuda", seed=5, batch=2048, n_fields=4, num_keys=50_000_000, alpha=1.2, mean_len=200,
            max_len=1000):
    """Long behaviour sequences (benchmark config 5): per field `batch` sequences with lognormal
    lengths (sigma 1, mean `mean_len`, clipped to [1, max_len]) of Zipf(alpha) ids over `num_keys`
    keys. Returns per-field values / int32 offsets and the per-field padded length (= longest
    sequence of that field)."""
    rng = _rng(seed)
    g = torch.Generator(device=device).manual_seed(seed)
    cdf = zipf_cdf_torch(num_keys, alpha, device)
    mu = np.log(mean_len) - 0.5
    fields = []
    for f in range(n_fields):
        lens = np.clip(np.round(rng.lognormal(mu, 1.0, size=batch)), 1, max_len).astype(np.int64)
        off = np.zeros(batch + 1, np.int64)
        np.cumsum(lens, out=off[1:])
        ranks = zipf_ranks_torch(cdf, int(off[-1]), g)
        fields.append({"values": _lsr(splitmix64_torch(ranks + f * num_keys), 12),  # 52 id bits
                       "offsets": torch.from_numpy(off.astype(np.int32)).to(device),
                       "pad_len": int(lens.max()), "num_ids": int(off[-1])})
    del cdf
    return {"fields": fields, "batch": batch, "num_ids": sum(f["num_ids"] for f in fields)}
