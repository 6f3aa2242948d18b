"""Seeded synthetic inputs of the five benchmark configurations (shapes and distributions as the
baseline document defines them), shared by the parity tests and bench.py.  Everything is generated
on the CPU from torch.manual_seed-style generators so that the CPU oracle and the GPU see the same
bits; only the 8 GiB upstream gradient of the long-context dense case is generated on the device.
"""
import torch


def dense_inputs(B, T, H, W, seed, layernorm=False, with_v=False):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, T, H, W, generator=g)
    k = torch.randn(B, T, H, W, generator=g)
    v = torch.randn(B, T, H, W, generator=g) if with_v else None
    if layernorm:  # unit variance per token and head
        q = torch.nn.functional.layer_norm(q, (W,))
        k = torch.nn.functional.layer_norm(k, (W,))
    return q, k, v


def uniform_degree_graph(T, max_deg, seed):
    """Every dst gets a uniform-random 1..max_deg distinct src tokens; rows shuffled.  [E,2] int64."""
    g = torch.Generator().manual_seed(seed)
    deg = torch.randint(1, max_deg + 1, (T,), generator=g)
    rows = []
    for d in range(T):
        src = torch.randperm(T, generator=g)[: int(deg[d])]
        rows.append(torch.stack((torch.full_like(src, d), src), 1))
    co = torch.cat(rows, 0)
    return co[torch.randperm(co.shape[0], generator=g)]


def powerlaw_graph(T, seed, alpha=2.0, scale=3.2, max_deg=2048, self_loops=True):
    """Per-dst degree = clip(round(scale * Zipf(alpha)), 1, max_deg) (mean about 16 for the
    defaults), src uniform without replacement, plus [i,i] self loops, rows shuffled.  [E,2] int64."""
    import numpy as np
    rng = np.random.default_rng(seed)
    deg = np.clip(np.rint(scale * rng.zipf(alpha, size=T)), 1, min(max_deg, T)).astype(np.int64)
    dst = np.repeat(np.arange(T, dtype=np.int64), deg)
    src = np.empty_like(dst)
    pos = 0
    for d in range(T):
        n = int(deg[d])
        if n * 4 < T:
            # rejection sampling of n distinct values: cheap for short rows
            s = rng.choice(T, size=n, replace=False) if n > 64 else _distinct(rng, T, n)
        else:
            s = rng.permutation(T)[:n]
        src[pos:pos + n] = s
        pos += n
    if self_loops:
        loops = np.arange(T, dtype=np.int64)
        dst = np.concatenate((dst, loops))
        src = np.concatenate((src, loops))
    perm = rng.permutation(dst.shape[0])
    return torch.from_numpy(np.stack((dst[perm], src[perm]), 1))


def _distinct(rng, T, n):
    import numpy as np
    s = np.unique(rng.integers(0, T, size=n))
    while s.shape[0] < n:
        s = np.unique(np.concatenate((s, rng.integers(0, T, size=n - s.shape[0]))))
    return rng.permutation(s)


def sparse_inputs(B, T, H, W, seed, n=4):
    g = torch.Generator().manual_seed(seed)
    return [torch.randn(B, T, H, W, generator=g) for _ in range(n)]
