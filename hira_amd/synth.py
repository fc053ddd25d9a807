"""Seeded synthetic workloads: the five benchmark configurations of this path.

Keys of one KV head are ``k = mu + s * z`` with ``z ~ N(0, I)``, a fixed per-channel scale
``s ~ LogNormal(0, 0.5)`` and a fixed offset ``mu ~ N(0, 0.3^2 I)``; values are ``N(0, I)``;
a query head is a noisy copy of a random cached key, ``q = k_j + 0.5 N(0, I)``.  Configs 2
and 3 multiply 8 channels per KV head by 20 in keys and queries ("massive activations").
Everything is drawn on the host from ``torch.Generator().manual_seed(...)`` streams, in
fp32, and rounded once to the storage dtype.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

import torch


@dataclass(frozen=True)
class Workload:
    name: str
    cfg: int
    batch: int
    h_q: int
    h_kv: int
    n: int
    d: int
    dtype: torch.dtype
    num_levels: int
    bf: int
    kmeans_iters: int
    select_frac: Tuple[float, float]  # (lo, hi): per-sequence fraction, lo == hi -> fixed
    massive: bool

    @property
    def group(self) -> int:
        return self.h_q // self.h_kv


WORKLOADS = {
    0: Workload("cfg0_single_head_4k_fp32", 0, 1, 1, 1, 4096, 128, torch.float32, 2, 16, 10,
                (0.05, 0.05), False),
    1: Workload("cfg1_llama8b_8k_bf16", 1, 1, 32, 8, 8192, 128, torch.bfloat16, 3, 32, 1,
                (0.02, 0.02), False),
    2: Workload("cfg2_llama8b_32k_bf16_massive", 2, 1, 32, 8, 32768, 128, torch.bfloat16, 3, 32,
                1, (0.01, 0.01), True),
    3: Workload("cfg3_llama8b_32k_bf16_batch16", 3, 16, 32, 8, 32768, 128, torch.bfloat16, 3,
                32, 1, (0.005, 0.05), True),
    4: Workload("cfg4_llama70b_128k_bf16_stream", 4, 1, 64, 8, 131072, 128, torch.bfloat16, 4,
                32, 1, (0.01, 0.01), False),
}

SEED_BASE = 20260000


def _gen(cfg: int, seq: int, kv_head: int, salt: int = 0) -> torch.Generator:
    return torch.Generator().manual_seed(SEED_BASE + 1000 * cfg + 10 * seq + kv_head
                                         + 1_000_000 * salt)


@dataclass
class HeadDist:
    mu: torch.Tensor  # (D,)
    s: torch.Tensor  # (D,)
    massive: Optional[torch.Tensor]  # (8,) channel ids or None


def head_dist(w: Workload, seq: int, kv_head: int) -> HeadDist:
    g = _gen(w.cfg, seq, kv_head, salt=1)
    mu = 0.3 * torch.randn(w.d, generator=g)
    s = torch.exp(0.5 * torch.randn(w.d, generator=g))
    massive = torch.randperm(w.d, generator=g)[:8] if w.massive else None
    return HeadDist(mu, s, massive)


def _boost(x: torch.Tensor, dist: HeadDist) -> torch.Tensor:
    if dist.massive is not None:
        x = x.clone()
        x[..., dist.massive] *= 20.0
    return x


def make_kv(w: Workload, n: Optional[int] = None):
    """keys, values (B, H_kv, n, D) in the workload dtype (rounded once from fp32)."""
    n = w.n if n is None else n
    keys = torch.empty((w.batch, w.h_kv, n, w.d), dtype=torch.float32)
    values = torch.empty_like(keys)
    for b in range(w.batch):
        for h in range(w.h_kv):
            dist = head_dist(w, b, h)
            g = _gen(w.cfg, b, h, salt=2)
            z = torch.randn((n, w.d), generator=g)
            keys[b, h] = _boost(dist.mu + dist.s * z, dist)
            values[b, h] = torch.randn((n, w.d), generator=g)
    return keys.to(w.dtype), values.to(w.dtype)


def make_stream(w: Workload, steps: int):
    """keys, values (B, H_kv, steps, D) appended one per decode step after the prefill: the
    same distribution with a slow drift of the mean, mu_t = mu_0 + 1e-4 t g, g ~ N(0, I)
    fixed per head."""
    keys = torch.empty((w.batch, w.h_kv, steps, w.d), dtype=torch.float32)
    values = torch.empty_like(keys)
    t = torch.arange(steps, dtype=torch.float32)[:, None]
    for b in range(w.batch):
        for h in range(w.h_kv):
            dist = head_dist(w, b, h)
            g = _gen(w.cfg, b, h, salt=3)
            drift = torch.randn(w.d, generator=g)
            z = torch.randn((steps, w.d), generator=g)
            keys[b, h] = _boost(dist.mu + 1e-4 * t * drift + dist.s * z, dist)
            values[b, h] = torch.randn((steps, w.d), generator=g)
    return keys.to(w.dtype), values.to(w.dtype)


def make_queries(w: Workload, keys: torch.Tensor, steps: int, seed: int = 0) -> torch.Tensor:
    """(steps, B, H_q, D) fresh queries: q = k_j + 0.5 N(0, I), j uniform.  The massive
    channels are already scaled in k_j; the noise on them is scaled by 20 as well."""
    b, h_kv, n, d = keys.shape
    g = torch.Generator().manual_seed(SEED_BASE + 1000 * w.cfg + 777 + seed)
    j = torch.randint(0, n, (steps, b, w.h_q), generator=g)
    noise = 0.5 * torch.randn((steps, b, w.h_q, d), generator=g)
    kf = keys.float()
    q = torch.empty((steps, b, w.h_q, d), dtype=torch.float32)
    for bb in range(b):
        for h in range(w.h_q):
            kv = h // w.group
            dist = head_dist(w, bb, kv)
            q[:, bb, h] = kf[bb, kv, j[:, bb, h]] + _boost(noise[:, bb, h], dist)
    return q.to(w.dtype)


def load_capture(path: str, w: Workload, steps: int, seed: int = 0):
    """Keys and queries captured from a model, in the file format of the reference's sampler
    (benchmark_area/kv_sampling/collect_kv_data.py:393-397; read by
    benchmark_area/utils/data_loader.py:5-22): an ``.npz`` with ``keys`` (N_k, D) and
    ``queries`` (N_q, D) fp32, heads flattened into the rows.  The pool of keys is dealt to the
    workload's B x H_kv trees (as many keys per tree as the pool allows, at most ``w.n``), the
    queries are drawn from the pool of queries with replacement; values stay synthetic
    (the sampler keeps none).  Returns (workload with the key count in use, keys, values,
    queries (steps, B, H_q, D))."""
    import dataclasses

    import numpy as np

    with np.load(path) as f:  # allow_pickle stays False
        pool_k = torch.from_numpy(np.ascontiguousarray(f["keys"], dtype=np.float32))
        pool_q = torch.from_numpy(np.ascontiguousarray(f["queries"], dtype=np.float32))
    if pool_k.ndim != 2 or pool_q.ndim != 2 or pool_k.shape[1] != w.d or pool_q.shape[1] != w.d:
        raise ValueError(f"{path}: keys {tuple(pool_k.shape)} / queries {tuple(pool_q.shape)}: "
                         f"expected (N, {w.d}) each")
    trees = w.batch * w.h_kv
    n = min(w.n, pool_k.shape[0] // trees)
    if n < w.bf:
        raise ValueError(f"{path}: {pool_k.shape[0]} keys are too few for {trees} trees")
    g = torch.Generator().manual_seed(SEED_BASE + 1000 * w.cfg + 999 + seed)
    order = torch.randperm(pool_k.shape[0], generator=g)[: trees * n]
    keys = pool_k[order].reshape(w.batch, w.h_kv, n, w.d)
    values = torch.randn((w.batch, w.h_kv, n, w.d), generator=g)
    pick = torch.randint(0, pool_q.shape[0], (steps, w.batch, w.h_q), generator=g)
    queries = pool_q[pick]
    w2 = dataclasses.replace(w, name=w.name + "+capture", n=n, massive=False)
    return w2, keys.to(w.dtype), values.to(w.dtype), queries.to(w.dtype)


def select_fractions(w: Workload) -> torch.Tensor:
    """(B,) fraction of keys each sequence's threshold targets."""
    lo, hi = w.select_frac
    if lo == hi:
        return torch.full((w.batch,), lo)
    g = torch.Generator().manual_seed(SEED_BASE + 1000 * w.cfg + 555)
    return lo + (hi - lo) * torch.rand(w.batch, generator=g)
