"""Shared test helpers: seeded inputs in the style of the reference's tests and the
comparison rule for selected-key sets."""
from __future__ import annotations

import numpy as np
import torch


def normalized_keys(h: int, n: int, d: int, seed: int) -> np.ndarray:
    """tests/test_cpp_kernels.py:20-23 of the reference: unit-norm Gaussian keys (H, N, D)."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((1, h, n, d), generator=g, dtype=torch.float32)
    return (x / x.norm(dim=-1, keepdim=True).clamp_min(1e-12))[0].numpy()


def random_query(h: int, d: int, seed: int, normalize: bool = True) -> np.ndarray:
    g = torch.Generator().manual_seed(seed)
    q = torch.randn((h, d), generator=g, dtype=torch.float32)
    if normalize:
        q = q / q.norm(dim=-1, keepdim=True).clamp_min(1e-12)
    return q.numpy()


def midpoint_threshold(scores: np.ndarray, keep: int) -> np.ndarray:
    """Per row: the midpoint between the keep-th and (keep+1)-th largest score, so that no
    score sits at the threshold (the reference's tests/test_customized.py:77-83)."""
    s = np.sort(scores.astype(np.float64), axis=1)[:, ::-1]
    keep = min(max(keep, 1), s.shape[1] - 1)
    return ((s[:, keep - 1] + s[:, keep]) * 0.5).astype(np.float32)


def assert_same_selection(got_mask: np.ndarray, scores: np.ndarray, th: np.ndarray,
                          rel_band: float = 1e-5) -> int:
    """The selected set must equal {i : s_i >= th}, except for keys whose fp32 score lies
    within rel_band * |th| of the threshold.  Returns the number of keys in the band."""
    want = scores >= th[:, None]
    band = np.abs(scores - th[:, None]) <= rel_band * np.abs(th[:, None])
    bad = (got_mask != want) & ~band
    assert not bad.any(), f"{int(bad.sum())} keys differ outside the threshold band"
    return int(band.sum())


def band_free_heads(scores: np.ndarray, th: np.ndarray, valid=None, rel_band: float = 1e-5) -> np.ndarray:
    """Heads none of whose (valid) keys scores within rel_band * |th| of the threshold: only
    for those is the selected set, and with it the attention output, fixed by the inputs."""
    band = np.abs(scores - th[:, None]) <= rel_band * np.abs(th[:, None])
    if valid is not None:
        band &= valid
    return ~band.any(axis=1)


def clustered_keys(h: int, n: int, d: int, seed: int, clusters: int = 16,
                   spread: float = 0.15) -> np.ndarray:
    """Keys around `clusters` well-separated centres, so that ball bounds really prune."""
    g = torch.Generator().manual_seed(seed)
    cen = torch.randn((h, clusters, d), generator=g)
    cen = cen / cen.norm(dim=-1, keepdim=True)
    which = torch.randint(0, clusters, (h, n), generator=g)
    x = torch.gather(cen, 1, which[..., None].expand(h, n, d))
    x = x + spread * torch.randn((h, n, d), generator=g) / d ** 0.5
    return x.numpy()


def bf16_round(a: np.ndarray) -> np.ndarray:
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(torch.bfloat16).float().numpy()


def rel_err(got: np.ndarray, ref: np.ndarray) -> float:
    """max |got - ref| over max |ref|, per row, worst row."""
    den = np.maximum(np.abs(ref).max(axis=-1), 1e-30)
    return float((np.abs(got - ref).max(axis=-1) / den).max())
