"""Per-head thresholds for the range search.

The reference names two sample-based rules and leaves both unwritten
(cache/threshold_finder.py:1-14: ``sample_max`` and ``sample_mean_topk`` raise
NotImplementedError) and picks thresholds in its tests as the k-th largest exact score
(tests/test_cpu_pipeline.py:53-66) or the midpoint between two neighbouring scores
(tests/test_customized.py:77-83).  All rules here take

    samples : (H_kv, S, D)  keys (a sample, or all of them)
    query   : (H_q, D) or (1, H_q, 1, D)

and return a ``(H_q,)`` fp32 tensor on the samples' device.  Scores are computed in fp32.
Threshold selection happens once per decode step on small inputs (or offline); it is not
part of the search kernels.
"""
from __future__ import annotations

from typing import Optional

import torch


def _scores(samples: torch.Tensor, query: torch.Tensor,
            q_head_to_kv: Optional[torch.Tensor] = None) -> torch.Tensor:
    if query.ndim == 4:
        query = query.squeeze(0).squeeze(-2)
    h_kv, h_q = samples.shape[0], query.shape[0]
    if q_head_to_kv is None:
        if h_q % h_kv:
            raise ValueError(f"H_q={h_q} must be a multiple of H_kv={h_kv}")
        q = query.reshape(h_kv, h_q // h_kv, -1).float().to(samples.device)
        return torch.einsum("hsd,hgd->hgs", samples.float(), q).reshape(h_q, -1)
    s = samples.float().index_select(0, q_head_to_kv.to(samples.device).long())
    return torch.einsum("hsd,hd->hs", s, query.float().to(samples.device))


def sample_max(samples, query, q_head_to_kv=None) -> torch.Tensor:
    """Threshold = the largest score among the samples."""
    return _scores(samples, query, q_head_to_kv).max(dim=-1).values


def sample_mean_topk(samples, query, k, q_head_to_kv=None) -> torch.Tensor:
    """Threshold = mean of the k largest sample scores."""
    s = _scores(samples, query, q_head_to_kv)
    k = max(1, min(int(k), s.shape[-1]))
    return s.topk(k, dim=-1).values.mean(dim=-1)


def exact_topk(keys, query, k, q_head_to_kv=None, midpoint: bool = True) -> torch.Tensor:
    """Threshold that selects exactly the k best-scoring keys of each head: the k-th
    largest score or, with ``midpoint``, halfway between the k-th and the (k+1)-th so that
    no score coincides with the threshold."""
    s = _scores(keys, query, q_head_to_kv)
    n = s.shape[-1]
    k = max(1, min(int(k), n))
    top = s.topk(min(k + 1, n), dim=-1).values
    if not midpoint or k == n:
        return top[:, k - 1].contiguous()
    return ((top[:, k - 1].double() + top[:, k].double()) * 0.5).float()


THRESHOLD_METHODS = {
    "sample_max": sample_max,
    "sample_mean_topk": sample_mean_topk,
    "exact_topk": exact_topk,
}
