"""Per-head thresholds for the range search.

The reference names two sample-based rules and leaves both unwritten
(cache/threshold_finder.py:1-14: ``sample_max`` and ``sample_mean_topk`` raise
NotImplementedError) and picks thresholds in its tests as the k-th largest exact score
(tests/test_cpu_pipeline.py:53-66) or the midpoint between two neighbouring scores
(tests/test_customized.py:77-83).  All rules here take

    samples : (H_kv, S, D)  keys (a sample, or all of them)
    query   : (H_q, D) or (1, H_q, 1, D)

and return a ``(H_q,)`` fp32 tensor on the samples' device.  Scores are computed in fp32.

``sample_max`` and ``sample_mean_topk`` on device tensors are one launch of the library's
``hira_threshold`` kernel (it can sit on the decode stream right ahead of the search);
on host tensors they are the same rule in torch ops, for offline use.  ``exact_topk`` scans
every key: a test and benchmark utility, torch ops on either device.
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


MAX_DEVICE_SAMPLES = 4096  # per tree, in one hira_threshold launch


def device_thresholds(samples: torch.Tensor, query: torch.Tensor, method: str, k: int = 1,
                      q_head_to_kv: Optional[torch.Tensor] = None,
                      out: Optional[torch.Tensor] = None, stream: Optional[int] = None) -> torch.Tensor:
    """One ``hira_threshold`` launch: samples (T, S, D) and query (H_q, D) device tensors of the
    same dtype (fp32 or bf16); heads map to trees as in the searcher (default: head h belongs
    to tree h // (H_q / T))."""
    import ctypes as C

    from hira_amd import _lib

    if query.ndim == 4:
        query = query.reshape(-1, query.shape[-1])
    if samples.ndim != 3 or query.ndim != 2 or samples.shape[-1] != query.shape[-1]:
        raise ValueError(f"samples {tuple(samples.shape)} / query {tuple(query.shape)}: expected "
                         "(T, S, D) and (H_q, D)")
    if samples.dtype not in (torch.float32, torch.bfloat16):
        raise ValueError(f"samples dtype {samples.dtype}: fp32 or bf16")
    t, n_s, d = samples.shape
    h_q = query.shape[0]
    if n_s > MAX_DEVICE_SAMPLES:
        raise ValueError(f"{n_s} samples per tree: at most {MAX_DEVICE_SAMPLES}")
    samples = samples.contiguous()
    query = query.to(device=samples.device, dtype=samples.dtype).contiguous()
    keep = None
    if q_head_to_kv is None:
        if h_q % t:
            raise ValueError(f"H_q={h_q} must be a multiple of the {t} trees")
        qs = _lib.HiraQuery(h_q, query.data_ptr(), None, None, None, None, h_q // t, h_q // t)
    else:
        m = q_head_to_kv.to("cpu", torch.int64).reshape(-1)
        if m.numel() != h_q or int(m.min()) < 0 or int(m.max()) >= t:
            raise ValueError("q_head_to_kv must name a tree for each of the H_q heads")
        order = torch.argsort(m, stable=True).to(torch.int32)
        off = torch.zeros(t + 1, dtype=torch.int32)
        off[1:] = torch.cumsum(torch.bincount(m, minlength=t), 0)
        keep = (off.to(samples.device), order.to(samples.device))
        qs = _lib.HiraQuery(h_q, query.data_ptr(), None, None, keep[0].data_ptr(),
                            keep[1].data_ptr(), int(off.diff().max()), 0)
    if out is None:
        out = torch.empty((h_q,), dtype=torch.float32, device=samples.device)
    if stream is None:
        stream = _lib.current_stream(samples.device)
    code = {"sample_max": 0, "sample_mean_topk": 1}[method]
    _lib.check(_lib.lib().hira_threshold(
        samples.data_ptr(), _lib.HIRA_BF16 if samples.dtype == torch.bfloat16 else _lib.HIRA_F32,
        t, n_s, d, C.byref(qs), code, int(k), out.data_ptr(), stream))
    del keep
    return out


def sample_max(samples, query, q_head_to_kv=None) -> torch.Tensor:
    """Threshold = the largest score among the samples."""
    if samples.is_cuda:
        return device_thresholds(samples, query, "sample_max", 1, q_head_to_kv)
    return _scores(samples, query, q_head_to_kv).max(dim=-1).values


def sample_mean_topk(samples, query, k, q_head_to_kv=None) -> torch.Tensor:
    """Threshold = mean of the k largest sample scores."""
    k = max(1, min(int(k), samples.shape[-2]))
    if samples.is_cuda:
        return device_thresholds(samples, query, "sample_mean_topk", k, q_head_to_kv)
    s = _scores(samples, query, q_head_to_kv)
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
