"""The attention function the reference leaves unwritten (attention/hira_attention.py:1-3
only points at transformers' AttentionInterface).

Calling convention of transformers' attention functions:

    fn(module, query (B, H_q, L_q, D), key, value, attention_mask, dropout=0.0,
       scaling=None, **kwargs) -> (attn_output (B, L_q, H_q, Dv), None)

``key`` is what ``HiraCache.update`` returned in place of the key states: a ``CacheOutput``
(cache/hira_cache.py:19-26 of the reference).

* prefill (``prefill_keys`` present): ordinary causal attention over the prompt;
* decode (L_q == 1): out[h] = softmax over {indexed keys with q_h.k >= tau_h} + {queued
  keys} of scaling * q_h.k, times V -- one fused search + sparse-attention launch.

The threshold comes from ``hira_threshold`` (tensor (B*H_q,) or scalar), from ``hira_topk``
(int: select exactly the k best indexed keys per head; scans every key, for tests), or, with
neither given, from the cache layer's key sample by its configured rule (HiraConfig
``threshold_method`` / ``sample_size``).
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn.functional as F



def _repeat_kv(x: torch.Tensor, n_rep: int) -> torch.Tensor:
    if n_rep == 1:
        return x
    b, h, l, d = x.shape
    return x[:, :, None].expand(b, h, n_rep, l, d).reshape(b, h * n_rep, l, d)


def _dense(query, key, value, attention_mask, scaling, is_causal):
    n_rep = query.shape[1] // key.shape[1]
    out = F.scaled_dot_product_attention(
        query, _repeat_kv(key, n_rep), _repeat_kv(value, n_rep),
        attn_mask=attention_mask, scale=scaling,
        is_causal=is_causal and attention_mask is None and query.shape[2] > 1)
    return out.transpose(1, 2).contiguous()


def _hides_a_key(attention_mask) -> bool:
    """Does the mask hide a key from the LAST query position?  Causal masking never does (the
    last position sees every key before it), so what it hides there is padding.  Boolean masks:
    True = attend; floating masks are additive (0 = attend); integer masks: 1 = attend."""
    if attention_mask is None:
        return False
    last = attention_mask[..., -1, :] if attention_mask.ndim >= 3 else attention_mask
    if last.dtype == torch.bool:
        return bool((~last).any())
    if last.is_floating_point():
        return bool((last != 0).any())
    return bool((last == 0).any())


_PADDING_ERROR = (
    "hira attention: the attention mask hides key positions (a padded batch). The index holds "
    "every cached position and the sparse decode step attends to all it selects, so padded "
    "prompts would silently attend to pad keys; run sequences of equal length per batch, or "
    "one sequence per cache")


def index_thresholds(indexer, query: torch.Tensor, topk: int) -> torch.Tensor:
    """(B*H_q,) thresholds that keep exactly the `topk` best indexed keys of every head."""
    keys = indexer.keys_rowmajor()  # (T, N_pad, D) slot order
    q = query.reshape(-1, query.shape[-1])
    t = indexer.num_trees
    qg = q.reshape(t, -1, q.shape[-1]).float()
    s = torch.einsum("tnd,tgd->tgn", keys.float(), qg)
    s = s.masked_fill((indexer.perm[:, None, : indexer.size[0]] < 0), float("-inf"))
    s = s.reshape(q.shape[0], -1)
    k = max(1, min(int(topk), indexer.num_keys))
    top = s.topk(min(k + 1, s.shape[-1]), dim=-1).values
    if top.shape[-1] == k or k == indexer.num_keys:
        return top[:, k - 1].contiguous()
    return ((top[:, k - 1].double() + top[:, k].double()) * 0.5).float()


def hira_attention_forward(module, query, key, value, attention_mask=None, dropout: float = 0.0,
                           scaling: Optional[float] = None, hira_threshold=None,
                           hira_topk: Optional[int] = None, **kwargs):
    d = query.shape[-1]
    if scaling is None:
        scaling = getattr(module, "scaling", None) or d ** -0.5
    if not hasattr(key, "indexer"):  # plain tensors: no cache in use
        return _dense(query, key, value, attention_mask, scaling, True), None
    cache = key
    if cache.prefill_keys is not None:
        if _hides_a_key(attention_mask):
            raise ValueError(_PADDING_ERROR)
        return _dense(query, cache.prefill_keys, cache.prefill_values, attention_mask, scaling,
                      True), None
    if query.shape[2] != 1:
        raise ValueError("sparse decode expects one query position per step")
    indexer, searcher = cache.indexer, cache.searcher
    b, h_q = query.shape[0], query.shape[1]
    # a mask that hides keys cannot be honoured by the decode step: looked at once per index
    # (padding does not move between steps, and the look costs a host synchronisation)
    if attention_mask is not None and not getattr(indexer, "_decode_mask_checked", False):
        if _hides_a_key(attention_mask):
            raise ValueError(_PADDING_ERROR)
        indexer._decode_mask_checked = True
    if hira_threshold is None:
        hira_threshold = getattr(module, "hira_threshold", None)
    if hira_topk is None:
        hira_topk = getattr(module, "hira_topk", None)
    # with neither given: the cache layer's configured rule on its key sample, one small launch
    # ahead of the search
    sampled = hira_threshold is None and hira_topk is None and getattr(cache, "samples", None) is not None
    if hira_threshold is None and not sampled:
        hira_threshold = index_thresholds(indexer, query, hira_topk or max(1, indexer.num_keys // 100))
    # one plan per (index, head count, scale): a decode step is then a single library call
    plan = searcher.decode_plan(indexer, b * h_q, scaling)
    q2 = query.reshape(b * h_q, d)
    if q2.dtype != indexer.dtype or q2.device != indexer.device:
        q2 = q2.to(device=indexer.device, dtype=indexer.dtype)
    q2 = q2.contiguous()
    out = torch.empty((b * h_q, indexer.vdim), dtype=torch.float32, device=indexer.device)
    # the queue: the cache layer's own buffers as they are when they already hold the index's
    # storage type (rows in use, rows per head), else a converted copy of the rows in use
    qk = qv = None
    qlen = int(cache.queued_keys.shape[-2]) if cache.queued_keys is not None else 0
    if qlen > 0:
        store = getattr(cache, "queue_store", None)
        if store is not None and store[0].dtype == indexer.dtype and store[0].device == indexer.device \
                and store[0].is_contiguous() and store[1].is_contiguous():
            qk, qv = store
        else:
            qk = cache.queued_keys.to(device=indexer.device, dtype=indexer.dtype).reshape(
                indexer.num_trees, qlen, d).contiguous()
            qv = cache.queued_values.to(device=indexer.device, dtype=indexer.dtype).reshape(
                indexer.num_trees, qlen, -1).contiguous()
    if sampled:
        plan.run_sampled(q2, cache.samples, cache.threshold_method, cache.threshold_topk, out,
                         queue_keys=qk, queue_values=qv, queue_len=qlen)
    else:
        th = torch.as_tensor(hira_threshold, dtype=torch.float32, device=indexer.device)
        if th.ndim == 0:
            th = th.expand(b * h_q)
        th = th.reshape(b * h_q).contiguous()
        plan.run(q2, th, out, queue_keys=qk, queue_values=qv, queue_len=qlen)
    return out.reshape(b, 1, h_q, -1).to(query.dtype), None


def register_hira_attention(name: str = "hira") -> str:
    """Make the function selectable as ``attn_implementation=name``."""
    from transformers import AttentionInterface

    AttentionInterface.register(name, hira_attention_forward)
    return name
