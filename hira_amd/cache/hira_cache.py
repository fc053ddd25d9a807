"""HiraCache / HiraCacheLayer: HuggingFace cache objects that own one index per layer.

Mirrors the reference's cache/hira_cache.py:19-249: the first ``update`` of a layer
(prefill) builds the index and returns the prefill tensors untouched; later updates queue
the new keys/values and fold the queue into the index every ``update_every`` tokens.
``update`` returns ``(CacheOutput, None)``, as the reference does, and the attention
function (attention/hira_attention.py) reads indexer, searcher and queue from it.

Both spellings of the two methods whose name or signature changed between transformers
releases are provided: ``get_max_cache_shape`` (reference, cache/hira_cache.py:167-168) /
``get_max_length``, and ``get_mask_sizes(cache_position tensor | query_length int)``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any

import torch
from transformers.cache_utils import Cache, CacheLayerMixin

from hira_amd.cache.hira_config import DeviceMode, HiraConfig
from hira_amd.indexer import HIPIndexer
from hira_amd.searcher import HIPSearcher

# names the reference binds in this module (tests patch them there)
CUDAIndexer = HIPIndexer
CUDASearcher = HIPSearcher


@dataclass
class CacheOutput:
    queued_keys: torch.Tensor
    queued_values: torch.Tensor
    prefill_keys: torch.Tensor | None
    prefill_values: torch.Tensor | None
    indexer: Any
    searcher: Any
    # beyond the reference's fields: the layer's key sample (B*H_kv, S, D) and the rule that
    # turns it into per-head thresholds (cache/hira_config.py:20-22 of the reference)
    samples: torch.Tensor | None = None
    threshold_method: str | None = None
    threshold_topk: int = 1
    # the buffers queued_keys / queued_values are views of: (B, H_kv, cap, D) in the index's
    # storage type and on its device, the first queued_keys.shape[-2] rows of every head in
    # use.  The attention function hands them to the library as they are.
    queue_store: tuple | None = None


class HiraCacheLayer(CacheLayerMixin):
    """One layer, all KV heads.  key_states / value_states: (B, H_kv, L, D)."""

    def __init__(
        self,
        device_mode: str,
        update_every: int,
        indexer_kwargs: dict[str, Any],
        searcher_kwargs: dict[str, Any],
        threshold_kwargs: dict[str, Any] | None = None,
    ):
        super().__init__()
        self.threshold_kwargs = threshold_kwargs or {}
        self.samples = None
        self.device_mode = device_mode
        self.update_every = update_every
        self.indexer_kwargs = indexer_kwargs
        self.searcher_kwargs = searcher_kwargs
        if self.device_mode == DeviceMode.CUDA_ONLY:
            # looked up at call time so that the module-level names can be replaced
            import hira_amd.cache.hira_cache as me

            self.indexer_cls = me.CUDAIndexer
            self.searcher_cls = me.CUDASearcher
        elif self.device_mode == DeviceMode.CPU_ONLY:
            raise NotImplementedError(
                "cpu_only is the reference's host path; this package is the MI355X path "
                "(device_mode='cuda_only')")
        else:
            raise NotImplementedError(f"Device mode {self.device_mode} not supported yet")
        self.indexed_len = 0
        self.queued_len = 0
        self._update_takes_sync = None

    def _alloc_queue(self, rows: int):
        """Room for `rows` queued keys and values per head, allocated once (the reference
        concatenates per token, cache/hira_cache.py:121-140): in the index's storage type and
        on its device, so that a decode step passes the buffers on without a copy."""
        dt = getattr(self.indexer, "dtype", None) or self.dtype
        dev = getattr(self.indexer, "device", None) or self.device
        self._queue_k = torch.empty((self.batch, self.H_kv, rows, self.dim), dtype=dt, device=dev)
        self._queue_v = torch.empty((self.batch, self.H_kv, rows, self.vdim), dtype=dt, device=dev)

    @property
    def queued_keys(self):
        return self._queue_k.narrow(2, 0, self.queued_len)

    @property
    def queued_values(self):
        return self._queue_v.narrow(2, 0, self.queued_len)

    def _enqueue(self, key_states, value_states):
        m = key_states.shape[-2]
        if self.queued_len + m > self._queue_k.shape[-2]:  # (a step of many tokens)
            old_k, old_v, n = self._queue_k, self._queue_v, self.queued_len
            self._alloc_queue(max(2 * old_k.shape[-2], n + m))
            self._queue_k[:, :, :n] = old_k[:, :, :n]
            self._queue_v[:, :, :n] = old_v[:, :, :n]
        if key_states.ndim != 4:
            key_states = key_states.reshape(self.batch, self.H_kv, m, self.dim)
            value_states = value_states.reshape(self.batch, self.H_kv, m, self.vdim)
        self._queue_k.narrow(2, self.queued_len, m).copy_(key_states)
        self._queue_v.narrow(2, self.queued_len, m).copy_(value_states)
        self.queued_len += m

    def lazy_initialization(self, key_states, value_states):
        self.dim = key_states.shape[-1]
        self.vdim = value_states.shape[-1]
        self.H_kv = key_states.shape[-3]
        self.batch = key_states.shape[0] if key_states.ndim == 4 else 1
        self.dtype = key_states.dtype
        self.device = key_states.device
        self.indexer = self.indexer_cls(**self.indexer_kwargs)
        self.searcher = self.searcher_cls(**self.searcher_kwargs)
        self.queued_len = 0
        self._queue_k = self._queue_v = None  # allocated once the index knows its storage type
        self.keys = None  # the index holds the keys
        self.values = None
        self.is_initialized = True

    def update(self, key_states: torch.Tensor, value_states: torch.Tensor,
               cache_kwargs: dict[str, Any] | None = None, *args, **kwargs):
        if not self.is_initialized:
            self.lazy_initialization(key_states, value_states)
            self.indexer.build(key_states, value_states)
            # what the first append and the first subtree rebuild of a process load on first use
            # is loaded now, beside the prefill, not in the middle of the decode
            if hasattr(self.indexer, "warm_up"):
                try:
                    self.indexer.warm_up()
                except Exception as ex:  # (a courtesy, not a step of the prefill)
                    import warnings

                    warnings.warn(f"index warm-up skipped: {ex}")
            self._alloc_queue(max(1, min(int(self.update_every), 4096)))
            self.indexed_len = key_states.shape[-2]
            self._take_samples(key_states)
            return self._output(key_states, value_states), None
        self._enqueue(key_states, value_states)
        if self.queued_len >= self.update_every:
            self.update_index()
        return self._output(), None

    def _take_samples(self, key_states):
        """A seeded random sample of the prompt's keys per KV head, for the sample-based
        threshold rules; none when the configured rule does not use one."""
        kw = self.threshold_kwargs
        if kw.get("method") not in ("sample_max", "sample_mean_topk") or kw.get("sample_size", 0) <= 0:
            return
        n = key_states.shape[-2]
        self._sample_target = min(int(kw["sample_size"]), 4096)
        s = min(self._sample_target, n)
        self._sample_gen = torch.Generator().manual_seed(12345)
        pick = torch.randperm(n, generator=self._sample_gen)[:s].sort().values
        k4 = key_states if key_states.ndim == 4 else key_states[None]
        # (in the index's storage dtype: the threshold kernel reads samples and queries alike)
        store = getattr(self.indexer, "dtype", None) or k4.dtype
        self.samples = k4[:, :, pick.to(k4.device)].reshape(-1, s, self.dim).to(store).contiguous()

    def _refresh_samples(self, new_keys, seen: int):
        """Keep the sample uniform over all indexed keys as the index grows (reservoir
        sampling, the same positions for every head): key number i (0-based) of the sequence
        joins with probability S/(i+1) in place of a random member; while the sample is still
        smaller than S every new key joins."""
        if self.samples is None:
            return
        k4 = new_keys if new_keys.ndim == 4 else new_keys[None]
        m = k4.shape[-2]
        rows = k4.reshape(-1, m, self.dim).to(self.samples.dtype)
        room = self._sample_target - self.samples.shape[1]
        if room > 0:  # a short prompt: the sample holds every key so far
            take = min(room, m)
            self.samples = torch.cat([self.samples, rows[:, :take]], dim=1).contiguous()
            rows, seen, m = rows[:, take:], seen + take, m - take
            if m == 0:
                return
        s = self.samples.shape[1]
        idx = seen + torch.arange(m)
        join = torch.rand(m, generator=self._sample_gen) < s / (idx + 1).double()
        if bool(join.any()):
            who = join.nonzero().squeeze(1)
            slots = torch.randint(0, s, (who.numel(),), generator=self._sample_gen)
            # a slot drawn twice keeps its last arrival (an indexed assignment with repeated
            # targets has no defined order)
            last = {int(sl): int(wh) for sl, wh in zip(slots.tolist(), who.tolist())}
            slots = torch.tensor(list(last.keys()), dtype=torch.long)
            who = torch.tensor(list(last.values()), dtype=torch.long)
            self.samples[:, slots.to(self.samples.device)] = rows[:, who.to(rows.device)]

    def _output(self, prefill_keys=None, prefill_values=None):
        kw = self.threshold_kwargs
        return CacheOutput(
            queued_keys=self.queued_keys,
            queued_values=self.queued_values,
            prefill_keys=prefill_keys,
            prefill_values=prefill_values,
            indexer=self.indexer,
            searcher=self.searcher,
            samples=self.samples,
            threshold_method=kw.get("method") if self.samples is not None else None,
            threshold_topk=max(1, min(int(kw.get("topk", 1)),
                                      self.samples.shape[1] if self.samples is not None else 1)),
            queue_store=(self._queue_k, self._queue_v),
        )

    def update_index(self):
        # no read-back of the level sizes: the host carries their bounds (HIPIndexer.update,
        # sync=False), so folding the queue into the index does not wait for the GPU; a
        # one-level index has no node counts to bound with and keeps the synchronous form
        if self._update_takes_sync is None:
            import inspect

            self._update_takes_sync = "sync" in inspect.signature(self.indexer.update).parameters
        if self._update_takes_sync:
            self.indexer.update(self.queued_keys, self.queued_values,
                                sync=getattr(self.indexer, "num_levels", 1) < 2)
        else:  # an indexer with the reference's two-argument update
            self.indexer.update(self.queued_keys, self.queued_values)
        self._refresh_samples(self.queued_keys, self.indexed_len)
        self.indexed_len += self.queued_len
        self.queued_len = 0

    def get_mask_sizes(self, cache_position):
        kv_offset = 0
        query_length = (int(cache_position) if isinstance(cache_position, int)
                        else cache_position.shape[0])
        return self.get_seq_length() + query_length, kv_offset

    def get_seq_length(self):
        if not self.is_initialized:
            return 0
        return self.indexed_len + self.queued_len

    def get_max_cache_shape(self):
        return -1

    def get_max_length(self):
        return -1

    def reset(self):
        if self.is_initialized:
            self.indexer = self.indexer_cls(**self.indexer_kwargs)
            self._queue_k = self._queue_v = None
            self.queued_len = 0
            self.indexed_len = 0
            self.samples = None
            self.is_initialized = False
        if hasattr(self, "cumulative_length"):
            self.cumulative_length = 0


class HiraCache(Cache):
    """HuggingFace ``Cache`` whose layers are HiraCacheLayer (cache/hira_cache.py:187-249)."""

    def __init__(self, cache_config, hira_config: HiraConfig):
        self.device_mode = hira_config.device_mode
        self.update_every = hira_config.update_every
        config = cache_config.get_text_config(decoder=True)
        layer_types = getattr(config, "layer_types", None)
        if layer_types is None:
            if getattr(config, "sliding_window", None) is not None:
                layer_types = ["sliding_attention" for _ in range(config.num_hidden_layers)]
            elif getattr(config, "attention_chunk_size", None) is not None:
                layer_types = ["chunked_attention" for _ in range(config.num_hidden_layers)]
            else:
                layer_types = ["full_attention" for _ in range(config.num_hidden_layers)]
        if hasattr(config, "num_kv_shared_layers"):
            layer_types = layer_types[: -config.num_kv_shared_layers]
        # query heads per KV head: the indexer's layout="auto" weighs it (an 8-bit shadow of the
        # keys pays from 8 heads a tree on)
        heads, kv_heads = (getattr(config, "num_attention_heads", None),
                           getattr(config, "num_key_value_heads", None))
        group = heads // kv_heads if heads and kv_heads and heads % kv_heads == 0 else None
        layers = [
            HiraCacheLayer(
                device_mode=self.device_mode,
                update_every=self.update_every,
                indexer_kwargs=self._indexer_kwargs(hira_config, group),
                searcher_kwargs=hira_config.get_searcher_kwargs(),
                threshold_kwargs=hira_config.get_threshold_kwargs(),
            )
            for _ in layer_types
        ]
        super().__init__(layers=layers, offloading=False)

    @staticmethod
    def _indexer_kwargs(hira_config: HiraConfig, group):
        """The configuration's indexer arguments, plus the heads per tree where the indexer in
        use takes them (one with the reference's constructor does not)."""
        import inspect

        import hira_amd.cache.hira_cache as me

        kw = dict(hira_config.get_indexer_kwargs())
        try:
            params = inspect.signature(me.CUDAIndexer.__init__).parameters
        except (TypeError, ValueError):
            params = {}
        if group is not None and "heads_per_tree" in params:
            kw["heads_per_tree"] = group
        return kw

    def update(self, key_states: torch.Tensor, value_states: torch.Tensor, layer_idx: int,
               cache_kwargs: dict[str, Any] | None = None, *args, **kwargs):
        cache_output, _ = self.layers[layer_idx].update(key_states, value_states, cache_kwargs)
        return cache_output, None
