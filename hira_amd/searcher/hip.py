"""HIPSearcher: halfspace range search (and fused sparse attention) on one MI355X.

Replaces the reference's GPU searcher (searcher/cuda.py:15-143) and, through
``index_space="position"``, the CPU searcher's contract (searcher/cpu.py:44-101):
``search(query (1,H_q,1,D), threshold (H_q,), indexer, q_head_to_kv=None, scaling=None)``
returns an ``(H_q, N)`` fp32 tensor holding ``score * scaling`` for every key with
``q.k >= threshold`` and ``output_fill_value`` elsewhere.

Semantics follow the CPU kernels (keep a node when ``q.c + ||q|| r >= t``, a key when
``q.k >= t``: kernels/cpp/torch_ext_v3.cpp:182, 212, 238), not the Triton kernels, which
gate with a strict ``>`` and never filter the leaves (kernels/triton_search_kernels.py:
49-63).  Like the reference's GPU searcher the dense result lives in a buffer this object
keeps and reuses: clone it to hold on to a result across calls (searcher/cuda.py:35-54).
"""
from __future__ import annotations

import ctypes as C
from typing import Optional, Tuple

import torch

from .. import _lib
from .base import BaseSearcher

DEFAULT_OUTPUT_FILL_VALUE = 0.0


def _on(t: torch.Tensor, device) -> bool:
    """Is tensor `t` on `device`?  ("cuda" without an index means the current device, which a
    tensor's own device always spells out.)"""
    device = torch.device(device)
    if t.device.type != device.type:
        return False
    if device.index is None:
        return device.type != "cuda" or t.device.index == torch.cuda.current_device()
    return t.device.index == device.index


class HIPSearcher(BaseSearcher):
    def __init__(self, block_c=None, output_fill_value: float = DEFAULT_OUTPUT_FILL_VALUE,
                 *, index_space: str = "slot", block_threads: int = 0, nodes_per_wave: int = 0,
                 kernel: int = 0, separate_merge: bool = False):
        super().__init__()
        if index_space not in ("slot", "position"):
            raise ValueError("index_space must be 'slot' or 'position'")
        self.block_c = block_c  # accepted for HiraConfig.get_searcher_kwargs(); unused
        self.output_fill_value = float(output_fill_value)
        self.index_space = index_space
        self.launch = _lib.HiraLaunch(int(block_threads), int(nodes_per_wave), int(kernel),
                                      int(bool(separate_merge)))
        self._tmp_out: Optional[torch.Tensor] = None
        self._map_cache = {}
        self._workspace: Optional[torch.Tensor] = None
        self._decode_plans: dict = {}
        self._sel = None

    # -------------------------------------------------------------- input coercion
    @staticmethod
    def _coerce_query(query, d: int) -> torch.Tensor:
        """(H_q, D), (1, H_q, 1, D) or, for B sequences, (B, H_q, 1, D) -> (B*H_q, D)
        (kernels/triton_search_wrappers.py:9-27)."""
        if not isinstance(query, torch.Tensor):
            raise TypeError(f"q must be a torch.Tensor, got {type(query)}")
        if query.ndim == 4:
            if query.shape[2] != 1:
                raise ValueError(f"4D query must be (B,H,1,D), got {tuple(query.shape)}")
            query = query.squeeze(2).reshape(-1, query.shape[-1])
        elif query.ndim != 2:
            raise ValueError(f"q must be (H,d) or (1,H,1,D), got {tuple(query.shape)}")
        if query.shape[-1] != d:
            raise ValueError(f"query dim mismatch: expected d={d}, got {query.shape[-1]}")
        return query

    @staticmethod
    def _coerce_threshold(t, h: int, device) -> torch.Tensor:
        """scalar or (H_q,) (kernels/triton_search_wrappers.py:57-71)."""
        if torch.is_tensor(t):
            t = t.to(device=device, dtype=torch.float32).reshape(-1)
        else:
            t = torch.tensor([float(t)], device=device, dtype=torch.float32)
        if t.numel() == 1 and h > 1:
            t = t.expand(h)
        if t.numel() != h:
            raise ValueError(f"threshold must be scalar or length H={h}, got {t.numel()}")
        return t.contiguous()

    @staticmethod
    def _coerce_scaling(scaling, h: int, device) -> torch.Tensor:
        """None or (H_q,) (kernels/triton_search_wrappers.py:74-89; the finiteness check
        there costs a host sync per call and is left to the caller)."""
        if scaling is None:
            return torch.ones((h,), device=device, dtype=torch.float32)
        if not torch.is_tensor(scaling):
            raise TypeError(f"scaling must be a torch.Tensor with shape (H,), got {type(scaling)}")
        s = scaling.to(device=device, dtype=torch.float32).reshape(-1)
        if s.numel() != h:
            raise ValueError(f"scaling must have length H={h}, got {s.numel()}")
        return s.contiguous()

    def _head_map(self, h_q: int, indexer, q_head_to_kv) -> Tuple[torch.Tensor, torch.Tensor, int, int]:
        """CSR of the query heads of each tree.  Default map: head h of sequence b belongs
        to tree b*H_kv + h // (H_q/H_kv) (searcher/cuda.py:23-33)."""
        t, batch, h_kv = indexer.num_trees, indexer.batch, indexer.num_heads
        key = (h_q, t, batch, None if q_head_to_kv is None
               else tuple(int(x) for x in torch.as_tensor(q_head_to_kv).reshape(-1).tolist()))
        hit = self._map_cache.get(key)
        if hit is not None:
            return hit
        group = 0
        if q_head_to_kv is None:
            if h_q % batch:
                raise ValueError(f"H_q={h_q} not divisible by batch={batch}")
            per_seq = h_q // batch
            if per_seq == h_kv:
                local = torch.arange(per_seq)
            else:
                if per_seq % h_kv:
                    raise ValueError(
                        f"Unsupported head mapping: H_q={per_seq} must equal or be divisible "
                        f"by H_kv={h_kv}")
                local = torch.arange(per_seq) // (per_seq // h_kv)
            m = (torch.arange(batch)[:, None] * h_kv + local[None, :]).reshape(-1)
            group = per_seq // h_kv  # head h of the launch belongs to tree h // group
        else:
            if not torch.is_tensor(q_head_to_kv):
                raise TypeError(
                    f"q_head_to_kv must be a torch.Tensor or None, got {type(q_head_to_kv)}")
            m = q_head_to_kv.detach().to("cpu", torch.long).reshape(-1)
            if m.numel() != h_q:
                raise ValueError(f"q_head_to_kv length mismatch: expected H_q={h_q}, got {m.numel()}")
            if bool(((m < 0) | (m >= t)).any()):
                raise ValueError(f"q_head_to_kv values must be in [0, {t - 1}]")
        order = torch.argsort(m, stable=True)
        counts = torch.bincount(m, minlength=t)
        off = torch.zeros(t + 1, dtype=torch.int32)
        off[1:] = counts.cumsum(0).to(torch.int32)
        dev = indexer.device
        val = (off.to(dev), order.to(torch.int32).to(dev), int(counts.max().item()), group)
        self._map_cache = {key: val}
        return val

    def _query_struct(self, query, threshold, indexer, q_head_to_kv, scaling):
        dev = indexer.device
        q = self._coerce_query(query, indexer.dim).to(device=dev, dtype=indexer.dtype).contiguous()
        h_q = q.shape[0]
        tau = self._coerce_threshold(threshold, h_q, dev)
        sc = self._coerce_scaling(scaling, h_q, dev)
        off, heads, gmax, group = self._head_map(h_q, indexer, q_head_to_kv)
        qs = _lib.HiraQuery(h_q, q.data_ptr(), tau.data_ptr(), sc.data_ptr(), off.data_ptr(),
                            heads.data_ptr(), gmax, group)
        return qs, (q, tau, sc, off, heads)

    def _get_workspace(self, nbytes: int, device) -> torch.Tensor:
        if self._workspace is None or self._workspace.numel() < nbytes or \
                not _on(self._workspace, device):
            # zero once: the arrival counters inside must start at zero and are left at
            # zero by every call
            self._workspace = torch.zeros(max(nbytes, 1), dtype=torch.uint8, device=device)
        return self._workspace

    def _prepare_output_buffer(self, h_q: int, n: int, device, fill: bool = True) -> torch.Tensor:
        """searcher/cuda.py:35-54.  fill=False: the search writes the fill value itself."""
        if self._tmp_out is None or not _on(self._tmp_out, device) or \
                tuple(self._tmp_out.shape) != (h_q, n):
            self._tmp_out = torch.full((h_q, n), self.output_fill_value, device=device,
                                       dtype=torch.float32)
        elif fill:
            self._tmp_out.fill_(self.output_fill_value)
        return self._tmp_out

    def _run(self, indexer, qs, out: _lib.HiraSearchOut, queue: Optional[_lib.HiraQueue]):
        lib = _lib.lib()
        tree = indexer.tree_struct()
        ws_ptr, ws_bytes, ws = None, 0, None
        if out.attn_out:
            ws_bytes = lib.hira_search_workspace_bytes(
                C.byref(tree), C.byref(qs), C.byref(queue) if queue else None,
                C.byref(self.launch))
            ws = self._get_workspace(ws_bytes, indexer.device)
            ws_ptr = ws.data_ptr()
        stream = _lib.current_stream(indexer.device)
        rc = lib.hira_search(C.byref(tree), C.byref(qs), C.byref(queue) if queue else None,
                             C.byref(out), C.byref(self.launch), ws_ptr, ws_bytes, stream)
        _lib.check(rc)

    # -------------------------------------------------------------- public API
    def search(self, query, threshold, indexer, q_head_to_kv: Optional[torch.Tensor] = None,
               scaling: Optional[torch.Tensor] = None, *, index_space: Optional[str] = None,
               stats: Optional[torch.Tensor] = None) -> torch.Tensor:
        if indexer.keys_buf is None:
            raise ValueError("Indexer is not built: missing children tensor.")
        space = index_space or self.index_space
        qs, keep = self._query_struct(query, threshold, indexer, q_head_to_kv, scaling)
        n = indexer.size[0] if space == "slot" else indexer.num_keys
        # in slot space the search fills what it does not select itself: one launch per call
        fused_fill = space == "slot"
        dense = self._prepare_output_buffer(qs.num_q_heads, n, indexer.device, fill=not fused_fill)
        out = _lib.HiraSearchOut()
        out.dense = dense.data_ptr()
        out.dense_stride = dense.stride(0)
        out.dense_by_position = 1 if space == "position" else 0
        out.dense_fill = 1 if fused_fill else 0
        out.dense_fill_value = self.output_fill_value
        out.stats = None if stats is None else stats.data_ptr()
        self._run(indexer, qs, out, None)
        del keep
        return dense

    def search_compact(self, query, threshold, indexer, q_head_to_kv=None, scaling=None, *,
                       capacity: Optional[int] = None, index_space: Optional[str] = None):
        """Compact result: (index (H_q, cap) int32, score (H_q, cap) fp32 raw q.k,
        count (H_q,) int32); entries of a head are unordered."""
        space = index_space or self.index_space
        qs, keep = self._query_struct(query, threshold, indexer, q_head_to_kv, scaling)
        cap = int(capacity or indexer.size[0])
        h_q, dev = qs.num_q_heads, indexer.device
        if self._sel is None or self._sel[0].shape != (h_q, cap) or not _on(self._sel[0], dev):
            self._sel = (torch.empty((h_q, cap), dtype=torch.int32, device=dev),
                         torch.empty((h_q, cap), dtype=torch.float32, device=dev),
                         torch.zeros((h_q,), dtype=torch.int32, device=dev))
        idx, score, count = self._sel
        count.zero_()
        out = _lib.HiraSearchOut()
        out.dense_by_position = 1 if space == "position" else 0
        out.sel_index, out.sel_score, out.sel_count = idx.data_ptr(), score.data_ptr(), count.data_ptr()
        out.sel_cap = cap
        self._run(indexer, qs, out, None)
        del keep
        return idx, score, count

    def sparse_attention(self, index: torch.Tensor, score: torch.Tensor, count: torch.Tensor,
                         indexer, q_head_to_kv=None, scaling=None,
                         out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """softmax(scaling * score) V over given lists (``search_compact`` in the slot index
        space, possibly edited): index (H_q, cap) int32 key slots, score (H_q, cap) fp32 raw
        q.k, count (H_q,) int32.  Returns (H_q, Dv) fp32; zeros where a list is empty."""
        if indexer.values_buf is None:
            raise ValueError("the index was built without values: nothing to attend to")
        if index.ndim != 2 or index.shape != score.shape or count.shape != (index.shape[0],):
            raise ValueError(f"lists must be (H_q, cap), (H_q, cap), (H_q,): got "
                             f"{tuple(index.shape)}, {tuple(score.shape)}, {tuple(count.shape)}")
        h_q, cap = index.shape
        dev = indexer.device
        index = index.to(device=dev, dtype=torch.int32).contiguous()
        score = score.to(device=dev, dtype=torch.float32).contiguous()
        count = count.to(device=dev, dtype=torch.int32).contiguous()
        sc = self._coerce_scaling(scaling, h_q, dev)
        off, heads, gmax, group = self._head_map(h_q, indexer, q_head_to_kv)
        qs = _lib.HiraQuery(h_q, None, None, sc.data_ptr(), off.data_ptr(), heads.data_ptr(),
                            gmax, group)
        if out is None:
            out = torch.empty((h_q, indexer.vdim), dtype=torch.float32, device=dev)
        tree = indexer.tree_struct()
        stream = _lib.current_stream(dev)
        _lib.check(_lib.lib().hira_sparse_attention(
            C.byref(tree), C.byref(qs), index.data_ptr(), score.data_ptr(), count.data_ptr(),
            int(cap), out.data_ptr(), stream))
        return out

    def search_attention(self, query, threshold, indexer, q_head_to_kv=None, scaling=None, *,
                         queue_keys: Optional[torch.Tensor] = None,
                         queue_values: Optional[torch.Tensor] = None,
                         out: Optional[torch.Tensor] = None,
                         stats: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Fused search + softmax(scaling * q.K_S^T) V_S over the selected keys and, when
        given, every queued key (T, m, D) / value (T, m, Dv).  Returns (H_q, Dv) fp32."""
        if indexer.values_buf is None:
            raise ValueError("the index was built without values: nothing to attend to")
        qs, keep = self._query_struct(query, threshold, indexer, q_head_to_kv, scaling)
        h_q, dev = qs.num_q_heads, indexer.device
        if out is None:
            out = torch.empty((h_q, indexer.vdim), dtype=torch.float32, device=dev)
        so = _lib.HiraSearchOut()
        so.attn_out = out.data_ptr()
        so.stats = None if stats is None else stats.data_ptr()
        queue = None
        if queue_keys is not None and queue_keys.shape[-2] > 0:
            qk = queue_keys.reshape(indexer.num_trees, -1, indexer.dim)
            qv = queue_values.reshape(indexer.num_trees, -1, indexer.vdim)
            qk = qk.to(device=dev, dtype=indexer.dtype).contiguous()
            qv = qv.to(device=dev, dtype=indexer.dtype).contiguous()
            queue = _lib.HiraQueue(qk.data_ptr(), qv.data_ptr(), qk.shape[1], qk.shape[1])
            keep = keep + (qk, qv)
        self._run(indexer, qs, so, queue)
        del keep
        return out

    def decode_plan(self, indexer, num_q_heads: int, scaling: float) -> "DecodePlan":
        """The plan for (this index, head count, one softmax scale for all heads), made on
        first use and kept: callers that come once per decode step and layer (the attention
        function) then pay one library call per step."""
        plans = self._decode_plans
        key = (id(indexer), int(num_q_heads), float(scaling))
        plan = plans.get(key)
        if plan is None or plan.indexer is not indexer:  # (ids are reused once an index is gone)
            scale = torch.full((num_q_heads,), float(scaling), dtype=torch.float32,
                               device=indexer.device)
            plan = plans[key] = self.plan_attention(indexer, num_q_heads, scaling=scale)
        return plan

    def plan_attention(self, indexer, num_q_heads: int, scaling=None, q_head_to_kv=None,
                       stats: Optional[torch.Tensor] = None) -> "DecodePlan":
        """Pre-resolve everything that does not change between decode steps (head map,
        scaling, workspace) so that a step is one library call on ready device tensors."""
        return DecodePlan(self, indexer, num_q_heads, scaling, q_head_to_kv, stats)


class DecodePlan:
    """One fused search + attention call per ``run``: ``query`` (H_q, D) in the tree dtype,
    ``threshold`` (H_q,) fp32 and ``out`` (H_q, Dv) fp32 must be contiguous device tensors."""

    def __init__(self, searcher: HIPSearcher, indexer, num_q_heads: int, scaling, q_head_to_kv,
                 stats):
        if indexer.values_buf is None:
            raise ValueError("the index was built without values: nothing to attend to")
        self.indexer = indexer
        self.searcher = searcher
        self.lib = _lib.lib()
        dev = indexer.device
        self.scaling = searcher._coerce_scaling(scaling, num_q_heads, dev)
        off, heads, gmax, group = searcher._head_map(num_q_heads, indexer, q_head_to_kv)
        self._keep = (off, heads, stats)
        self.query = _lib.HiraQuery(num_q_heads, None, None, self.scaling.data_ptr(),
                                    off.data_ptr(), heads.data_ptr(), gmax, group)
        self.out = _lib.HiraSearchOut()
        self.out.stats = None if stats is None else stats.data_ptr()
        self.launch = searcher.launch
        self.tree = indexer.tree_struct()
        self.queue = _lib.HiraQueue(1, 1, 1, 1)  # sizes only: room for a queue's partials
        self.tau_buf: Optional[torch.Tensor] = None  # (H_q,) thresholds written by run_sampled
        self.ws_bytes = self._workspace_need()
        self.ws = torch.zeros(max(self.ws_bytes, 1), dtype=torch.uint8, device=dev)
        self._refs = (C.byref(self.tree), C.byref(self.query), C.byref(self.out),
                      C.byref(self.launch))

    def _workspace_need(self) -> int:
        fake_q = _lib.HiraQuery(self.query.num_q_heads, 1, 1, 1, 1, 1, self.query.max_group,
                                self.query.group_size)  # sizes only
        return self.lib.hira_search_workspace_bytes(
            C.byref(self.tree), C.byref(fake_q), C.byref(self.queue), C.byref(self.launch))

    def _follow_index(self) -> None:
        if self.indexer.tree_struct() is not self.tree:  # the index grew since the plan was made
            self.tree = self.indexer.tree_struct()
            need = self._workspace_need()
            if need > self.ws.numel():
                self.ws = torch.zeros(need, dtype=torch.uint8, device=self.indexer.device)
            self.ws_bytes = need
            self._refs = (C.byref(self.tree), C.byref(self.query), C.byref(self.out),
                          C.byref(self.launch))

    def run(self, query: torch.Tensor, threshold: torch.Tensor, out: torch.Tensor,
            stream: Optional[int] = None, queue_keys: Optional[torch.Tensor] = None,
            queue_values: Optional[torch.Tensor] = None, queue_len: Optional[int] = None) -> None:
        """queue_keys / queue_values: (..., cap, D) / (..., cap, Dv) contiguous, tree dtype, the
        leading dimensions amounting to T trees: keys not in the index yet, attended by every
        head of their tree; the first `queue_len` rows of every tree are in use (all `cap`
        when not given)."""
        self._follow_index()
        self.query.q = query.data_ptr()
        self.query.tau = threshold.data_ptr()
        self.out.attn_out = out.data_ptr()
        if stream is None:
            stream = _lib.current_stream(self.indexer.device)
        t, q, o, l = self._refs
        qu = None
        if queue_keys is not None and queue_keys.shape[-2] > 0 and queue_len != 0:
            cap = int(queue_keys.shape[-2])
            m = cap if queue_len is None else int(queue_len)
            if not 0 < m <= cap or queue_values.shape[-2] != cap:
                raise ValueError(f"queue: {m} rows in use of {cap} "
                                 f"(values hold {queue_values.shape[-2]})")
            self.queue = _lib.HiraQueue(queue_keys.data_ptr(), queue_values.data_ptr(), m, cap)
            qu = C.byref(self.queue)
        rc = self.lib.hira_search(t, q, qu, o, l, self.ws.data_ptr(), self.ws_bytes, stream)
        if rc:
            _lib.check(rc)

    def run_sampled(self, query: torch.Tensor, samples: torch.Tensor, method: str, k: int,
                    out: torch.Tensor, stream: Optional[int] = None,
                    queue_keys: Optional[torch.Tensor] = None,
                    queue_values: Optional[torch.Tensor] = None,
                    queue_len: Optional[int] = None, append=None) -> torch.Tensor:
        """A decode step whose thresholds come from a key sample (T, S, D), tree dtype,
        contiguous: ``hira_threshold`` ("sample_max" or "sample_mean_topk" with k) writes them
        into a buffer of the plan, ``run`` follows on the same stream.  Returns that buffer.
        ``append`` = (new_keys (T, m, D), new_values (T, m, Dv) or None, state): the step first
        appends these rows to the index (``hira_update``'s arguments), in the launch that takes
        the thresholds (``hira_update_threshold``)."""
        if self.tau_buf is None:
            self.tau_buf = torch.empty((self.query.num_q_heads,), dtype=torch.float32,
                                       device=self.indexer.device)
        if samples.ndim != 3 or samples.shape[0] != self.tree.num_trees or \
                samples.shape[2] != self.tree.dim or samples.dtype != self.indexer.dtype or \
                not samples.is_contiguous():
            raise ValueError(f"samples {tuple(samples.shape)} {samples.dtype}: expected contiguous "
                             f"({self.tree.num_trees}, S, {self.tree.dim}) {self.indexer.dtype}")
        if stream is None:
            stream = _lib.current_stream(self.indexer.device)
        self._follow_index()
        self.query.q = query.data_ptr()
        rule = 0 if method == "sample_max" else 1
        if append is not None:
            new_keys, new_values, state = append
            rc = self.lib.hira_update_threshold(
                self._refs[0], new_keys.data_ptr(),
                new_values.data_ptr() if new_values is not None else None,
                int(new_keys.shape[-2]), state.data_ptr(), samples.data_ptr(),
                int(samples.shape[1]), self._refs[1], rule, int(k), self.tau_buf.data_ptr(), stream)
        else:
            rc = self.lib.hira_threshold(
                samples.data_ptr(), self.tree.dtype, self.tree.num_trees, int(samples.shape[1]),
                self.tree.dim, self._refs[1], rule, int(k), self.tau_buf.data_ptr(), stream)
        if rc:
            _lib.check(rc)
        self.run(query, self.tau_buf, out, stream, queue_keys, queue_values, queue_len)
        return self.tau_buf


class StreamingStep:
    """One decode step over a growing index as ONE captured HIP graph: append a key/value per
    tree (``hira_update``), thresholds from a key sample (optional; then ``hira_update_threshold``
    does both in one launch), search + sparse attention (``hira_search``) -- no host work between
    the launches and no read-back.  The graph works on fixed device buffers that ``step`` fills:
    ``new_keys`` (T, 1, D), ``new_values`` (T, 1, Dv), ``query`` (H_q, D), ``threshold`` (H_q)
    and writes ``out`` (H_q, Dv).  It is good for ``horizon`` steps (the index reserves room for
    that many appends and searches with level sizes fixed at their bound); ``refresh`` reads
    the sizes back and captures anew.  The reference does the same three things per decode
    token from Python with host synchronisation in between (cache/hira_cache.py:121-153,
    indexer/cuda.py:544-701)."""

    def __init__(self, searcher: HIPSearcher, indexer, num_q_heads: int, scaling=None, *,
                 horizon: int = 512, samples: Optional[torch.Tensor] = None,
                 method: str = "sample_mean_topk", k: int = 10, q_head_to_kv=None):
        if indexer.values_buf is None:
            raise ValueError("the index holds no values: nothing to attend to")
        self.searcher, self.indexer = searcher, indexer
        self.horizon = int(horizon)
        self.samples, self.method, self.k = samples, method, int(k)
        self._args = (num_q_heads, scaling, q_head_to_kv)
        dev, t = indexer.device, indexer.num_trees
        self.new_keys = torch.zeros((t, 1, indexer.dim), dtype=indexer.dtype, device=dev)
        self.new_values = torch.zeros((t, 1, indexer.vdim), dtype=indexer.dtype, device=dev)
        self.query = torch.zeros((num_q_heads, indexer.dim), dtype=indexer.dtype, device=dev)
        self.threshold = torch.zeros((num_q_heads,), dtype=torch.float32, device=dev)
        self.out = torch.zeros((num_q_heads, indexer.vdim), dtype=torch.float32, device=dev)
        self.refresh()

    def refresh(self) -> None:
        """Exact level sizes from the device, room for another ``horizon`` appends, new capture."""
        idx = self.indexer
        idx.begin_unsynced(self.horizon)
        h_q, scaling, q2kv = self._args
        self.plan = self.searcher.plan_attention(idx, h_q, scaling=scaling, q_head_to_kv=q2kv)
        lib, tree = _lib.lib(), idx.tree_struct()
        stream = torch.cuda.Stream(device=idx.device)
        stream.wait_stream(torch.cuda.current_stream(idx.device))
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(stream):
            with torch.cuda.graph(self.graph, stream=stream):
                if self.samples is not None:
                    # the append and the thresholds share a launch
                    self.plan.tau_buf = self.threshold
                    self.plan.run_sampled(self.query, self.samples, self.method, self.k, self.out,
                                          stream=stream.cuda_stream,
                                          append=(self.new_keys, self.new_values, idx._state))
                else:
                    _lib.check(lib.hira_update(C.byref(tree), self.new_keys.data_ptr(),
                                               self.new_values.data_ptr(), 1, idx._state.data_ptr(),
                                               stream.cuda_stream))
                    self.plan.run(self.query, self.threshold, self.out, stream=stream.cuda_stream)
        torch.cuda.current_stream(idx.device).wait_stream(stream)
        self.left = self.horizon

    def step(self, new_keys: torch.Tensor, new_values: torch.Tensor, query: torch.Tensor,
             threshold: Optional[torch.Tensor] = None) -> torch.Tensor:
        """new_keys / new_values: one row per tree (any shape with T*D / T*Dv elements), query
        (H_q, D); threshold (H_q,) unless the step takes it from the key sample.  Returns
        ``out`` (the graph's buffer: copy it before the next step if it has to survive)."""
        if self.left == 0:
            self.refresh()
        self.new_keys.copy_(new_keys.reshape(self.new_keys.shape))
        self.new_values.copy_(new_values.reshape(self.new_values.shape))
        self.query.copy_(query.reshape(self.query.shape))
        if self.samples is None:
            if threshold is None:
                raise ValueError("threshold missing (the step has no key sample to take it from)")
            self.threshold.copy_(threshold.reshape(self.threshold.shape))
        return self.replay()

    def replay(self) -> torch.Tensor:
        """The step on whatever the buffers hold (for callers that write new_keys, new_values,
        query and threshold in place, e.g. as outputs of their own kernels)."""
        if self.left == 0:
            self.refresh()
        self.graph.replay()
        self.indexer.note_unsynced(1)
        self.left -= 1
        return self.out


# the class name the reference's searcher/cuda.py defines (PyTorch-ROCm calls the device "cuda")
CUDASearcher = HIPSearcher
