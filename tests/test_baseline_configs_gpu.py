"""The benchmark's own configurations as parity tests: configuration 1 at its exact shape
against the CPU oracle (selected set and attention), configuration 3 reduced (4 sequences x 8
trees x 2048 keys, a threshold per sequence) against the oracle and at full size through
properties that hold at any size, and a search on configuration 4's index after it has grown
(a grafted window, single appends, a subtree rebuild).  Shapes: hira_amd.synth.WORKLOADS;
the per-head recall checks of the reference's tests/test_cuda_pipeline.py:337-395 are the
model for the full-size cases."""
import dataclasses

import numpy as np
import pytest
import torch

from oracle import hira_oracle as ho
from helpers import assert_same_selection, band_free_heads, rel_err

pytestmark = pytest.mark.gpu


def _oracle_check(w, keys, values, q, tau, dense, attn, label):
    """keys/values (B, H_kv, n, D) host tensors in the workload dtype, q (B*H_q, D), tau (B*H_q,),
    dense (B*H_q, n) scores by position, attn (B*H_q, Dv): selected set bit-exact outside the
    1e-5 band, attention within 2e-3 (bf16) of the fp64 oracle."""
    sc = np.full(w.h_q, w.d ** -0.5, np.float32)
    worst = 0.0
    for b in range(w.batch):
        hs = slice(b * w.h_q, (b + 1) * w.h_q)
        kf, vf = keys[b].float().numpy(), values[b].float().numpy()
        qf, th = q[hs].float().cpu().numpy(), tau[hs].cpu().numpy()
        s = ho.scores(kf, qf)
        got = dense[hs].cpu().numpy() != 0
        assert_same_selection(got, s, th)
        ref = ho.attention(kf, vf, qf, sc, got)
        free = band_free_heads(s, th)
        assert free.any(), f"{label}: every head of sequence {b} has a key inside the band"
        worst = max(worst, rel_err(attn[hs].cpu().numpy()[free], ref[free]))
    assert worst <= 2e-3, f"{label}: attention off by {worst}"
    return worst


def _check_set_on_device(se, idx, q, tau, keys_b, ks, w):
    """Full-size check of the selected set, in torch on the GPU: scores of every key by fp32
    matrix products, the dense result by position; the set must be {s >= tau} outside the
    1e-5 |tau| band, so every head holds its k best keys give or take the keys inside the band.
    keys_b(b) -> (H_kv, n, D) keys of sequence b; ks[b] = keys per head of sequence b."""
    dense = se.search(q, tau, idx, index_space="position")
    for b in range(len(ks)):
        hs = slice(b * w.h_q, (b + 1) * w.h_q)
        s = torch.einsum("hnd,hgd->hgn", keys_b(b).float(),
                         q[hs].view(w.h_kv, w.group, w.d).float()).reshape(w.h_q, -1)
        th = tau[hs, None]
        got, want = dense[hs] != 0, s >= th
        band = (s - th).abs() <= 1e-5 * th.abs()
        assert not bool(((got != want) & ~band).any()), f"sequence {b}: set differs outside the band"
        assert bool(((got.sum(1) - ks[b]).abs() <= band.sum(1)).all())
        m = got & want
        assert torch.allclose(dense[hs][m], s[m], rtol=2e-5, atol=1e-6 * float(s.abs().max()))


def test_cfg1_exact_shape_against_the_oracle(gpu_device):
    """Configuration 1 as the benchmark runs it: 32 query / 8 KV heads, 8192 keys, bf16, three
    levels of fan-out 32, 2 % of the keys per head."""
    from hira_amd import synth
    from hira_amd.cache.threshold_finder import exact_topk
    from hira_amd.indexer import HIPIndexer
    from hira_amd.searcher import HIPSearcher

    w = synth.WORKLOADS[1]
    print(f"workload {w.name}", flush=True)
    keys, values = synth.make_kv(w)
    steps = 3
    queries = synth.make_queries(w, keys, steps).reshape(steps, w.h_q, w.d)
    kd, vd = keys.cuda(), values.cuda()
    idx = HIPIndexer(w.num_levels, w.kmeans_iters, w.bf).build(kd, vd)
    assert idx.tiled and idx.size == [8192, 256, 8]
    k = int(np.ceil(w.select_frac[0] * w.n))
    assert k == 164
    se = HIPSearcher(index_space="position")
    scale = torch.full((w.h_q,), w.d ** -0.5)
    for i in range(steps):
        q = queries[i].cuda()
        tau = exact_topk(kd[0], q, k)
        dense = se.search(q, tau, idx, scaling=scale).clone()
        assert bool(((dense != 0).sum(1) == k).all())
        attn = se.search_attention(q, tau, idx, scaling=scale)
        _oracle_check(w, keys, values, q, tau, dense, attn, f"cfg 1 step {i}")


def test_cfg3_reduced_per_sequence_thresholds_against_the_oracle(gpu_device):
    """Configuration 3's shape at a size the oracle walks in seconds: 4 sequences, each with its
    own keys, index and target fraction, 8 KV / 32 query heads each, 2048 keys per head -- 32
    trees and 128 heads in one launch."""
    from hira_amd import synth
    from hira_amd.cache.threshold_finder import exact_topk
    from hira_amd.indexer import HIPIndexer
    from hira_amd.searcher import HIPSearcher

    w = dataclasses.replace(synth.WORKLOADS[3], batch=4, n=2048)
    keys, values = synth.make_kv(w)
    fr = synth.select_fractions(w)
    assert len(set(fr.tolist())) == w.batch          # a fraction of its own per sequence
    q = synth.make_queries(w, keys, 1).reshape(w.batch * w.h_q, w.d).cuda()
    kd, vd = keys.cuda(), values.cuda()
    idx = HIPIndexer(w.num_levels, w.kmeans_iters, w.bf).build(kd, vd)
    assert idx.num_trees == 32 and idx.batch == 4
    ks = [int(np.ceil(float(fr[b]) * w.n)) for b in range(w.batch)]
    tau = torch.cat([exact_topk(kd[b], q[b * w.h_q:(b + 1) * w.h_q], ks[b]) for b in range(w.batch)])
    se = HIPSearcher(index_space="position")
    scale = torch.full((w.batch * w.h_q,), w.d ** -0.5)
    dense = se.search(q, tau, idx, scaling=scale).clone()
    for b in range(w.batch):
        assert bool(((dense[b * w.h_q:(b + 1) * w.h_q] != 0).sum(1) == ks[b]).all())
    attn = se.search_attention(q, tau, idx, scaling=scale)
    _oracle_check(w, keys, values, q, tau, dense, attn, "cfg 3 reduced")
    # the vector-ALU kernel on the same index: same set
    dense1 = HIPSearcher(index_space="position", kernel=1).search(q, tau, idx, scaling=scale)
    assert torch.equal(dense1 != 0, dense != 0)


def test_cfg3_full_size_properties(gpu_device):
    """Configuration 3 at its full size (16 sequences x 8 trees x 32768 keys, 512 heads in one
    launch): exactly k_b keys per head of sequence b and they are the k_b best, every key
    selected == dense attention, a repeated call repeats its result."""
    from hira_amd import synth
    from hira_amd.cache.threshold_finder import exact_topk
    from hira_amd.indexer import HIPIndexer
    from hira_amd.searcher import HIPSearcher

    w = synth.WORKLOADS[3]
    print(f"workload {w.name}", flush=True)
    keys, values = synth.make_kv(w)
    fr = synth.select_fractions(w)
    q = synth.make_queries(w, keys, 1).reshape(w.batch * w.h_q, w.d).cuda()
    kd, vd = keys.cuda(), values.cuda()
    del keys, values
    idx = HIPIndexer(w.num_levels, w.kmeans_iters, w.bf).build(kd, vd)
    assert idx.num_trees == 128
    ks = [int(np.ceil(float(fr[b]) * w.n)) for b in range(w.batch)]
    kmax = max(ks)
    tau = torch.cat([exact_topk(kd[b], q[b * w.h_q:(b + 1) * w.h_q], ks[b]) for b in range(w.batch)])
    se = HIPSearcher()
    h_all = w.batch * w.h_q
    scale = torch.full((h_all,), w.d ** -0.5)
    _check_set_on_device(se, idx, q, tau, lambda b: kd[b], ks, w)
    # the compact lists hold the same keys as the dense result
    sel_idx, sel_sco, cnt = se.search_compact(q, tau, idx, capacity=2 * kmax)
    dense = se.search(q, tau, idx)
    assert torch.equal(cnt.long(), (dense != 0).sum(1))
    a = se.search_attention(q, tau, idx, scaling=scale).clone()
    assert torch.equal(a, se.search_attention(q, tau, idx, scaling=scale))
    assert bool(torch.isfinite(a).all())
    everything = torch.full((h_all,), -3.0e38)
    dense = se.search_attention(q, everything, idx, scaling=scale)
    for b in range(w.batch):
        hs = slice(b * w.h_q, (b + 1) * w.h_q)
        ref = torch.nn.functional.scaled_dot_product_attention(
            q[hs].view(1, w.h_q, 1, w.d).float(), kd[b:b + 1].float().repeat_interleave(w.group, 1),
            vd[b:b + 1].float().repeat_interleave(w.group, 1), scale=w.d ** -0.5).reshape(w.h_q, w.d)
        err = ((dense[hs] - ref).abs().max(dim=1).values / ref.abs().max(dim=1).values).max()
        assert float(err) <= 2e-3, (b, float(err))


def test_cfg4_search_on_the_grown_index(gpu_device):
    """Configuration 4's streaming protocol, then a search: after a grafted window of 2048 keys,
    40 single appends and a subtree rebuild, the grown index (8 x 133160 keys) still selects
    exactly the k best keys of every one of the 64 heads, and attention over everything equals
    dense attention over all keys, old and new."""
    from hira_amd import synth
    from hira_amd.cache.threshold_finder import exact_topk
    from hira_amd.indexer import HIPIndexer
    from hira_amd.searcher import HIPSearcher

    w = synth.WORKLOADS[4]
    keys, values = synth.make_kv(w)
    more_k, more_v = synth.make_stream(w, 2048 + 40)
    kd, vd = keys.cuda(), values.cuda()
    mk, mv = more_k.cuda(), more_v.cuda()
    idx = HIPIndexer(w.num_levels, w.kmeans_iters, w.bf).build(kd, vd)
    idx.update(mk[:, :, :2048], mv[:, :, :2048])
    for i in range(2048, 2088):
        idx.update(mk[:, :, i:i + 1], mv[:, :, i:i + 1], sync=False)
    idx.rebuild_subtree(3)
    n_all = w.n + 2088
    assert idx.num_keys == n_all
    k_all, v_all = torch.cat([kd, mk], dim=2), torch.cat([vd, mv], dim=2)
    q = synth.make_queries(w, k_all.cpu(), 2, seed=5).reshape(2, w.h_q, w.d).cuda()
    k = int(np.ceil(0.01 * n_all))
    se = HIPSearcher()
    scale = torch.full((w.h_q,), w.d ** -0.5)
    for i in range(2):
        tau = exact_topk(k_all[0], q[i], k)
        _check_set_on_device(se, idx, q[i], tau, lambda b: k_all[0], [k], w)
        a = se.search_attention(q[i], tau, idx, scaling=scale).clone()
        assert torch.equal(a, se.search_attention(q[i], tau, idx, scaling=scale))
    dense = se.search_attention(q[0], torch.full((w.h_q,), -3.0e38), idx, scaling=scale)
    ref = torch.nn.functional.scaled_dot_product_attention(
        q[0].view(1, w.h_q, 1, w.d).float(), k_all.float().repeat_interleave(w.group, 1),
        v_all.float().repeat_interleave(w.group, 1), scale=w.d ** -0.5).reshape(w.h_q, w.d)
    err = ((dense - ref).abs().max(dim=1).values / ref.abs().max(dim=1).values).max()
    assert float(err) <= 2e-3, float(err)


def test_captured_keys_file_replayed_against_the_oracle(gpu_device, tmp_path):
    """A capture in the reference sampler's file format (an .npz with keys (N, D) and queries
    (N, D), benchmark_area/kv_sampling/collect_kv_data.py:393-397) is loaded by
    synth.load_capture, indexed and searched; the result is compared with the oracle.  (No real
    capture ships with the reference; this one is synthetic and anisotropic.)"""
    from hira_amd import synth
    from hira_amd.cache.threshold_finder import exact_topk
    from hira_amd.indexer import HIPIndexer
    from hira_amd.searcher import HIPSearcher

    rng = np.random.default_rng(7)
    d, trees_keys = 128, 8 * 1500
    basis = rng.normal(size=(d, d)).astype(np.float32) * np.exp(rng.normal(size=d) * 0.7).astype(np.float32)
    pool_k = (rng.normal(size=(trees_keys, d)).astype(np.float32) @ basis) / np.sqrt(d)
    pool_q = pool_k[rng.integers(0, trees_keys, 300)] + 0.3 * rng.normal(size=(300, d)).astype(np.float32)
    path = tmp_path / "capture.npz"
    np.savez(path, keys=pool_k, queries=pool_q)
    w0 = synth.WORKLOADS[1]
    w, keys, values, queries = synth.load_capture(str(path), w0, 2)
    assert w.n == 1500 and keys.shape == (1, 8, 1500, d) and queries.shape == (2, 1, 32, d)
    kd, vd = keys.cuda(), values.cuda()
    idx = HIPIndexer(w.num_levels, w.kmeans_iters, w.bf).build(kd, vd)
    se = HIPSearcher(index_space="position")
    scale = torch.full((w.h_q,), d ** -0.5)
    for i in range(2):
        q = queries[i, 0].cuda()
        tau = exact_topk(kd[0], q, 30)
        dense = se.search(q, tau, idx, scaling=scale).clone()
        attn = se.search_attention(q, tau, idx, scaling=scale)
        _oracle_check(w, keys, values, q, tau, dense, attn, f"capture step {i}")
