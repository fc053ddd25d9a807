"""GPU tests of the append path (hira_update through HIPIndexer.update): every key present
exactly once, counts and radii stay valid bounds, search after update == brute force
(tests/test_cuda_indexer_searcher.py:205-262, 594-607 and tests/test_cuda_pipeline.py:215-226
of the reference)."""
import numpy as np
import pytest
import torch

from oracle import hira_oracle as ho
from helpers import (assert_same_selection, bf16_round, clustered_keys, midpoint_threshold,
                     random_query, rel_err)

pytestmark = pytest.mark.gpu


def _check_tree(idx, keys_all, vals_all):
    """Structure after updates: perm is a permutation of the inserted positions, rows follow
    their slot, children packed from slot 0, every radius covers its subtree."""
    t, n, d = keys_all.shape
    bf, nl = idx.branching_factor, idx.num_levels
    kr = idx.keys_rowmajor().float().cpu().numpy()
    perm = idx.perm[:, : idx.size[0]].cpu().numpy().astype(np.int64)
    vals = idx.values_buf[:, : idx.size[0]].float().cpu().numpy()
    for h in range(t):
        ok = perm[h] >= 0
        assert np.array_equal(np.sort(perm[h][ok]), np.arange(n))
        assert np.array_equal(kr[h][ok], keys_all[h][perm[h][ok]])
        assert np.array_equal(vals[h][ok], vals_all[h][perm[h][ok]])
        if nl == 1:
            continue
        child_c, child_r, child_ok = kr[h], np.zeros(idx.size[0], np.float32), ok
        for l in range(1, nl):
            k = idx.size[l]
            cen = idx.centers_rowmajor(l)[h].float().cpu().numpy()
            rad = idx.radii[l][h, :k].cpu().numpy()
            cnt = idx.counts[l][h, :k].cpu().numpy()
            short = k * bf - len(child_ok)      # slots past the level's size are absent
            if short > 0:
                child_c = np.concatenate([child_c, np.zeros((short, d), np.float32)])
                child_r = np.concatenate([child_r, np.zeros(short, np.float32)])
                child_ok = np.concatenate([child_ok, np.zeros(short, bool)])
            blk = child_ok[: k * bf].reshape(k, bf)
            assert np.array_equal(cnt, blk.sum(1)), f"counts level {l}"
            assert np.all(blk[:, :-1] >= blk[:, 1:])
            need = ho.radii_from_layout(child_c[: k * bf], child_r[: k * bf], child_ok[: k * bf], cen, bf)
            has = cnt > 0
            assert np.all(rad[has] >= need[has] * (1 - 1e-6) - 1e-6), f"radius level {l}"
            child_c, child_r, child_ok = cen, np.where(has, rad, 0).astype(np.float32), has


UPDATE_CASES = [
    # trees, n0, appended chunks, d, bf, levels, dtype
    (2, 128, [1, 1, 1, 7, 64, 30], 32, 8, 3, torch.float32),
    (2, 2048, [1] * 40 + [64, 500], 128, 32, 3, torch.bfloat16),    # tiled, full blocks at build
    (1, 1000, [33, 1, 1, 200], 64, 16, 4, torch.bfloat16),          # pad slots inside blocks
    (3, 50, [5, 5, 100], 64, 4, 2, torch.float32),
    (2, 40, [1, 2, 3, 50], 32, 8, 1, torch.float32),                # one level: plain append
    (1, 64, [1] * 70, 128, 32, 4, torch.bfloat16),                  # tree smaller than a block
    # large windows are clustered among themselves and grafted at the tail, small ones in between
    (2, 3000, [600, 1, 1, 1100, 5, 2048, 3], 128, 32, 3, torch.bfloat16),
    (2, 500, [300, 3, 700, 1], 32, 8, 3, torch.float32),
    (1, 400, [260, 1, 1, 256], 64, 16, 2, torch.bfloat16),
    (3, 100, [256, 2], 64, 16, 4, torch.bfloat16),                  # fits under the only root
    # mid-size windows become further children of the last root while it has room
    (2, 5000, [600, 3, 300, 2100, 400, 1, 3000, 5], 64, 16, 4, torch.bfloat16),
    (2, 3000, [300, 2, 600, 260, 1, 270, 280, 290], 128, 32, 3, torch.bfloat16),
    (2, 900, [260, 1, 300], 32, 16, 3, torch.float32),
]


@pytest.mark.parametrize("case", UPDATE_CASES, ids=[f"t{c[0]}_n{c[1]}_m{sum(c[2])}_d{c[3]}_bf{c[4]}_L{c[5]}_"
                                                      f"{'bf16' if c[6] == torch.bfloat16 else 'f32'}"
                                                      for c in UPDATE_CASES])
def test_update_keeps_tree_valid_and_search_exact(case, gpu_device):
    from hira_amd.indexer.hip import HIPIndexer
    from hira_amd.searcher.hip import HIPSearcher

    t, n0, chunks, d, bf, nl, dtype = case
    print(f"case {case}", flush=True)
    n = n0 + sum(chunks)
    rnd = bf16_round if dtype == torch.bfloat16 else (lambda x: x)
    keys = rnd(clustered_keys(t, n, d, seed=17 + n, clusters=max(2, n // 50)))
    vals = rnd(np.random.default_rng(n).normal(size=(t, n, d)).astype(np.float32))
    K, V = torch.from_numpy(keys)[None].to(dtype), torch.from_numpy(vals)[None].to(dtype)
    idx = HIPIndexer(nl, 1, bf).build(K[:, :, :n0], V[:, :, :n0])
    searcher = HIPSearcher(index_space="position")
    h_q = 2 * t
    q2kv = ho.default_q2kv(h_q, t)
    at = n0
    for ci, m in enumerate(chunks):
        ret = idx.update(K[:, :, at:at + m], V[:, :, at:at + m])
        assert ret is idx
        at += m
        if ci % 7 and m == 1 and ci < len(chunks) - 1:
            continue  # check after some of the single-key steps only
        assert idx.num_keys == at
        _check_tree(idx, keys[:, :at], vals[:, :at])
        q = rnd(random_query(h_q, d, seed=at))
        s = ho.scores(keys[:, :at], q, q2kv)
        th = midpoint_threshold(s, max(1, at // 20))
        out = searcher.search(torch.from_numpy(q), torch.from_numpy(th), idx).cpu().numpy()
        assert out.shape == (h_q, at)
        assert_same_selection(out != 0, s, th)
    # attention over the final index
    sc = torch.full((h_q,), d ** -0.5)
    att = HIPSearcher().search_attention(torch.from_numpy(q), torch.from_numpy(th), idx,
                                         scaling=sc).cpu().numpy()
    ref = ho.attention(keys, vals, q, sc.numpy(), s >= th[:, None], q2kv)
    assert rel_err(att, ref) <= (2e-3 if dtype == torch.bfloat16 else 1e-5)


@pytest.mark.parametrize("dtype,d,bf", [(torch.bfloat16, 128, 16), (torch.float32, 32, 8)])
def test_rebuild_subtree_after_appends(dtype, d, bf, gpu_device):
    """Appends loosen the balls of the nodes they land in; rebuilding a level-2 subtree
    re-clusters its keys in place: the tree stays valid, nothing is lost, search is exact,
    and the rebuilt level-1 balls are no larger on average than before."""
    from hira_amd.indexer.hip import HIPIndexer
    from hira_amd.searcher.hip import HIPSearcher

    t, n0, m = 2, bf * bf * 3, bf * bf // 2
    n = n0 + m
    rnd = bf16_round if dtype == torch.bfloat16 else (lambda x: x)
    keys = rnd(clustered_keys(t, n, d, seed=5, clusters=12))
    vals = rnd(np.random.default_rng(1).normal(size=(t, n, d)).astype(np.float32))
    K, V = torch.from_numpy(keys)[None].to(dtype), torch.from_numpy(vals)[None].to(dtype)
    idx = HIPIndexer(3, 2, bf).build(K[:, :, :n0 - m], V[:, :, :n0 - m])
    idx.update(K[:, :, n0 - m:], V[:, :, n0 - m:])
    _check_tree(idx, keys, vals)
    before = [idx.radii[1][:, : idx.size[1]].clone()]
    for node in range(idx.size[2]):
        idx.rebuild_subtree(node)
    assert idx.num_keys == n
    _check_tree(idx, keys, vals)
    r0, r1 = before[0], idx.radii[1][:, : idx.size[1]]
    assert float(r1[r1 > -1e30].mean()) <= float(r0[r0 > -1e30].mean()) * 1.05
    q = rnd(random_query(2 * t, d, seed=3))
    q2kv = ho.default_q2kv(2 * t, t)
    s = ho.scores(keys, q, q2kv)
    th = midpoint_threshold(s, n // 20)
    out = HIPSearcher(index_space="position").search(torch.from_numpy(q), torch.from_numpy(th), idx)
    assert_same_selection(out.cpu().numpy() != 0, s, th)
    # and the index keeps taking appends afterwards
    extra = rnd(clustered_keys(t, 40, d, seed=6, clusters=3))
    idx.update(torch.from_numpy(extra)[None].to(dtype), torch.from_numpy(extra)[None].to(dtype))
    _check_tree(idx, np.concatenate([keys, extra], 1), np.concatenate([vals, extra], 1))
    with pytest.raises(ValueError):
        idx.rebuild_subtree(idx.size[2])


def test_update_is_reproducible_and_grows_capacity(gpu_device):
    from hira_amd.indexer.hip import HIPIndexer

    keys = torch.from_numpy(clustered_keys(2, 600, 64, seed=2))[None]
    a = HIPIndexer(3, 1, 8).build(keys[:, :, :256])
    b = HIPIndexer(3, 1, 8, capacity=4096).build(keys[:, :, :256])
    cap0 = list(a.cap)
    for lo in range(256, 600, 43):
        a.update(keys[:, :, lo:lo + 43])
        b.update(keys[:, :, lo:lo + 43])
    assert a.cap[0] > cap0[0] and a.size == b.size and a.num_keys == b.num_keys == 600
    n0 = a.size[0]
    assert torch.equal(a.perm[:, :n0], b.perm[:, :n0])
    assert torch.equal(a.keys_buf[:, :n0], b.keys_buf[:, :n0])
    for l in (1, 2):
        assert torch.equal(a.radii[l][:, : a.size[l]], b.radii[l][:, : a.size[l]])


def test_update_rejects_bad_shapes(gpu_device):
    """tests/test_cuda_indexer_searcher.py:594-607 of the reference."""
    from hira_amd.indexer.hip import HIPIndexer

    keys = torch.from_numpy(clustered_keys(2, 128, 32, seed=61))[None]
    idx = HIPIndexer(3, 2, 8).build(keys)
    with pytest.raises(ValueError):
        idx.update(torch.randn(2, 2, 7, 32))          # batch 2 on a batch-1 index
    with pytest.raises(ValueError):
        idx.update(torch.randn(1, 2, 7, 16))          # wrong dim
    with pytest.raises(ValueError):
        idx.update(torch.randn(1, 2, 7, 32), torch.randn(1, 2, 7, 32))  # built without values
    with pytest.raises(ValueError):
        HIPIndexer(3, 2, 8).update(torch.randn(1, 2, 7, 32))            # not built


def test_cache_layer_end_to_end(gpu_device):
    """Prefill builds, decode steps queue and flush into the index, the attention function
    reads the CacheOutput: output == dense softmax attention when every key is selected."""
    from hira_amd.attention import hira_attention_forward
    from hira_amd.cache.hira_cache import HiraCacheLayer
    from hira_amd.cache.hira_config import DeviceMode, HiraConfig

    cfg = HiraConfig(device_mode=DeviceMode.CUDA_ONLY, update_every=4, num_levels=3,
                     branching_factor=16, max_iterations=1)
    layer = HiraCacheLayer(cfg.device_mode, cfg.update_every, cfg.get_indexer_kwargs(),
                           cfg.get_searcher_kwargs())
    g = torch.Generator().manual_seed(0)
    h_kv, h_q, d, n0 = 2, 4, 64, 300
    dev = "cuda"
    K = torch.randn((1, h_kv, n0 + 10, d), generator=g).to(torch.bfloat16).to(dev)
    V = torch.randn((1, h_kv, n0 + 10, d), generator=g).to(torch.bfloat16).to(dev)
    out, _ = layer.update(K[:, :, :n0], V[:, :, :n0])
    assert out.prefill_keys is not None
    for step in range(10):
        out, _ = layer.update(K[:, :, n0 + step:n0 + step + 1], V[:, :, n0 + step:n0 + step + 1])
        n = n0 + step + 1
        assert layer.get_seq_length() == n
        assert out.queued_keys.shape[-2] == (step + 1) % 4
        q = torch.randn((1, h_q, 1, d), generator=g).to(torch.bfloat16).to(dev)
        att, _ = hira_attention_forward(None, q, out, None, scaling=d ** -0.5, hira_threshold=-3e38)
        assert att.shape == (1, 1, h_q, d)
        kk = K[:, :, :n].float().repeat_interleave(h_q // h_kv, 1)
        vv = V[:, :, :n].float().repeat_interleave(h_q // h_kv, 1)
        ref = torch.nn.functional.scaled_dot_product_attention(q.float(), kk, vv, scale=d ** -0.5)
        err = (att.float().transpose(1, 2) - ref).abs().max() / ref.abs().max()
        # 2e-3 for the attention itself plus the rounding of the returned tensor to bf16 (half a
        # unit in the last place of the largest component: 2^-9, at most twice that below it)
        assert float(err) <= 2e-3 + 2.0 ** -8, float(err)


def test_decode_plan_survives_updates_and_queue_changes(gpu_device):
    """One DecodePlan (one workspace) reused while the tree grows and a queue comes and goes
    gives the same output as a fresh call with a fresh workspace each time."""
    from hira_amd.indexer.hip import HIPIndexer
    from hira_amd.searcher.hip import HIPSearcher

    t, h_q, d, bf, n0 = 2, 8, 128, 32, 3000
    keys = bf16_round(clustered_keys(t, n0 + 2200, d, seed=9, clusters=40))
    K = torch.from_numpy(keys)[None].to(torch.bfloat16)
    idx = HIPIndexer(3, 1, bf).build(K[:, :, :n0], K[:, :, :n0])
    searcher = HIPSearcher()
    scale = torch.full((h_q,), d ** -0.5)
    plan = searcher.plan_attention(idx, h_q, scaling=scale)
    q2kv = ho.default_q2kv(h_q, t)
    at = n0
    out = torch.empty((h_q, d), dtype=torch.float32, device="cuda")
    # appends of 1..1100 keys change the number of level-1 tiles (and so the partials per head);
    # queues of 0..3 keys add or drop the queue's partial
    for step, (m, qlen) in enumerate([(0, 0), (1, 2), (0, 0), (1100, 3), (0, 1), (1000, 0), (5, 2), (0, 0)]):
        print(f"step {step} append {m} queue {qlen}", flush=True)
        if m:
            idx.update(K[:, :, at:at + m], K[:, :, at:at + m])
            at += m
        q = bf16_round(random_query(h_q, d, seed=100 + step))
        s = ho.scores(keys[:, :at], q, q2kv)
        th = torch.from_numpy(midpoint_threshold(s, max(1, at // 30))).cuda()
        qd = torch.from_numpy(q).to(torch.bfloat16).cuda()
        qk = K[0, :, at:at + qlen].contiguous().cuda() if qlen else None
        plan.run(qd, th, out, queue_keys=qk, queue_values=qk)
        ref = searcher.search_attention(qd, th, idx, scaling=scale, queue_keys=qk, queue_values=qk)
        assert rel_err(out.cpu().numpy(), ref.cpu().numpy()) <= 1e-6, step


@pytest.mark.parametrize("dtype,d,bf,nl", [(torch.bfloat16, 128, 32, 3), (torch.float32, 32, 8, 4),
                                           (torch.float32, 16, 4, 1)])
def test_save_load_roundtrip(dtype, d, bf, nl, gpu_device, tmp_path):
    """An index that took appends, written to a file and read back: every array equal, the
    same search result, and the same tree after further appends as the index that never
    left the device."""
    from hira_amd.indexer.hip import HIPIndexer
    from hira_amd.searcher.hip import HIPSearcher

    t, n0, m1, m2 = 2, 700, 150, 90
    n = n0 + m1 + m2
    rnd = bf16_round if dtype == torch.bfloat16 else (lambda x: x)
    keys = rnd(clustered_keys(t, n, d, seed=21, clusters=14))
    K = torch.from_numpy(keys)[None].to(dtype)
    a = HIPIndexer(nl, 1, bf).build(K[:, :, :n0], K[:, :, :n0])
    a.update(K[:, :, n0:n0 + m1], K[:, :, n0:n0 + m1])
    path = str(tmp_path / "index.safetensors")
    a.save(path)
    b = HIPIndexer.load(path)
    assert (b.size, b.num_keys, b.tiled, b.dtype) == (a.size, a.num_keys, a.tiled, a.dtype)

    def same(x, y):
        s0 = a.size[0]
        assert torch.equal(x.perm[:, :s0], y.perm[:, :s0])
        assert torch.equal(x.keys_rowmajor()[:, :s0], y.keys_rowmajor()[:, :s0])
        assert torch.equal(x.values_buf[:, :s0], y.values_buf[:, :s0])
        for l in range(1, nl):
            k = x.size[l]
            assert torch.equal(x.centers_rowmajor(l)[:, :k], y.centers_rowmajor(l)[:, :k])
            assert torch.equal(x.radii[l][:, :k], y.radii[l][:, :k])
            assert torch.equal(x.counts[l][:, :k], y.counts[l][:, :k])

    same(a, b)
    q = rnd(random_query(2 * t, d, seed=3))
    q2kv = ho.default_q2kv(2 * t, t)
    s = ho.scores(keys[:, :n0 + m1], q, q2kv)
    th = midpoint_threshold(s, 40)
    se = HIPSearcher(index_space="position")
    out_a = se.search(torch.from_numpy(q), torch.from_numpy(th), a).clone()
    out_b = se.search(torch.from_numpy(q), torch.from_numpy(th), b)
    assert torch.equal(out_a, out_b)
    assert_same_selection(out_b.cpu().numpy() != 0, s, th)
    a.update(K[:, :, n0 + m1:], K[:, :, n0 + m1:])
    b.update(K[:, :, n0 + m1:], K[:, :, n0 + m1:])
    assert a.size == b.size and a.num_keys == b.num_keys == n
    same(a, b)
    _check_tree(b, keys, keys)
    with pytest.raises(ValueError):
        HIPIndexer(3, 1, 8).save(path)          # not built
    from safetensors.torch import save_file
    save_file({"x": torch.zeros(1)}, str(tmp_path / "other.safetensors"))
    with pytest.raises(ValueError):
        HIPIndexer.load(str(tmp_path / "other.safetensors"))


@pytest.mark.parametrize("sampled", [False, True])
def test_streaming_step_graph_matches_eager_updates(sampled, gpu_device):
    """update + (thresholds) + search + attention captured as one graph and replayed once per
    token == the same calls made one by one with the level sizes read back after each update;
    afterwards both indexes hold the same tree."""
    from hira_amd.cache import threshold_finder as tf
    from hira_amd.indexer.hip import HIPIndexer
    from hira_amd.searcher.hip import HIPSearcher, StreamingStep

    t, h_q, d, bf, n0, steps = 2, 8, 128, 32, 4000, 70
    keys = bf16_round(clustered_keys(t, n0 + steps, d, seed=31, clusters=40))
    K = torch.from_numpy(keys)[None].to(torch.bfloat16).cuda()
    a = HIPIndexer(3, 1, bf).build(K[:, :, :n0], K[:, :, :n0])
    b = HIPIndexer(3, 1, bf).build(K[:, :, :n0], K[:, :, :n0])
    se = HIPSearcher()
    scale = torch.full((h_q,), d ** -0.5)
    samples = K[0][:, ::8][:, :400].contiguous() if sampled else None
    step = StreamingStep(se, b, h_q, scale, horizon=32, samples=samples, method="sample_mean_topk", k=6)
    q2kv = ho.default_q2kv(h_q, t)
    for i in range(steps):
        if i % 10 == 0:
            print(f"token {i}", flush=True)
        nk = K[:, :, n0 + i:n0 + i + 1]
        q = bf16_round(random_query(h_q, d, seed=500 + i))
        qd = torch.from_numpy(q).to(torch.bfloat16).cuda()
        a.update(nk, nk)
        if sampled:
            th = tf.sample_mean_topk(samples, qd, 6)
        else:
            s = ho.scores(keys[:, :n0 + i + 1], q, q2kv)
            th = torch.from_numpy(midpoint_threshold(s, 60)).cuda()
        want = se.search_attention(qd, th, a, scaling=scale)
        got = step.step(nk, nk, qd, None if sampled else th)
        assert rel_err(got.cpu().numpy(), want.cpu().numpy()) <= 1e-5, i
        assert b.num_keys == a.num_keys
    assert step.left == 32 * 3 - steps          # two refreshes on the way
    b.sync_sizes()
    assert a.size == b.size
    s0 = a.size[0]
    assert torch.equal(a.perm[:, :s0], b.perm[:, :s0])
    for l in (1, 2):
        assert torch.equal(a.counts[l][:, : a.size[l]], b.counts[l][:, : a.size[l]])
        assert torch.equal(a.radii[l][:, : a.size[l]], b.radii[l][:, : a.size[l]])
    _check_tree(b, keys, keys)


def test_unsynced_updates_keep_search_exact(gpu_device):
    """update(sync=False): the host only knows bounds of the level sizes, the search result is
    the same; sync_sizes brings the exact sizes back."""
    from hira_amd.indexer.hip import HIPIndexer
    from hira_amd.searcher.hip import HIPSearcher

    t, d, bf, n0 = 2, 64, 16, 1000
    chunks = [1, 1, 40, 1, 300, 7]
    n = n0 + sum(chunks)
    keys = clustered_keys(t, n, d, seed=77, clusters=25)
    K = torch.from_numpy(keys)[None]
    a = HIPIndexer(3, 1, bf).build(K[:, :, :n0])
    b = HIPIndexer(3, 1, bf).build(K[:, :, :n0])
    se = HIPSearcher(index_space="position")
    q = random_query(2 * t, d, seed=9)
    q2kv = ho.default_q2kv(2 * t, t)
    at = n0
    for m in chunks:
        a.update(K[:, :, at:at + m])
        b.update(K[:, :, at:at + m], sync=False)
        at += m
        assert b.num_keys == a.num_keys and all(x >= y for x, y in zip(b.size, a.size))
        s = ho.scores(keys[:, :at], q, q2kv)
        th = midpoint_threshold(s, at // 25)
        out = se.search(torch.from_numpy(q), torch.from_numpy(th), b)
        assert_same_selection(out.cpu().numpy()[:, :at] != 0, s, th)
    b.sync_sizes()
    assert b.size == a.size
    with pytest.raises(ValueError):
        HIPIndexer(1, 1, bf).build(K[:, :, :n0]).update(K[:, :, n0:n0 + 1], sync=False)


def test_updates_inside_an_open_unsynced_stretch(gpu_device):
    """begin_unsynced(M) then update(sync=False) calls: the sizes of the last read-back stay the
    base of the capacity bound (so the bound does not creep up call by call), the stretch's room
    is debited, an append beyond it is refused, and the index stays valid and exact."""
    from hira_amd.indexer.hip import HIPIndexer
    from hira_amd.searcher.hip import HIPSearcher

    t, d, bf, n0 = 2, 64, 16, 600
    keys = clustered_keys(t, n0 + 40, d, seed=5, clusters=12)
    K = torch.from_numpy(keys)[None]
    idx = HIPIndexer(3, 1, bf).build(K[:, :, :n0], K[:, :, :n0])
    exact = list(idx.size)
    idx.begin_unsynced(8)
    held, caps = list(idx.size), list(idx.cap)
    assert idx._exact_size == exact and idx._unsynced_room == 8
    at = n0
    for m in (3, 3):
        idx.update(K[:, :, at:at + m], K[:, :, at:at + m], sync=False)
        at += m
        assert idx._exact_size == exact              # not overwritten by the bounds
        assert idx.size == held and idx.cap == caps  # bounds and pointers of the stretch hold
    assert idx._unsynced_room == 2 and idx._pending == 6
    with pytest.raises(RuntimeError):
        idx.update(K[:, :, at:at + 3], K[:, :, at:at + 3], sync=False)
    idx.sync_sizes()
    assert idx._exact_size is None and idx._pending == 0 and idx.num_keys == at
    _check_tree(idx, keys[:, :at], keys[:, :at])
    q = random_query(t, d, seed=3)
    s = ho.scores(keys[:, :at], q, ho.default_q2kv(t, t))
    th = midpoint_threshold(s, 20)
    out = HIPSearcher(index_space="position").search(torch.from_numpy(q), torch.from_numpy(th), idx)
    assert_same_selection(out.cpu().numpy()[:, :at] != 0, s, th)


@pytest.mark.parametrize("t,n0,m,d,bf,nl,dtype,layout", [
    (2, 2048, 100, 128, 32, 3, torch.bfloat16, "auto"),   # every node full: a node opens every 32 keys
    (2, 2048, 255, 128, 32, 4, torch.bfloat16, "q8"),     # with the 8-bit shadow, 4 levels
    (3, 1000, 70, 64, 16, 3, torch.bfloat16, "auto"),     # free slots here and there
    (2, 5000, 130, 32, 8, 3, torch.float32, "auto"),      # fp32 rows; more nodes with room than the list holds
    (1, 300, 40, 256, 16, 2, torch.float32, "auto"),      # wide rows (a short chunk), two levels
])
def test_a_window_placed_at_once_equals_key_by_key(t, n0, m, d, bf, nl, dtype, layout, gpu_device):
    """update() with a window of several keys (the kernel that reads the nodes with room into LDS
    once and places key after key from there) against the same keys appended one call each (the
    general kernel): the same slots, counts, centres and radii bit for bit, and a valid tree."""
    from hira_amd.indexer.hip import HIPIndexer

    keys = clustered_keys(t, n0 + m + 7, d, seed=31 + m, clusters=20)
    if dtype == torch.bfloat16:
        keys = bf16_round(keys)
    K = torch.from_numpy(keys)[None].to(dtype)
    mk = lambda: HIPIndexer(nl, 1, bf, layout=layout, graft_min=1 << 30).build(K[:, :, :n0], K[:, :, :n0])
    a, b = mk(), mk()
    a.update(K[:, :, n0:n0 + m], K[:, :, n0:n0 + m])
    for i in range(m):
        b.update(K[:, :, n0 + i:n0 + i + 1], K[:, :, n0 + i:n0 + i + 1])
    # and a second, short window on top (the list is read anew)
    a.update(K[:, :, n0 + m:n0 + m + 7], K[:, :, n0 + m:n0 + m + 7])
    for i in range(m, m + 7):
        b.update(K[:, :, n0 + i:n0 + i + 1], K[:, :, n0 + i:n0 + i + 1])
    assert a.size == b.size and a.num_keys == b.num_keys == n0 + m + 7
    n = a.size[0]
    assert torch.equal(a.perm[:, :n], b.perm[:, :n])
    assert torch.equal(a.keys_buf[:, :a.cap[0]], b.keys_buf[:, :b.cap[0]])
    assert torch.equal(a.values_buf[:, :n], b.values_buf[:, :n])
    for l in range(1, nl):
        k = a.size[l]
        assert torch.equal(a.counts[l][:, :k], b.counts[l][:, :k]), f"counts level {l}"
        assert torch.equal(a.radii[l][:, :k], b.radii[l][:, :k]), f"radii level {l}"
        assert torch.equal(a.centers[l][:, :a.cap[l]], b.centers[l][:, :b.cap[l]]), f"centres level {l}"
    if layout == "q8":
        assert torch.equal(a.keys8, b.keys8) and torch.equal(a.keps[:, :a.size[1]], b.keps[:, :b.size[1]])
    _check_tree(a, keys[:, :n0 + m + 7], keys[:, :n0 + m + 7])


@pytest.mark.parametrize("dtype,d,m,s,method,k", [
    (torch.bfloat16, 128, 1, 400, 1, 6),     # a key per tree, few of up to 1024 samples
    (torch.bfloat16, 128, 3, 1500, 1, 40),   # three keys, the sort with two registers a thread
    (torch.bfloat16, 64, 2, 3000, 0, 1),     # the maximum of 3000 samples
    (torch.float32, 128, 1, 700, 1, 20),
    (torch.float32, 32, 3, 2500, 1, 300),    # four registers a thread
    (torch.bfloat16, 128, 6, 400, 1, 6),     # a window: served by the two launches
    (torch.bfloat16, 128, 0, 400, 1, 6),     # nothing to append
])
def test_append_and_thresholds_in_one_launch_equal_the_two_calls(dtype, d, m, s, method, k, gpu_device):
    """hira_update_threshold == hira_update followed by hira_threshold, bit for bit: the
    thresholds, the update state and every array of the tree, over several calls in a row."""
    import ctypes as C

    from hira_amd import _lib
    from hira_amd.indexer.hip import HIPIndexer
    from hira_amd.searcher.hip import HIPSearcher

    t, h_q, bf, n0, calls = 3, 12, 8, 3200, 40
    rnd = bf16_round if dtype == torch.bfloat16 else (lambda x: x)
    keys = rnd(clustered_keys(t, n0 + calls * max(m, 1), d, seed=77, clusters=30))
    K = torch.from_numpy(keys)[None].to(dtype).cuda()
    a = HIPIndexer(3, 1, bf).build(K[:, :, :n0], K[:, :, :n0])
    b = HIPIndexer(3, 1, bf).build(K[:, :, :n0], K[:, :, :n0])
    se = HIPSearcher()
    plans = [se.plan_attention(i, h_q, scaling=torch.full((h_q,), d ** -0.5)) for i in (a, b)]
    for i in (a, b):
        i.begin_unsynced(calls * max(m, 1))
    samples = K[0][:, torch.randperm(n0, generator=torch.Generator().manual_seed(5))[:s].sort().values]
    samples = samples.contiguous()
    assert samples.shape == (t, s, d)
    lib = _lib.lib()
    stream = _lib.current_stream(a.device)
    tau_a = torch.zeros(h_q, dtype=torch.float32, device="cuda")
    tau_b = torch.zeros_like(tau_a)
    for c in range(calls):
        # (m = 0: a buffer that is not read, since the calls refuse a null pointer)
        nk = K[0][:, n0 + c * m:n0 + (c + 1) * m].contiguous() if m else K[0][:, :1].contiguous()
        q = torch.from_numpy(rnd(random_query(h_q, d, seed=900 + c))).to(dtype).cuda()
        for p in plans:
            p.query.q = q.data_ptr()
        ta, tb = a.tree_struct(), b.tree_struct()
        _lib.check(lib.hira_update(C.byref(ta), nk.data_ptr(), nk.data_ptr(), m, a._state.data_ptr(), stream))
        _lib.check(lib.hira_threshold(samples.data_ptr(), ta.dtype, t, s, d, C.byref(plans[0].query),
                                      method, k, tau_a.data_ptr(), stream))
        _lib.check(lib.hira_update_threshold(C.byref(tb), nk.data_ptr(), nk.data_ptr(), m,
                                             b._state.data_ptr(), samples.data_ptr(), s,
                                             C.byref(plans[1].query), method, k, tau_b.data_ptr(), stream))
        a.note_unsynced(m)
        b.note_unsynced(m)
        assert torch.equal(tau_a, tau_b), c
        assert torch.equal(a._state, b._state), c
    a.sync_sizes()
    b.sync_sizes()
    assert a.size == b.size and a.num_keys == b.num_keys == n0 + calls * m
    s0 = a.size[0]
    assert torch.equal(a.perm[:, :s0], b.perm[:, :s0])
    held = a.perm[:, :s0] >= 0
    assert torch.equal(a.keys_rowmajor()[held], b.keys_rowmajor()[held])
    assert torch.equal(a.values_buf[:, :s0][held], b.values_buf[:, :s0][held])
    for l in (1, 2):
        assert torch.equal(a.counts[l][:, : a.size[l]], b.counts[l][:, : a.size[l]])
        assert torch.equal(a.radii[l][:, : a.size[l]], b.radii[l][:, : a.size[l]])
    _check_tree(b, keys[:, :b.num_keys], keys[:, :b.num_keys])
    # the thresholds themselves: the two rules on the same sample, in fp64
    sc = np.einsum("hd,hsd->hs", q.float().cpu().numpy().astype(np.float64),
                   samples.float().cpu().numpy().astype(np.float64)[ho.default_q2kv(h_q, t)])
    want = sc.max(1) if method == 0 else np.sort(sc, 1)[:, ::-1][:, :k].mean(1)
    np.testing.assert_allclose(tau_b.cpu().numpy(), want, rtol=2e-5, atol=1e-5)


@pytest.mark.parametrize("dtype,d,bf,nl,layout", [
    (torch.float32, 32, 8, 2, "auto"),
    (torch.bfloat16, 128, 16, 3, "auto"),
    (torch.bfloat16, 64, 16, 4, "q8"),
    (torch.float32, 16, 5, 3, "auto"),
])
def test_warm_up_runs_the_first_use_paths_and_leaves_the_index_alone(dtype, d, bf, nl, layout, gpu_device):
    """warm_up runs an append, a window, a grafted window and a subtree rebuild on a throw-away
    index of the same kind; the index it was called on keeps every array, and appends to it
    afterwards behave as without the call."""
    from hira_amd.indexer.hip import HIPIndexer

    t, n = 2, 700
    rnd = bf16_round if dtype == torch.bfloat16 else (lambda x: x)
    keys = rnd(clustered_keys(t, n + 40, d, seed=3, clusters=12))
    K = torch.from_numpy(keys)[None].to(dtype).cuda()
    a = HIPIndexer(nl, 1, bf, layout=layout).build(K[:, :, :n], K[:, :, :n])
    b = HIPIndexer(nl, 1, bf, layout=layout).build(K[:, :, :n], K[:, :, :n])
    before = [x.clone() for x in (a.keys_buf, a.values_buf, a.perm)]
    HIPIndexer._warmed.clear()
    a.warm_up()
    assert len(HIPIndexer._warmed) == 1
    a.warm_up()  # a second call does nothing
    assert len(HIPIndexer._warmed) == 1
    for x, y in zip(before, (a.keys_buf, a.values_buf, a.perm)):
        assert torch.equal(x, y)
    for i in (a, b):
        i.update(K[:, :, n:n + 40], K[:, :, n:n + 40])
    assert a.size == b.size and a.num_keys == b.num_keys == n + 40
    assert torch.equal(a.perm[:, :a.size[0]], b.perm[:, :b.size[0]])
    for l in range(1, nl):
        assert torch.equal(a.radii[l][:, : a.size[l]], b.radii[l][:, : a.size[l]])
    _check_tree(a, keys, keys)
