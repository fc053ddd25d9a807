"""GPU parity of the HIP search / sparse-attention path against the CPU oracle, through
the C ABI (hira_search), on trees built on the host by the oracle."""
import numpy as np
import pytest
import torch

from oracle import hira_oracle as ho
from helpers import (assert_same_selection, band_free_heads, bf16_round, clustered_keys, midpoint_threshold,
                     normalized_keys, random_query, rel_err)

pytestmark = pytest.mark.gpu


def _setup(h_kv, h_q, n, d, bf, nl, dtype, seed, keep, clustered=True, q2kv=None, dv=None,
           unit_q=True, niter=2, layout="auto"):
    from hira_amd.indexer.hip import HIPIndexer

    keys = (clustered_keys if clustered else normalized_keys)(h_kv, n, d, seed)
    rng = np.random.default_rng(seed)
    dv = d if dv is None else dv
    vals = rng.normal(size=(h_kv, n, dv)).astype(np.float32)
    q = random_query(h_q, d, seed + 1, normalize=unit_q)
    if not unit_q:
        q = q * 3.0
    rnd = bf16_round if dtype == torch.bfloat16 else (lambda a: a)
    keys, vals, q = rnd(keys), rnd(vals), rnd(q)
    ff = ho.fixed_fanout_tree(keys, bf, nl, niter=niter, round_fn=rnd if nl > 1 else None)
    ok = ff.perm >= 0
    vslot = np.zeros((h_kv, ff.sizes[0], dv), np.float32)
    for h in range(h_kv):
        vslot[h][ok[h]] = vals[h][ff.perm[h][ok[h]]]
    q2kv = ho.default_q2kv(h_q, h_kv) if q2kv is None else np.asarray(q2kv)
    s = ho.scores(ff.keys, q, q2kv)
    valid = ok[q2kv]
    th = midpoint_threshold(np.where(valid, s, -1e30), keep)
    idx = HIPIndexer.from_layout(bf=bf, keys=ff.keys, perm=ff.perm, centers=ff.centers,
                                 radii=ff.radii, counts=ff.counts, values=vslot, dtype=dtype,
                                 num_keys=n, layout=layout)
    return dict(ff=ff, idx=idx, q=q, th=th, s=s, valid=valid, q2kv=q2kv, keys=keys, vals=vals,
                vslot=vslot)


CASES = [
    # h_kv, h_q, n, d, bf, levels, dtype, keep
    (2, 2, 192, 64, 8, 3, torch.float32, 48),
    (2, 6, 192, 128, 8, 3, torch.float32, 48),
    (1, 1, 4096, 128, 16, 2, torch.float32, 205),
    (2, 8, 2048, 128, 32, 3, torch.bfloat16, 41),
    (2, 16, 1024, 128, 32, 3, torch.bfloat16, 30),   # 8 heads per tree
    (1, 12, 600, 64, 8, 3, torch.bfloat16, 30),      # 12 heads per tree: two passes
    (3, 3, 203, 32, 4, 4, torch.float32, 25),        # pad slots, 4 levels
    (2, 4, 333, 16, 5, 3, torch.float32, 40),        # odd fan-out, narrow rows
    (2, 4, 333, 16, 5, 3, torch.bfloat16, 40),
    (1, 2, 500, 256, 16, 2, torch.float32, 50),
    (1, 2, 500, 256, 16, 2, torch.bfloat16, 50),
    (2, 2, 300, 64, 8, 1, torch.float32, 30),        # one level: flat scan
    (1, 4, 70000, 128, 32, 4, torch.bfloat16, 700),
]


@pytest.mark.parametrize("case", CASES, ids=[f"hkv{c[0]}_hq{c[1]}_n{c[2]}_d{c[3]}_bf{c[4]}_L{c[5]}_"
                                               f"{'bf16' if c[6] == torch.bfloat16 else 'f32'}"
                                               for c in CASES])
def test_selected_set_and_scores_match_oracle(case, gpu_device):
    from hira_amd.searcher.hip import HIPSearcher

    h_kv, h_q, n, d, bf, nl, dtype, keep = case
    print(f"case {case}", flush=True)
    c = _setup(h_kv, h_q, n, d, bf, nl, dtype, seed=100 + n, keep=keep, niter=1 if n > 5000 else 2)
    sc = torch.full((h_q,), 0.125)
    searcher = HIPSearcher()
    q4 = torch.from_numpy(c["q"]).view(1, h_q, 1, d)
    out = searcher.search(q4, torch.from_numpy(c["th"]), c["idx"], scaling=sc).cpu().numpy()
    # slot space: bit-exact set, outside the 1e-5 relative band around the threshold
    s = np.where(c["valid"], c["s"], -np.inf).astype(np.float32)
    assert_same_selection(out != 0, s, c["th"])
    m = out != 0
    np.testing.assert_allclose(out[m], (c["s"] * 0.125)[m], rtol=2e-5, atol=1e-6)
    # position space (the CPU searcher's contract): compare with the oracle on the keys in
    # insertion order
    pos = searcher.search(q4, torch.from_numpy(c["th"]), c["idx"], scaling=sc,
                          index_space="position").cpu().numpy()
    assert pos.shape == (h_q, n)
    s_pos = ho.scores(c["keys"], c["q"], c["q2kv"])
    assert_same_selection(pos != 0, s_pos, c["th"])
    # compact lists carry the same set
    idx, score, count = searcher.search_compact(q4, torch.from_numpy(c["th"]), c["idx"], scaling=sc)
    idx, score, count = idx.cpu().numpy(), score.cpu().numpy(), count.cpu().numpy()
    for h in range(h_q):
        got = np.sort(idx[h, :count[h]])
        assert np.array_equal(got, np.nonzero(m[h])[0])
        order = np.argsort(idx[h, :count[h]])
        np.testing.assert_allclose(score[h, :count[h]][order] * 0.125, out[h][m[h]], rtol=1e-6)


MFMA_CASES = [
    # h_kv, h_q, n, d, bf, levels, keep
    (2, 8, 2048, 128, 32, 3, 41),
    (1, 1, 1500, 128, 32, 2, 30),       # one head per tree, ragged last block
    (2, 16, 1024, 128, 32, 3, 30),      # 8 heads per tree
    (1, 16, 1100, 64, 16, 3, 33),       # 16 heads per tree, d = 64, fan-out 16
    (1, 20, 900, 64, 16, 2, 27),        # 20 heads per tree: two passes of the head loop
    (1, 4, 3000, 256, 48, 2, 60),       # d = 256, fan-out 48 (3 tiles per block)
    (1, 4, 5000, 128, 64, 3, 50),       # fan-out 64
    (2, 8, 40000, 128, 32, 4, 400),     # four levels
    (1, 8, 3000, 256, 64, 2, 40),       # d = 256, fan-out 64, 8 heads: nodes scanned as two halves
    (1, 16, 2600, 256, 64, 3, 30),      # the same with 16 heads
    (1, 8, 2000, 256, 48, 2, 30),       # halves of two tiles and one
]


@pytest.mark.parametrize("case", MFMA_CASES, ids=[f"hkv{c[0]}_hq{c[1]}_n{c[2]}_d{c[3]}_bf{c[4]}_L{c[5]}"
                                                    for c in MFMA_CASES])
def test_mfma_kernel_matches_oracle_and_vector_kernel(case, gpu_device):
    """bf16 trees in the tiled layout: the MFMA kernel (kernel=2), the vector-ALU kernel on
    the same tiled tree (kernel=1) and the oracle select the same keys; attention agrees
    with the fp64 oracle to 2e-3; the device counters of both kernels agree."""
    from hira_amd import _lib
    from hira_amd.searcher.hip import HIPSearcher

    h_kv, h_q, n, d, bf, nl, keep = case
    print(f"case {case}", flush=True)
    c = _setup(h_kv, h_q, n, d, bf, nl, torch.bfloat16, seed=500 + n, keep=keep,
               niter=1 if n > 5000 else 2, layout="tiled")
    assert c["idx"].tiled
    q, th = torch.from_numpy(c["q"]), torch.from_numpy(c["th"])
    scale = d ** -0.5
    sc = torch.full((h_q,), scale)
    s = np.where(c["valid"], c["s"], -np.inf).astype(np.float32)
    mask = (c["s"] >= c["th"][:, None]) & c["valid"]
    ref = ho.attention(c["ff"].keys, c["vslot"], c["q"], sc.numpy(), mask, c["q2kv"])
    stats = {}
    for kernel in (2, 1):
        se = HIPSearcher(kernel=kernel)
        st = torch.zeros((h_kv, _lib.HIRA_STATS_COLS), dtype=torch.int64, device="cuda")
        out = se.search(q, th, c["idx"], scaling=sc, stats=st).cpu().numpy()
        assert_same_selection(out != 0, s, c["th"])
        m = out != 0
        np.testing.assert_allclose(out[m], (c["s"] * scale)[m], rtol=2e-5, atol=1e-6)
        pos = se.search(q, th, c["idx"], scaling=sc, index_space="position").cpu().numpy()
        assert_same_selection(pos != 0, ho.scores(c["keys"], c["q"], c["q2kv"]), c["th"])
        idx, score, count = (t.cpu().numpy() for t in se.search_compact(q, th, c["idx"], scaling=sc))
        for h in range(h_q):
            assert np.array_equal(np.sort(idx[h, :count[h]]), np.nonzero(m[h])[0])
        att = se.search_attention(q, th, c["idx"], scaling=sc).cpu().numpy()
        assert rel_err(att, ref) <= 2e-3, (kernel, rel_err(att, ref))
        stats[kernel] = st.cpu().numpy()
    if h_q // h_kv <= 8:  # both kernels cover the group in one pass: same counters
        assert np.array_equal(stats[1], stats[2])
    pairs = int(mask.sum())
    assert stats[1][:, _lib.HIRA_MAX_LEVELS + 1].sum() == pairs == stats[2][:, _lib.HIRA_MAX_LEVELS + 1].sum()
    # every key selected: dense attention through the sparse path
    full = HIPSearcher(kernel=2).search_attention(q, -3e38, c["idx"], scaling=sc).cpu().numpy()
    ref_full = ho.attention(c["ff"].keys, c["vslot"], c["q"], sc.numpy(), c["valid"], c["q2kv"])
    assert rel_err(full, ref_full) <= 2e-3


@pytest.mark.parametrize("case", [
    # h_kv, h_q, n, d, bf, levels, dtype, keep, kernel
    (2, 6, 192, 128, 8, 3, torch.float32, 48, 1),
    (3, 3, 203, 32, 4, 4, torch.float32, 25, 1),       # pad slots, batched gates
    (2, 2, 300, 64, 8, 1, torch.float32, 30, 1),       # one level: flat scan
    (2, 8, 2048, 128, 32, 3, torch.bfloat16, 41, 2),
    (1, 12, 600, 64, 16, 3, torch.bfloat16, 30, 2),    # 12 heads a tree: two passes; a partial tile
    (2, 8, 2048, 128, 32, 3, torch.bfloat16, 41, 1),
], ids=lambda c: f"hkv{c[0]}_hq{c[1]}_n{c[2]}_d{c[3]}_bf{c[4]}_L{c[5]}_k{c[8]}")
def test_search_fills_what_it_does_not_select(case, gpu_device):
    """In slot space the search writes the fill value itself (HiraSearchOut.dense_fill; the
    reference fills its buffer before every search, searcher/cuda.py:35-54): a buffer that
    holds anything else beforehand comes back with the scores of the selected keys and the fill
    value everywhere else, pad slots included; in position space the wrapper still pre-fills."""
    from hira_amd.searcher.hip import HIPSearcher

    h_kv, h_q, n, d, bf, nl, dtype, keep, kernel = case
    print(f"case {case}", flush=True)
    su = _setup(h_kv, h_q, n, d, bf, nl, dtype, seed=77 + n, keep=keep)
    q, th = torch.from_numpy(su["q"]), torch.from_numpy(su["th"])
    for fill in (0.0, -5.0):
        se = HIPSearcher(kernel=kernel, output_fill_value=fill)
        first = se.search(q, th, su["idx"]).clone()
        se._tmp_out.fill_(7.0)                          # whatever an earlier call left behind
        again = se.search(q, th, su["idx"])
        assert torch.equal(first, again)
        out = again.cpu().numpy()
        want = np.where(su["valid"] & (su["s"] >= su["th"][:, None]), su["s"], np.float32(fill))
        band = np.abs(su["s"] - su["th"][:, None]) <= 1e-5 * np.abs(su["th"][:, None])
        ok = band | np.isclose(out, want, rtol=2e-5, atol=1e-6)
        assert ok.all(), int((~ok).sum())
        assert (out[~su["valid"]] == np.float32(fill)).all()
        se._tmp_out.fill_(7.0)
        pos = se.search(q, th, su["idx"], index_space="position").cpu().numpy()
        assert not (pos == 7.0).any()
        assert (pos != np.float32(fill)).sum() == (out != np.float32(fill)).sum()


def test_mfma_kernel_is_refused_where_it_does_not_apply(gpu_device):
    from hira_amd.searcher.hip import HIPSearcher

    c = _setup(2, 4, 333, 16, 5, 3, torch.bfloat16, seed=9, keep=20)
    assert not c["idx"].tiled
    with pytest.raises(ValueError):
        HIPSearcher(kernel=2).search(torch.from_numpy(c["q"]), torch.from_numpy(c["th"]), c["idx"])


def test_explicit_non_monotone_head_map(gpu_device):
    """tests/test_cpp_kernels.py:529-565 of the reference: q_head_to_kv = [1, 0, 1, 0]."""
    from hira_amd.searcher.hip import HIPSearcher

    c = _setup(2, 4, 192, 64, 8, 3, torch.float32, seed=311, keep=38, q2kv=[1, 0, 1, 0])
    out = HIPSearcher().search(torch.from_numpy(c["q"]), torch.from_numpy(c["th"]), c["idx"],
                               q_head_to_kv=torch.tensor([1, 0, 1, 0])).cpu().numpy()
    s = np.where(c["valid"], c["s"], -np.inf).astype(np.float32)
    assert_same_selection(out != 0, s, c["th"])


def test_non_unit_queries_use_norm_scaled_radius(gpu_device):
    """The gate q.c + ||q|| r stays conservative for ||q|| != 1 (searcher/cpu.py:61-63)."""
    from hira_amd.searcher.hip import HIPSearcher

    c = _setup(2, 4, 1000, 64, 8, 3, torch.float32, seed=21, keep=60, unit_q=False)
    out = HIPSearcher().search(torch.from_numpy(c["q"]), torch.from_numpy(c["th"]), c["idx"]).cpu().numpy()
    s = np.where(c["valid"], c["s"], -np.inf).astype(np.float32)
    assert_same_selection(out != 0, s, c["th"])


def test_low_threshold_returns_every_valid_score_and_zero_scaling_returns_zeros(gpu_device):
    """tests/test_triton_kernels.py:243-280, tests/test_cpu_pipeline.py:257-267."""
    from hira_amd.searcher.hip import HIPSearcher

    c = _setup(2, 2, 203, 32, 4, 3, torch.float32, seed=5, keep=10)
    se = HIPSearcher(output_fill_value=-7.0)
    out = se.search(torch.from_numpy(c["q"]), -2.0, c["idx"]).cpu().numpy()
    assert np.all(out[~c["valid"]] == -7.0)
    np.testing.assert_allclose(out[c["valid"]], c["s"][c["valid"]], rtol=2e-5, atol=1e-6)
    z = HIPSearcher().search(torch.from_numpy(c["q"]), -2.0, c["idx"], scaling=torch.zeros(2))
    assert float(z.abs().max()) == 0.0


def test_device_counters_match_oracle_traffic(gpu_device):
    from hira_amd.searcher.hip import HIPSearcher
    from hira_amd import _lib

    c = _setup(2, 8, 4096, 64, 16, 3, torch.float32, seed=8, keep=40)
    stats = torch.zeros((2, _lib.HIRA_STATS_COLS), dtype=torch.int64, device="cuda")
    HIPSearcher().search(torch.from_numpy(c["q"]), torch.from_numpy(c["th"]), c["idx"], stats=stats)
    tree, csr = ho.fixed_fanout_as_cpu_tree(c["ff"])
    tr = ho.group_traffic(tree, c["q"], c["th"], q2kv=c["q2kv"], csr=csr,
                          rscale=np.linalg.norm(c["q"], axis=1))
    st = stats.cpu().numpy()
    assert np.array_equal(st[:, :3], tr[:, :3])
    assert np.array_equal(st[:, _lib.HIRA_MAX_LEVELS], tr[:, 3])
    assert (tr[:, 0] < 4096).all()  # the clustered keys are really pruned


BATCHED_GATE_CASES = [
    # h_kv, h_q, n, d, bf, levels, dtype, keep, nodes per wave
    (1, 1, 3001, 128, 4, 3, torch.float32, 30, 8),
    (1, 1, 3001, 128, 4, 3, torch.float32, 30, 5),     # a batch that ends inside a step of gates
    (2, 8, 1500, 128, 4, 3, torch.float32, 25, 16),    # 4 heads per tree, two batches per wave
    (1, 12, 900, 128, 2, 3, torch.float32, 20, 8),     # fan-out 2, 12 heads per tree: two passes
    (2, 4, 1111, 128, 3, 4, torch.float32, 22, 8),     # odd fan-out, four levels
    (2, 4, 1500, 256, 4, 3, torch.bfloat16, 25, 8),
    (1, 2, 2000, 128, 2, 2, torch.bfloat16, 40, 16),
]


@pytest.mark.parametrize("case", BATCHED_GATE_CASES,
                         ids=[f"hkv{c[0]}_hq{c[1]}_n{c[2]}_d{c[3]}_bf{c[4]}_L{c[5]}_"
                              f"{'bf16' if c[6] == torch.bfloat16 else 'f32'}_npw{c[8]}"
                              for c in BATCHED_GATE_CASES])
def test_small_fanout_with_batched_gates(case, gpu_device):
    """Fan-outs of 2 .. 4: a wave evaluates the gates of several steps of nodes together and scans
    their keys as one block (what the library picks by itself for large trees; forced here through
    the launch override).  Same selected set, scores, lists, counters and attention output as the
    oracle and as the launch that takes one step of nodes at a time."""
    from hira_amd.searcher.hip import HIPSearcher
    from hira_amd import _lib

    h_kv, h_q, n, d, bf, nl, dtype, keep, npw = case
    print(f"case {case}", flush=True)
    c = _setup(h_kv, h_q, n, d, bf, nl, dtype, seed=700 + n, keep=keep)
    scale = d ** -0.5
    sc = torch.full((h_q,), scale)
    q, th = torch.from_numpy(c["q"]), torch.from_numpy(c["th"])
    plain, batched = HIPSearcher(nodes_per_wave=1), HIPSearcher(nodes_per_wave=npw)
    st0 = torch.zeros((h_kv, _lib.HIRA_STATS_COLS), dtype=torch.int64, device="cuda")
    st1 = torch.zeros_like(st0)
    ref_out = plain.search(q, th, c["idx"], scaling=sc, stats=st0)
    out = batched.search(q, th, c["idx"], scaling=sc, stats=st1)
    assert torch.equal(out, ref_out)
    assert torch.equal(st0, st1)
    out = out.cpu().numpy()
    s = np.where(c["valid"], c["s"], -np.inf).astype(np.float32)
    assert_same_selection(out != 0, s, c["th"])
    m = out != 0
    np.testing.assert_allclose(out[m], (c["s"] * scale)[m], rtol=2e-5, atol=1e-6)
    idx, score, count = batched.search_compact(q, th, c["idx"], scaling=sc)
    idx, count = idx.cpu().numpy(), count.cpu().numpy()
    for h in range(h_q):
        assert np.array_equal(np.sort(idx[h, :count[h]]), np.nonzero(m[h])[0])
    att = batched.search_attention(q, th, c["idx"], scaling=sc).cpu().numpy()
    mask = (c["s"] >= c["th"][:, None]) & c["valid"]
    ref = ho.attention(c["ff"].keys, c["vslot"], c["q"], sc.numpy(), mask, c["q2kv"])
    ok = band_free_heads(c["s"], c["th"], c["valid"])
    assert ok.sum() >= max(1, h_q - 1)
    tol = 2e-3 if dtype == torch.bfloat16 else 1e-5
    assert rel_err(att[ok], ref[ok]) <= tol, rel_err(att[ok], ref[ok])


@pytest.mark.parametrize("n", [40000, 90000])
def test_large_tree_of_small_fanout_picks_batched_gates(n, gpu_device):
    """At 40k / 90k keys with fan-out 4 the library batches two / four steps of gates by itself:
    same output as the one-step launch, and the selected set is the brute-force one."""
    from hira_amd.indexer.hip import HIPIndexer
    from hira_amd.searcher.hip import HIPSearcher

    g = torch.Generator().manual_seed(n)
    keys = torch.nn.functional.normalize(torch.randn(1, 1, n, 128, generator=g), dim=-1).cuda()
    q = torch.nn.functional.normalize(torch.randn(1, 128, generator=g), dim=-1).cuda()
    idx = HIPIndexer(3, 1, 4).build(keys)
    s = (keys[0, 0] @ q[0]).cpu().numpy()
    th = midpoint_threshold(s[None], 50)
    auto = HIPSearcher().search(q, torch.from_numpy(th), idx, index_space="position")
    plain = HIPSearcher(nodes_per_wave=2).search(q, torch.from_numpy(th), idx,
                                                 index_space="position")
    assert torch.equal(auto, plain)
    assert_same_selection(auto.cpu().numpy() != 0, s[None], th)


ATTN_CASES = [
    (1, 1, 4096, 128, 16, 2, torch.float32, 205, 1e-5),
    (2, 8, 2048, 128, 32, 3, torch.bfloat16, 41, 2e-3),
    (2, 16, 1024, 128, 32, 3, torch.bfloat16, 30, 2e-3),
    (3, 3, 203, 32, 4, 4, torch.float32, 25, 1e-5),
    (2, 4, 333, 16, 5, 3, torch.bfloat16, 40, 2e-3),
    (2, 2, 300, 64, 8, 1, torch.float32, 30, 1e-5),
]


@pytest.mark.parametrize("case", ATTN_CASES, ids=[f"hkv{c[0]}_hq{c[1]}_n{c[2]}_d{c[3]}_L{c[5]}_"
                                                    f"{'bf16' if c[6] == torch.bfloat16 else 'f32'}"
                                                    for c in ATTN_CASES])
def test_fused_attention_matches_fp64_oracle(case, gpu_device):
    """softmax(scaling q.K_S^T) V_S over the oracle's selected set; tolerance 1e-5 (fp32
    storage) / 2e-3 (bf16 storage) relative to the largest output component of the head."""
    from hira_amd.searcher.hip import HIPSearcher

    h_kv, h_q, n, d, bf, nl, dtype, keep, tol = case
    print(f"case {case}", flush=True)
    c = _setup(h_kv, h_q, n, d, bf, nl, dtype, seed=300 + n, keep=keep)
    scale = d ** -0.5
    sc = torch.full((h_q,), scale)
    out = HIPSearcher().search_attention(torch.from_numpy(c["q"]), torch.from_numpy(c["th"]),
                                         c["idx"], scaling=sc).cpu().numpy()
    mask = (c["s"] >= c["th"][:, None]) & c["valid"]
    ref = ho.attention(c["ff"].keys, c["vslot"], c["q"], sc.numpy(), mask, c["q2kv"])
    ok = band_free_heads(c["s"], c["th"], c["valid"])   # (a key within rounding of tau may go either way)
    assert ok.sum() >= max(1, h_q - 1)
    assert rel_err(out[ok], ref[ok]) <= tol, rel_err(out[ok], ref[ok])


def test_attention_with_queue_and_empty_selection(gpu_device):
    from hira_amd.searcher.hip import HIPSearcher

    c = _setup(2, 4, 512, 64, 8, 3, torch.float32, seed=55, keep=20)
    rng = np.random.default_rng(3)
    qk = rng.normal(size=(2, 37, 64)).astype(np.float32) * 0.1
    qv = rng.normal(size=(2, 37, 64)).astype(np.float32)
    sc = torch.full((4,), 0.5)
    th = c["th"].copy()
    th[3] = 1e9  # head 3 selects nothing from the index: only the queue remains
    out = HIPSearcher().search_attention(
        torch.from_numpy(c["q"]), torch.from_numpy(th), c["idx"], scaling=sc,
        queue_keys=torch.from_numpy(qk), queue_values=torch.from_numpy(qv)).cpu().numpy()
    keys_all = np.concatenate([c["ff"].keys, qk], axis=1)
    vals_all = np.concatenate([c["vslot"], qv], axis=1)
    mask = (c["s"] >= th[:, None]) & c["valid"]
    mask = np.concatenate([mask, np.ones((4, 37), bool)], axis=1)
    ref = ho.attention(keys_all, vals_all, c["q"], sc.numpy(), mask, c["q2kv"])
    assert rel_err(out, ref) <= 1e-5
    # no queue and nothing selected -> zeros
    z = HIPSearcher().search_attention(torch.from_numpy(c["q"]), 1e9, c["idx"], scaling=sc)
    assert float(z.abs().max()) == 0.0


@pytest.mark.parametrize("h_kv,h_q,m", [(2, 8, 1), (2, 8, 37), (1, 8, 200), (2, 32, 64)])
def test_mfma_attention_with_queue(h_kv, h_q, m, gpu_device):
    """bf16 tiled index (MFMA kernel) plus a row-major queue of m keys per tree that every
    head attends to; both kernels against the fp64 oracle over index rows >= tau + queue."""
    from hira_amd.searcher.hip import HIPSearcher

    d = 128
    print(f"case h_kv={h_kv} h_q={h_q} m={m}", flush=True)
    c = _setup(h_kv, h_q, 2048, d, 32, 3, torch.bfloat16, seed=77 + m, keep=40)
    assert c["idx"].tiled
    rng = np.random.default_rng(m)
    qk = bf16_round(rng.normal(size=(h_kv, m, d)).astype(np.float32) * 0.3)
    qv = bf16_round(rng.normal(size=(h_kv, m, d)).astype(np.float32))
    sc = torch.full((h_q,), d ** -0.5)
    th = c["th"].copy()
    th[1] = 1e9  # head 1 selects nothing from the index: only the queue remains
    keys_all = np.concatenate([c["ff"].keys, qk], axis=1)
    vals_all = np.concatenate([c["vslot"], qv], axis=1)
    mask = (c["s"] >= th[:, None]) & c["valid"]
    mask = np.concatenate([mask, np.ones((h_q, m), bool)], axis=1)
    ref = ho.attention(keys_all, vals_all, c["q"], sc.numpy(), mask, c["q2kv"])
    for kernel in (2, 1):
        out = HIPSearcher(kernel=kernel).search_attention(
            torch.from_numpy(c["q"]), torch.from_numpy(th), c["idx"], scaling=sc,
            queue_keys=torch.from_numpy(qk).to(torch.bfloat16),
            queue_values=torch.from_numpy(qv).to(torch.bfloat16)).cpu().numpy()
        assert rel_err(out, ref) <= 2e-3, (kernel, rel_err(out, ref))


def test_bad_inputs_raise_value_error(gpu_device):
    """tests/test_triton_kernels.py:547-601 of the reference."""
    from hira_amd.searcher.hip import HIPSearcher

    c = _setup(2, 2, 192, 64, 8, 3, torch.float32, seed=1, keep=10)
    se = HIPSearcher()
    q = torch.from_numpy(c["q"])
    with pytest.raises(ValueError):
        se.search(q[:, :32], torch.from_numpy(c["th"]), c["idx"])       # wrong dim
    with pytest.raises(ValueError):
        se.search(q.view(2, 1, 1, 64)[:, :, :, :], torch.zeros(3), c["idx"])  # threshold length
    with pytest.raises(ValueError):
        se.search(q, torch.from_numpy(c["th"]), c["idx"], scaling=torch.ones(5))
    with pytest.raises(ValueError):
        se.search(torch.zeros(3, 64), torch.zeros(3), c["idx"])         # 3 heads over 2 trees


def test_wrapper_contract_of_the_reference_searcher(gpu_device):
    """tests/test_triton_kernels.py:152-199 (2-D and 4-D queries agree), :283-332 (scaling
    scales the scores and leaves the mask alone), searcher/cuda.py:35-54 (a persistent output
    buffer, pre-filled with output_fill_value), tests/test_cuda_pipeline.py:517-523 (no values
    given: none kept) of the reference."""
    from hira_amd.indexer.hip import HIPIndexer
    from hira_amd.searcher.hip import HIPSearcher

    h_kv, h_q, n, d = 2, 4, 700, 64
    keys = clustered_keys(h_kv, n, d, seed=12, clusters=20)
    q = random_query(h_q, d, seed=13)
    K = torch.from_numpy(keys)[None]
    idx = HIPIndexer(3, 1, 8).build(K)
    assert idx.values is None and idx.values_buf is None
    s = ho.scores(keys, q, ho.default_q2kv(h_q, h_kv))
    th = torch.from_numpy(midpoint_threshold(s, 35))
    q2, q4 = torch.from_numpy(q), torch.from_numpy(q).view(1, h_q, 1, d)
    se = HIPSearcher(block_c=8, output_fill_value=-7.0)
    a = se.search(q2, th, idx).clone()
    b = se.search(q4, th, idx)
    assert torch.equal(a, b)
    assert b.data_ptr() == se.search(q2, th, idx).data_ptr()       # the same buffer every call
    sel = a != -7.0
    assert int(sel.sum()) == h_q * 35 and float(a[~sel].abs().max()) == 7.0
    sc = torch.tensor([2.0, 0.5, 1.0, 3.0])
    c = se.search(q2, th, idx, scaling=sc).clone()
    assert torch.equal(c != -7.0, sel)
    assert torch.allclose(c[sel], (a * sc.cuda()[:, None])[sel], rtol=1e-6)
    with pytest.raises(ValueError):
        se.search_attention(q2, th, idx)                           # nothing to attend to


@pytest.mark.parametrize("h_kv,h_q,n,d,bf,nl,dtype", [(2, 8, 2048, 128, 32, 3, torch.bfloat16),
                                                      (1, 3, 600, 64, 8, 3, torch.float32),
                                                      (2, 4, 500, 256, 16, 2, torch.bfloat16),
                                                      (2, 2, 333, 16, 5, 3, torch.float32)])
def test_attention_over_given_lists(h_kv, h_q, n, d, bf, nl, dtype, gpu_device):
    """hira_sparse_attention on the lists search_compact returns == the fused launch == the
    float64 oracle; on edited lists (entries dropped, one list emptied) == the oracle over what
    is left."""
    from hira_amd.searcher.hip import HIPSearcher

    c = _setup(h_kv, h_q, n, d, bf, nl, dtype, seed=90 + n, keep=max(4, n // 20))
    se = HIPSearcher()
    q, th = torch.from_numpy(c["q"]), torch.from_numpy(c["th"])
    sc = torch.full((h_q,), d ** -0.5)
    idx, sco, cnt = se.search_compact(q, th, c["idx"])
    got = se.sparse_attention(idx, sco, cnt, c["idx"], scaling=sc).cpu().numpy()
    fused = se.search_attention(q, th, c["idx"], scaling=sc).cpu().numpy()
    mask = (c["s"] >= c["th"][:, None]) & c["valid"]
    ref = ho.attention(c["ff"].keys, c["vslot"], c["q"], sc.numpy(), mask, c["q2kv"])
    tol = 2e-3 if dtype == torch.bfloat16 else 1e-5
    assert rel_err(got, ref) <= tol and rel_err(got, fused) <= 1e-5
    # edited lists: every head keeps the first half of its entries, head 0 none
    idx2, sco2, cnt2 = idx.clone(), sco.clone(), (cnt // 2).clone()
    cnt2[0] = 0
    got2 = se.sparse_attention(idx2, sco2, cnt2, c["idx"], scaling=sc).cpu().numpy()
    mask2 = np.zeros_like(mask)
    ic, cc = idx2.cpu().numpy(), cnt2.cpu().numpy()
    for h in range(h_q):
        mask2[h, ic[h, : cc[h]]] = True
    ref2 = ho.attention(c["ff"].keys, c["vslot"], c["q"], sc.numpy(), mask2, c["q2kv"])
    assert np.all(got2[0] == 0)
    assert rel_err(got2[1:], ref2[1:]) <= tol
    with pytest.raises(ValueError):
        se.sparse_attention(idx, sco[:, :-1], cnt, c["idx"], scaling=sc)
