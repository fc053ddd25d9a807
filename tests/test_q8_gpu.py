"""The index layout with an 8-bit shadow of the keys (HIRA_TILE16_Q8): the shadow is what its
definition says (pinned against numpy), and a search that scans the shadow first selects exactly
what the search over the bf16 keys selects -- against the CPU oracle and against the same tree in
the tiled layout, for the selected set, the scores, the attention output and the counters; after
appends (clipping keys included), grafts, subtree rebuilds and a save / load round trip too."""
import numpy as np
import pytest
import torch

from oracle import hira_oracle as ho
from helpers import assert_same_selection, bf16_round, midpoint_threshold, rel_err
from test_search_gpu import _setup

pytestmark = pytest.mark.gpu


def shadow_rowmajor(k8: torch.Tensor) -> np.ndarray:
    """(T, R, D) int8 in tiles of 16 rows x 64 columns (the 16-byte chunk with columns
    [64 s + 16 kb, +16) of row 16 t + i at chunk (t*(D/64) + s)*64 + kb*16 + i) -> row-major."""
    t, r, d = k8.shape
    v = k8.reshape(t, r // 16, d // 64, 4, 16, 16).permute(0, 1, 4, 2, 3, 5)
    return v.contiguous().reshape(t, r, d).cpu().numpy()


def expected_shadow(keys: np.ndarray, perm: np.ndarray, bf: int, kscale=None):
    """numpy statement of the shadow: step = largest magnitude of a channel over the live keys /
    127, k8 = round-half-even(k / step) clipped to +-127, bound per level-1 node = largest
    |k / step - k8| among its live keys; empty slots hold zeros."""
    live = perm >= 0
    k = np.where(live[..., None], keys, 0.0).astype(np.float32)
    if kscale is None:
        kscale = np.maximum(np.abs(k).max(axis=1) / np.float32(127.0), np.float32(1e-30)).astype(np.float32)
    u = (k / kscale[:, None, :]).astype(np.float32)
    k8 = np.clip(np.rint(u), -127, 127)
    err = np.where(live[..., None], np.abs(u - k8), 0.0).max(axis=2)
    t, n = err.shape
    keps = err.reshape(t, n // bf, bf).max(axis=2)
    return kscale, k8.astype(np.int8), keps.astype(np.float32)


Q8_CASES = [
    # h_kv, h_q, n, d, bf, levels, keep
    (2, 8, 2048, 128, 32, 3, 41),
    (1, 1, 1500, 128, 32, 2, 30),       # one head per tree, ragged last block
    (2, 16, 1024, 128, 32, 3, 30),      # 8 heads per tree
    (1, 16, 1100, 64, 16, 3, 33),       # 16 heads per tree, d = 64, fan-out 16
    (1, 20, 900, 64, 16, 2, 27),        # 20 heads per tree: two passes of the head loop
    (1, 4, 3000, 128, 48, 2, 60),       # fan-out 48 (3 tiles per block)
    (1, 4, 5000, 128, 64, 3, 50),       # fan-out 64
    (2, 8, 40000, 128, 32, 4, 400),     # four levels
    (1, 8, 3000, 128, 64, 2, 40),       # fan-out 64, 8 heads
    (1, 16, 2600, 64, 64, 3, 30),       # d = 64, fan-out 64, 16 heads
]


@pytest.mark.parametrize("case", Q8_CASES, ids=[f"hkv{c[0]}_hq{c[1]}_n{c[2]}_d{c[3]}_bf{c[4]}_L{c[5]}"
                                                  for c in Q8_CASES])
def test_shadow_scan_selects_what_the_bf16_scan_selects(case, gpu_device):
    from hira_amd import _lib
    from hira_amd.searcher.hip import HIPSearcher

    h_kv, h_q, n, d, bf, nl, keep = case
    print(f"case {case}", flush=True)
    kw = dict(seed=500 + n, keep=keep, niter=1 if n > 5000 else 2)
    c = _setup(h_kv, h_q, n, d, bf, nl, torch.bfloat16, layout="q8", **kw)
    t = _setup(h_kv, h_q, n, d, bf, nl, torch.bfloat16, layout="tiled", **kw)
    idx = c["idx"]
    assert idx.q8 and idx.tiled and not idx.keys_tiled

    # the shadow itself
    n_pad = idx.size[0]
    kscale, k8, keps = expected_shadow(c["ff"].keys, c["ff"].perm, bf)
    np.testing.assert_array_equal(idx.kscale.cpu().numpy(), kscale)
    np.testing.assert_array_equal(shadow_rowmajor(idx.keys8)[:, :n_pad], k8)
    np.testing.assert_array_equal(idx.keps.cpu().numpy()[:, : n_pad // bf], keps)

    q, th = torch.from_numpy(c["q"]), torch.from_numpy(c["th"])
    scale = d ** -0.5
    sc = torch.full((h_q,), scale)
    s = np.where(c["valid"], c["s"], -np.inf).astype(np.float32)
    mask = (c["s"] >= c["th"][:, None]) & c["valid"]
    ref = ho.attention(c["ff"].keys, c["vslot"], c["q"], sc.numpy(), mask, c["q2kv"])
    se = HIPSearcher(kernel=2)
    st = torch.zeros((h_kv, _lib.HIRA_STATS_COLS), dtype=torch.int64, device="cuda")
    st_t = torch.zeros_like(st)
    out = se.search(q, th, idx, scaling=sc, stats=st).cpu().numpy()
    out_t = se.search(q, th, t["idx"], scaling=sc, stats=st_t).cpu().numpy()
    assert_same_selection(out != 0, s, c["th"])
    # the exact test multiplies what the scan of the tiled keys multiplies: same bits
    np.testing.assert_array_equal(out, out_t)
    pos = se.search(q, th, idx, scaling=sc, index_space="position").cpu().numpy()
    assert_same_selection(pos != 0, ho.scores(c["keys"], c["q"], c["q2kv"]), c["th"])
    m = out != 0
    lists = [x.cpu().numpy() for x in se.search_compact(q, th, idx, scaling=sc)]
    for h in range(h_q):
        got = lists[0][h, : lists[2][h]]
        assert np.array_equal(np.sort(got), np.nonzero(m[h])[0])
        np.testing.assert_array_equal(lists[1][h, : lists[2][h]][np.argsort(got)] * np.float32(scale),
                                      out[h][m[h]])
    att = se.search_attention(q, th, idx, scaling=sc).cpu().numpy()
    att_t = se.search_attention(q, th, t["idx"], scaling=sc).cpu().numpy()
    assert rel_err(att, ref) <= 2e-3
    np.testing.assert_allclose(att, att_t, rtol=1e-5, atol=1e-6)
    # counters: the gates and the selections are those of the tiled tree; the rows fetched for the
    # exact test lie between the selected and the candidate keys
    st, st_t = st.cpu().numpy(), st_t.cpu().numpy()
    ml = _lib.HIRA_MAX_LEVELS
    np.testing.assert_array_equal(st[:, : ml + 2], st_t[:, : ml + 2])
    if h_q // h_kv <= 16:
        assert (st[:, ml + 2] >= st[:, ml]).all() and (st[:, ml + 2] <= st[:, 0]).all()
    assert (st_t[:, ml + 2] == 0).all()
    # the vector-ALU kernel reads the row-major keys of this layout directly
    out_v = HIPSearcher(kernel=1).search(q, th, idx, scaling=sc).cpu().numpy()
    assert_same_selection(out_v != 0, s, c["th"])
    # every key selected: dense attention through the sparse path
    full = se.search_attention(q, -3e38, idx, scaling=sc).cpu().numpy()
    ref_full = ho.attention(c["ff"].keys, c["vslot"], c["q"], sc.numpy(), c["valid"], c["q2kv"])
    assert rel_err(full, ref_full) <= 2e-3


def _massive(h_kv, n, d, seed):
    """Keys with per-channel scales, an offset and 8 channels blown up twentyfold (the
    benchmark's headline keys), and queries that are noisy copies of keys."""
    rng = np.random.default_rng(seed)
    s = np.exp(rng.normal(0, 0.5, size=(h_kv, 1, d)))
    mu = rng.normal(0, 0.3, size=(h_kv, 1, d))
    k = mu + s * rng.normal(size=(h_kv, n, d))
    ch = np.stack([rng.choice(d, 8, replace=False) for _ in range(h_kv)])
    for h in range(h_kv):
        k[h][:, ch[h]] *= 20.0
    return bf16_round(k.astype(np.float32)), ch


@pytest.mark.parametrize("group", [1, 4, 8])
def test_shadow_scan_on_keys_with_massive_channels(group, gpu_device):
    """Built on the device (HIPIndexer.build, layout q8), searched with thresholds that keep 1 %:
    selected set against brute force, attention against the oracle, and how few rows the exact
    test has to fetch."""
    from hira_amd import _lib
    from hira_amd.indexer.hip import HIPIndexer
    from hira_amd.searcher.hip import HIPSearcher

    h_kv, n, d, bf = 2, 8192, 128, 32
    h_q = h_kv * group
    keys, ch = _massive(h_kv, n, d, 77)
    rng = np.random.default_rng(78)
    vals = bf16_round(rng.normal(size=(h_kv, n, d)).astype(np.float32))
    q2kv = np.repeat(np.arange(h_kv), group)
    q = keys[q2kv, rng.integers(0, n, h_q)] + 0.5 * rng.normal(size=(h_q, d)).astype(np.float32)
    q = bf16_round(q.astype(np.float32))
    s = ho.scores(keys, q, q2kv)
    th = midpoint_threshold(s, 82)
    idx = HIPIndexer(3, 1, bf, layout="q8").build(
        torch.from_numpy(keys)[None].to(torch.bfloat16).cuda(), torch.from_numpy(vals)[None].to(torch.bfloat16).cuda())
    assert idx.q8
    se = HIPSearcher(kernel=2, index_space="position")
    st = torch.zeros((h_kv, _lib.HIRA_STATS_COLS), dtype=torch.int64, device="cuda")
    sc = torch.full((h_q,), d ** -0.5)
    out = se.search(torch.from_numpy(q), torch.from_numpy(th), idx, scaling=sc, stats=st).cpu().numpy()
    assert_same_selection(out != 0, s, th)
    att = se.search_attention(torch.from_numpy(q), torch.from_numpy(th), idx, scaling=sc).cpu().numpy()
    ref = ho.attention(keys, vals, q, sc.numpy(), s >= th[:, None], q2kv)
    assert rel_err(att, ref) <= 2e-3
    st = st.cpu().numpy()
    ml = _lib.HIRA_MAX_LEVELS
    fetched, union, cand = st[:, ml + 2].sum(), st[:, ml].sum(), st[:, 0].sum()
    print(f"group {group}: candidates {cand}, fetched for the exact test {fetched}, selected {union}")
    assert union <= fetched <= 1.5 * union + 64


def test_appends_grafts_and_rebuilds_keep_the_shadow_valid(gpu_device, tmp_path):
    """Keys appended one by one (some far outside the range the steps were made for: they clip,
    and the node's bound must cover it), a grafted window, a rebuilt subtree, a save / load round
    trip: after each the shadow obeys its definition with the index's steps, and the search still
    selects exactly the brute-force set."""
    from hira_amd.indexer.hip import HIPIndexer
    from hira_amd.searcher.hip import HIPSearcher

    h_kv, n, d, bf, group = 2, 4096, 128, 32, 4
    h_q = h_kv * group
    keys, _ = _massive(h_kv, n + 1200, d, 5)
    rng = np.random.default_rng(6)
    keys[:, n + 10:n + 20] *= 3.0  # beyond +-127 steps in the shadow
    vals = bf16_round(rng.normal(size=keys.shape).astype(np.float32))
    tk = torch.from_numpy(keys)[None].to(torch.bfloat16).cuda()
    tv = torch.from_numpy(vals)[None].to(torch.bfloat16).cuda()
    idx = HIPIndexer(3, 1, bf, layout="q8", capacity=n + 4096).build(tk[:, :, :n], tv[:, :, :n])
    q2kv = np.repeat(np.arange(h_kv), group)
    se = HIPSearcher(kernel=2, index_space="position")
    sc = torch.full((h_q,), d ** -0.5)

    def check(idx, upto, tag):
        kscale = idx.kscale.cpu().numpy()
        n_pad = idx.size[0]
        kk = idx.keys_buf[:, :n_pad].float().cpu().numpy()
        pp = idx.perm[:, :n_pad].cpu().numpy()
        _, k8, keps = expected_shadow(kk, pp, bf, kscale)
        np.testing.assert_array_equal(shadow_rowmajor(idx.keys8)[:, :n_pad], k8, err_msg=tag)
        got = idx.keps.cpu().numpy()[:, : n_pad // bf]
        assert (got >= keps).all(), tag  # a bound: never below the error of a key in the node
        for seed in range(3):
            r = np.random.default_rng(100 + seed)
            q = keys[q2kv, r.integers(0, upto, h_q)] + 0.5 * r.normal(size=(h_q, d)).astype(np.float32)
            q = bf16_round(q.astype(np.float32))
            s = ho.scores(keys[:, :upto], q, q2kv)
            th = midpoint_threshold(s, max(upto // 100, 8))
            out = se.search(torch.from_numpy(q), torch.from_numpy(th), idx, scaling=sc).cpu().numpy()
            assert out.shape[1] == upto, tag
            assert_same_selection(out != 0, s, th)
            att = se.search_attention(torch.from_numpy(q), torch.from_numpy(th), idx, scaling=sc).cpu().numpy()
            ref = ho.attention(keys[:, :upto], vals[:, :upto], q, sc.numpy(), s >= th[:, None], q2kv)
            assert rel_err(att, ref) <= 2e-3, tag

    check(idx, n, "built")
    for i in range(n, n + 40):  # one by one; ten of them clip
        idx.update(tk[:, :, i:i + 1], tv[:, :, i:i + 1])
    assert float(idx.keps.max()) > 0.5
    check(idx, n + 40, "appended")
    idx.update(tk[:, :, n + 40:n + 40 + 1024], tv[:, :, n + 40:n + 40 + 1024])  # a grafted window
    check(idx, n + 1064, "grafted")
    idx.update(tk[:, :, n + 1064:n + 1200], tv[:, :, n + 1064:n + 1200])
    idx.rebuild_subtree(0)
    check(idx, n + 1200, "rebuilt")
    path = tmp_path / "q8.safetensors"
    idx.save(str(path))
    back = HIPIndexer.load(str(path))
    assert back.q8
    np.testing.assert_array_equal(back.keys8.cpu().numpy()[:, : idx.size[0]], idx.keys8.cpu().numpy()[:, : idx.size[0]])
    check(back, n + 1200, "restored")
