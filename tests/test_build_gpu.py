"""GPU tests of the HIP index build (hira_build through HIPIndexer.build): layout contract of
the reference's GPU indexer (tests/test_cuda_indexer_searcher.py:134-195 of the reference),
radius invariant (tests/test_cpu_indexer_searcher.py:62-81) and search parity on the built
tree."""
import numpy as np
import pytest
import torch

from oracle import hira_oracle as ho
from helpers import (assert_same_selection, bf16_round, clustered_keys, midpoint_threshold,
                     normalized_keys, random_query)

pytestmark = pytest.mark.gpu


def _download(idx):
    n0 = idx.size[0]
    out = dict(keys=idx.keys_rowmajor().float().cpu().numpy(),
               perm=idx.perm[:, :n0].cpu().numpy().astype(np.int64),
               values=None if idx.values_buf is None else idx.values_buf[:, :n0].float().cpu().numpy(),
               centers=[None], radii=[None], counts=[None])
    for l in range(1, idx.num_levels):
        k = idx.size[l]
        out["centers"].append(idx.centers_rowmajor(l).float().cpu().numpy())
        out["radii"].append(idx.radii[l][:, :k].cpu().numpy())
        out["counts"].append(idx.counts[l][:, :k].cpu().numpy())
    return out


def _check_layout(idx, keys, vals, dtype):
    from hira_amd.indexer.hip import level_sizes

    t, n, d = keys.shape
    bf, nl = idx.branching_factor, idx.num_levels
    assert idx.size == level_sizes(n, bf, nl) == ho.fixed_fanout_sizes(n, bf, nl)
    a = _download(idx)
    rnd = bf16_round if dtype == torch.bfloat16 else (lambda x: x)
    for h in range(t):
        perm = a["perm"][h]
        ok = perm >= 0
        # every key exactly once, rows travel with their slot, pads are zero
        assert np.array_equal(np.sort(perm[ok]), np.arange(n))
        assert np.array_equal(a["keys"][h][ok], keys[h][perm[ok]])
        assert not a["keys"][h][~ok].any()
        if vals is not None:
            assert np.array_equal(a["values"][h][ok], vals[h][perm[ok]])
        child_c, child_r, child_ok = a["keys"][h], np.zeros(idx.size[0], np.float32), ok
        for l in range(1, nl):
            k = idx.size[l]
            blk = child_ok.reshape(k, bf)
            assert np.array_equal(a["counts"][l][h], blk.sum(1)), f"counts level {l}"
            assert np.all(blk[:, :-1] >= blk[:, 1:]), "children must be packed from slot 0"
            assert a["counts"][l][h].min() >= 0 and a["counts"][l][h].max() <= bf
            # centre = mean of the children in the block, rounded to the storage type
            cc = child_c.reshape(k, bf, d)
            cnt = np.maximum(blk.sum(1), 1)[:, None]
            mean = rnd((np.where(blk[..., None], cc, 0).sum(1) / cnt).astype(np.float32))
            has = blk.any(1)
            np.testing.assert_allclose(a["centers"][l][h][has], mean[has], rtol=1e-2 if dtype == torch.bfloat16 else 1e-5,
                                       atol=1e-2 if dtype == torch.bfloat16 else 1e-5)
            # radius = recomputation from the layout (never smaller), -inf for empty nodes
            want = ho.radii_from_layout(child_c, child_r, child_ok, a["centers"][l][h], bf)
            got = a["radii"][l][h]
            assert np.all(np.isneginf(got[~has]))
            assert np.all(got[has] >= want[has] * (1 - 1e-6) - 1e-7)
            np.testing.assert_allclose(got[has], want[has], rtol=1e-5, atol=1e-6)
            child_c, child_r, child_ok = a["centers"][l][h], got, has
    return a


BUILD_CASES = [
    # trees, n, d, bf, levels, dtype, niter
    (2, 192, 64, 8, 3, torch.float32, 2),
    (1, 4096, 128, 16, 2, torch.float32, 10),
    (2, 2048, 128, 32, 3, torch.bfloat16, 1),
    (3, 203, 32, 4, 4, torch.float32, 1),      # n not a multiple of bf: pad slots
    (2, 333, 16, 5, 3, torch.bfloat16, 2),
    (2, 100, 64, 1, 2, torch.float32, 0),      # bf = 1: every key its own parent
    (1, 300, 64, 8, 1, torch.float32, 1),      # one level: keys only
    (2, 20, 32, 32, 3, torch.float32, 1),      # fewer keys than one block
    (1, 500, 256, 16, 2, torch.bfloat16, 1),
    (8, 8192, 128, 32, 3, torch.bfloat16, 1),
    (2, 1000, 64, 16, 3, torch.bfloat16, 1),   # tiled layout, partial tiles at every level
    (1, 3000, 256, 48, 2, torch.bfloat16, 1),
]


@pytest.mark.parametrize("case", BUILD_CASES, ids=[f"t{c[0]}_n{c[1]}_d{c[2]}_bf{c[3]}_L{c[4]}_"
                                                     f"{'bf16' if c[5] == torch.bfloat16 else 'f32'}_it{c[6]}"
                                                     for c in BUILD_CASES])
def test_build_layout_radii_and_search_parity(case, gpu_device):
    from hira_amd.indexer.hip import HIPIndexer
    from hira_amd.searcher.hip import HIPSearcher

    t, n, d, bf, nl, dtype, niter = case
    print(f"case {case}", flush=True)
    rnd = bf16_round if dtype == torch.bfloat16 else (lambda x: x)
    keys = rnd(clustered_keys(t, n, d, seed=7 + n, clusters=max(2, n // 40)))
    vals = rnd(np.random.default_rng(n).normal(size=(t, n, d)).astype(np.float32))
    idx = HIPIndexer(nl, niter, bf).build(torch.from_numpy(keys)[None].to(dtype),
                                           torch.from_numpy(vals)[None].to(dtype))
    torch.cuda.synchronize()
    _check_layout(idx, keys, vals, dtype)
    # search on the built tree == brute force, in insertion order
    h_q = t * 2
    q = rnd(random_query(h_q, d, seed=n + 1))
    q2kv = ho.default_q2kv(h_q, t)
    s = ho.scores(keys, q, q2kv)
    th = midpoint_threshold(s, max(1, n // 20))
    out = HIPSearcher(index_space="position").search(
        torch.from_numpy(q), torch.from_numpy(th), idx).cpu().numpy()
    assert_same_selection(out != 0, s, th)


def test_build_is_reproducible_and_seed_dependent(gpu_device):
    from hira_amd.indexer.hip import HIPIndexer

    keys = torch.from_numpy(normalized_keys(2, 1000, 64, seed=3))[None]
    a = HIPIndexer(3, 2, 8, seed=5).build(keys)
    b = HIPIndexer(3, 2, 8, seed=5).build(keys)
    c = HIPIndexer(3, 2, 8, seed=6).build(keys)
    torch.cuda.synchronize()
    assert not a.tiled
    assert torch.equal(a.perm, b.perm) and torch.equal(a.centers[2], b.centers[2])
    assert torch.equal(a.radii[1], b.radii[1])
    assert not torch.equal(a.perm, c.perm)


def test_lloyd_rounds_tighten_the_balls(gpu_device):
    """More k-means rounds -> smaller leaf balls on clustered data (sum of radii)."""
    from hira_amd.indexer.hip import HIPIndexer

    keys = torch.from_numpy(clustered_keys(1, 4096, 64, seed=11, clusters=128, spread=0.5))[None]
    r0 = HIPIndexer(2, 0, 32).build(keys).radii[1].sum().item()
    r5 = HIPIndexer(2, 5, 32).build(keys).radii[1].sum().item()
    assert r5 < r0


@pytest.mark.parametrize("dtype,d,n,same,bf,nl,niter", [
    (torch.float32, 64, 3000, 700, 16, 2, 2),      # a bucket of 700: sorting network in LDS
    (torch.bfloat16, 128, 8192, 3000, 16, 3, 2),   # 3000: packing sorts it in two goes
    (torch.float32, 32, 8192, 6000, 8, 2, 1),      # 6000: the mean orders it through a bit map
    (torch.bfloat16, 64, 140000, 5000, 32, 2, 1),  # ... with more item ids than one bit map holds
])
def test_buckets_far_larger_than_a_block(dtype, d, n, same, bf, nl, niter, gpu_device):
    """`same` copies of one key all have the same nearest centroid: one bucket of that many
    members in every round.  The layout holds, and two builds give the same tree bit for bit
    although the members of a bucket arrive in a different order in every run."""
    from hira_amd.indexer.hip import HIPIndexer

    print(f"case {dtype} d={d} n={n} same={same} bf={bf} levels={nl}", flush=True)
    rnd = bf16_round if dtype == torch.bfloat16 else (lambda x: x)
    rng = np.random.default_rng(n + same)
    keys = rnd(normalized_keys(2, n, d, seed=n))
    where = rng.permutation(n)[:same]
    keys[0, where] = keys[0, where[0]]
    keys[1, where] = keys[1, where[0]] * np.float32(0.5)
    kt = torch.from_numpy(keys)[None].to(dtype)
    a = HIPIndexer(nl, niter, bf, seed=3).build(kt, kt.clone())
    b = HIPIndexer(nl, niter, bf, seed=3).build(kt, kt.clone())
    torch.cuda.synchronize()
    _check_layout(a, keys, keys, dtype)
    assert torch.equal(a.perm, b.perm)
    for l in range(1, nl):
        assert torch.equal(a.centers[l], b.centers[l]) and torch.equal(a.radii[l], b.radii[l])
        assert torch.equal(a.counts[l], b.counts[l])


def test_tiled_and_row_major_builds_hold_the_same_tree(gpu_device):
    """The tile arrangement only moves 16-byte chunks around: same tree, same answers."""
    from hira_amd.indexer.hip import HIPIndexer, from_tiled, to_tiled

    keys = torch.from_numpy(bf16_round(clustered_keys(2, 2000, 128, seed=4)))[None].to(torch.bfloat16)
    a = HIPIndexer(3, 1, 32, layout="tiled").build(keys, keys.clone())
    b = HIPIndexer(3, 1, 32, layout="row_major").build(keys, keys.clone())
    torch.cuda.synchronize()
    assert a.tiled and not b.tiled and a.cap[0] % 16 == 0
    assert torch.equal(a.perm[:, : a.size[0]], b.perm[:, : b.size[0]])
    assert torch.equal(a.keys_rowmajor(), b.keys_rowmajor())
    assert torch.equal(a.children, b.children) and torch.equal(a.parents, b.parents)
    for l in (1, 2):
        assert torch.equal(a.centers_rowmajor(l), b.centers_rowmajor(l))
        assert torch.equal(a.radii[l][:, : a.size[l]], b.radii[l][:, : b.size[l]])
        assert torch.equal(a.counts[l][:, : a.size[l]], b.counts[l][:, : b.size[l]])
    assert torch.equal(a.values, b.values)
    x = torch.randn(3, 48, 96)
    assert torch.equal(from_tiled(to_tiled(x)), x)


def test_reference_attribute_views(gpu_device):
    """Names and shapes other code reads from the reference's GPU indexer
    (tests/test_cuda_indexer_searcher.py:134-176 of the reference)."""
    from hira_amd.indexer.hip import HIPIndexer

    h, n, d, bf = 2, 203, 32, 4
    keys = torch.from_numpy(normalized_keys(h, n, d, seed=1))[None]
    idx = HIPIndexer(HIPIndexer.DEPTH.THREE_LEVELS, 1, bf).build(keys, keys.clone())
    m = -(-n // bf)
    g = -(-m // bf)
    assert idx.depth == HIPIndexer.DEPTH.THREE_LEVELS
    assert tuple(idx.children.shape) == (h, g * bf * bf, d)
    assert tuple(idx.values.shape) == (1, h, g * bf * bf, d)
    assert tuple(idx.parents.shape) == (h, g * bf, d)
    assert tuple(idx.parent_radii.shape) == (h, g * bf)
    assert tuple(idx.grand_parents.shape) == (h, g, d)
    assert tuple(idx.grand_parent_radii.shape) == (h, g)
    assert idx.num_heads == h and idx.dim == d and idx.branching_factor == bf
    cc = idx._child_counts
    assert int(cc.sum()) == h * n and int(cc.min()) >= 0 and int(cc.max()) <= bf
    assert int(idx._parent_valid.sum()) == h * m
    assert int(idx._gp_child_counts.sum()) == h * m
    assert HIPIndexer(2, 1, bf).build(keys).values is None


def test_build_rejects_bad_shapes(gpu_device):
    from hira_amd.indexer.hip import HIPIndexer

    with pytest.raises(ValueError):
        HIPIndexer(2, 1, 8).build(torch.zeros(2, 10, 64))           # not 4-D
    with pytest.raises(ValueError):
        HIPIndexer(2, 1, 8).build(torch.zeros(1, 2, 10, 6))         # rows not 16-byte multiples
    with pytest.raises(ValueError):
        HIPIndexer(2, 1, 8).build(torch.zeros(1, 2, 10, 64), torch.zeros(1, 2, 9, 64))
    with pytest.raises(ValueError):
        HIPIndexer(9, 1, 8)
    with pytest.raises(ValueError):
        HIPIndexer(2, 1, 65)


@pytest.mark.parametrize("dtype,d,bf", [(torch.bfloat16, 128, 32), (torch.float32, 32, 8),
                                        (torch.bfloat16, 64, 16)])
def test_build_of_trees_with_different_numbers_of_keys(dtype, d, bf, gpu_device):
    """hira_build_ragged (HIPIndexer.build(key_counts=...)): every tree gets the layout of n keys
    but holds only its first n_t; each of those sits in exactly one slot, the others in none;
    a tree uses ceil(n_t / bf) nodes, counts are exact, radii cover, an empty tree is all empty;
    the search over every tree is the brute-force search over its own keys."""
    from hira_amd.indexer.hip import HIPIndexer
    from hira_amd.searcher.hip import HIPSearcher

    n = bf * bf
    counts = [n, n // 3 + 5, 1, 0, bf, bf + 1]
    t = len(counts)
    rnd = bf16_round if dtype == torch.bfloat16 else (lambda x: x)
    keys = rnd(clustered_keys(t, n, d, seed=11, clusters=10))
    vals = rnd(np.random.default_rng(2).normal(size=(t, n, d)).astype(np.float32))
    kc = torch.tensor(counts, dtype=torch.int32, device="cuda")
    idx = HIPIndexer(2, 2, bf).build(torch.from_numpy(keys)[None].to(dtype),
                                     torch.from_numpy(vals)[None].to(dtype), key_counts=kc)
    assert idx.size == [n, bf]
    got = _download(idx)
    for h, n_t in enumerate(counts):
        perm = got["perm"][h]
        ok = perm >= 0
        assert np.array_equal(np.sort(perm[ok]), np.arange(n_t))
        assert np.array_equal(got["keys"][h][ok], keys[h][perm[ok]])
        assert np.array_equal(got["values"][h][ok], vals[h][perm[ok]])
        blk = ok.reshape(bf, bf)
        cnt = got["counts"][1][h]
        assert np.array_equal(cnt, blk.sum(1))
        assert np.all(blk[:, :-1] >= blk[:, 1:])            # a node's keys fill it from slot 0
        used = -(-n_t // bf)
        assert (cnt[used:] == 0).all() and (cnt[:used] > 0).all()
        rad, cen = got["radii"][1][h], got["centers"][1][h]
        assert np.all(rad[cnt == 0] == -np.inf)
        need = ho.radii_from_layout(got["keys"][h], np.zeros(n, np.float32), ok, cen, bf)
        assert np.all(rad[cnt > 0] >= need[cnt > 0] * (1 - 1e-6) - 1e-6)
    q = rnd(random_query(t, d, seed=4))
    s = ho.scores(keys, q, np.arange(t))
    s = np.where(np.arange(n)[None] < np.array(counts)[:, None], s, -np.inf).astype(np.float32)
    # thresholds that keep about a tenth of a tree's keys (its only key; nothing of an empty tree)
    th = np.array([np.sort(s[h])[::-1][min(counts[h] // 10, counts[h] - 1)] if counts[h] else 0.0
                   for h in range(t)], np.float32) - 1e-3
    out = HIPSearcher(index_space="position").search(torch.from_numpy(q), torch.from_numpy(th), idx)
    out = out.cpu().numpy()
    assert out.shape[1] == n
    assert_same_selection(out != 0, s, th)
    with pytest.raises(ValueError):
        HIPIndexer(3, 1, bf).build(torch.from_numpy(keys)[None].to(dtype), key_counts=kc)


@pytest.mark.parametrize("dtype,dv", [(torch.bfloat16, 8), (torch.float32, 12), (torch.bfloat16, 40)])
def test_value_rows_of_any_width_follow_their_keys(dtype, dv, gpu_device):
    """Value rows narrower and wider than the keys, of one to five 16-byte chunks: every slot
    holds the value of the key it holds."""
    from hira_amd.indexer.hip import HIPIndexer

    t, n, d, bf = 2, 700, 64, 8
    rnd = bf16_round if dtype == torch.bfloat16 else (lambda x: x)
    keys = rnd(clustered_keys(t, n, d, seed=77, clusters=20))
    vals = rnd(np.random.default_rng(dv).normal(size=(t, n, dv)).astype(np.float32))
    idx = HIPIndexer(3, 1, bf).build(torch.from_numpy(keys)[None].to(dtype),
                                     torch.from_numpy(vals)[None].to(dtype))
    perm = idx.perm.cpu().numpy()
    got_v = idx.values_buf[:, : idx.size[0]].float().cpu().numpy()
    got_k = idx.keys_rowmajor()[:, : idx.size[0]].float().cpu().numpy()
    for h in range(t):
        ok = perm[h, : idx.size[0]] >= 0
        assert ok.sum() == n
        assert np.array_equal(got_v[h][ok], vals[h][perm[h, : idx.size[0]][ok]])
        assert np.array_equal(got_k[h][ok], keys[h][perm[h, : idx.size[0]][ok]])
