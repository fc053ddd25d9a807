"""Properties that hold at any size, checked at the benchmark's full sizes (configurations 2
and 4 of hira_amd.synth: 8 x 32768 and 8 x 131072 keys), where the CPU oracle would take too
long to be the checker: exactly k keys selected per head with the k best scores, doubling
the values doubles the output bit for bit, every key selected == dense attention, a repeated
call repeats its result."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("cfg", [2, 4])
def test_size_independent_properties_at_full_size(cfg, gpu_device):
    from hira_amd import synth
    from hira_amd.cache.threshold_finder import exact_topk
    from hira_amd.indexer import HIPIndexer
    from hira_amd.searcher import HIPSearcher

    w = synth.WORKLOADS[cfg]
    print(f"workload {w.name}", flush=True)
    keys, values = synth.make_kv(w)
    q = synth.make_queries(w, keys, 2).cuda().reshape(2, w.h_q, w.d)
    kd, vd = keys.cuda(), values.cuda()
    k = int(np.ceil(w.select_frac[0] * w.n))
    idx = HIPIndexer(w.num_levels, w.kmeans_iters, w.bf).build(kd, vd)
    idx2 = HIPIndexer(w.num_levels, w.kmeans_iters, w.bf).build(kd, vd * 2)   # same tree, values doubled
    assert torch.equal(idx.perm, idx2.perm)
    se = HIPSearcher()
    sc = torch.full((w.h_q,), w.d ** -0.5)
    for i in range(2):
        tau = exact_topk(kd[0], q[i], k)
        # exactly the k best keys of every head
        sel_idx, sel_sco, cnt = se.search_compact(q[i], tau, idx, capacity=2 * k)
        assert bool((cnt == k).all()), cnt.tolist()
        s = torch.einsum("hnd,hgd->hgn", kd[0].float(), q[i].view(w.h_kv, w.group, w.d).float())
        want = s.reshape(w.h_q, -1).topk(k, dim=-1).values
        got = sel_sco[:, :k].sort(dim=-1, descending=True).values
        assert torch.allclose(got, want, rtol=2e-5, atol=1e-6 * float(want.abs().max()))
        # the listed slots hold exactly those keys
        pos = torch.gather(idx.perm.long().repeat_interleave(w.group, 0), 1, sel_idx[:, :k].long())
        assert int(pos.min()) >= 0
        assert torch.equal(pos.sort(dim=-1).values,
                           s.reshape(w.h_q, -1).topk(k, dim=-1).indices.sort(dim=-1).values)
        # repeated call, doubled values
        a = se.search_attention(q[i], tau, idx, scaling=sc).clone()
        assert torch.equal(a, se.search_attention(q[i], tau, idx, scaling=sc))
        assert torch.equal(se.search_attention(q[i], tau, idx2, scaling=sc), 2 * a)
    # every key selected: dense attention
    everything = torch.full((w.h_q,), -3.0e38)
    dense = se.search_attention(q[0], everything, idx, scaling=sc)
    ref = torch.nn.functional.scaled_dot_product_attention(
        q[0].view(1, w.h_q, 1, w.d).float(),
        kd.float().repeat_interleave(w.group, 1), vd.float().repeat_interleave(w.group, 1),
        scale=w.d ** -0.5).reshape(w.h_q, w.d)
    err = ((dense - ref).abs().max(dim=1).values / ref.abs().max(dim=1).values).max()
    assert float(err) <= 2e-3, float(err)


def _check_tree_on_device(idx, keys_all):
    """The structure check of the update tests, in torch on the GPU: every key present once and
    in its slot, children packed from slot 0, every radius covers its subtree."""
    t, n, d = keys_all.shape
    bf, nl = idx.branching_factor, idx.num_levels
    s0 = idx.size[0]
    perm = idx.perm[:, :s0].long()
    ok = perm >= 0
    kr = idx.keys_rowmajor()[:, :s0].float()
    for h in range(t):
        assert torch.equal(perm[h][ok[h]].sort().values, torch.arange(n, device=perm.device))
        assert torch.equal(kr[h][ok[h]], keys_all[h][perm[h][ok[h]]].float())
    child_c, child_r, child_ok = kr, torch.zeros_like(kr[..., 0]), ok
    for l in range(1, nl):
        k = idx.size[l]
        cen = idx.centers_rowmajor(l)[:, :k].float()
        rad = idx.radii[l][:, :k]
        cnt = idx.counts[l][:, :k]
        short = k * bf - child_ok.shape[1]
        if short > 0:
            child_c = torch.cat([child_c, child_c.new_zeros((t, short, d))], 1)
            child_r = torch.cat([child_r, child_r.new_zeros((t, short))], 1)
            child_ok = torch.cat([child_ok, child_ok.new_zeros((t, short))], 1)
        blk = child_ok[:, : k * bf].reshape(t, k, bf)
        assert torch.equal(cnt.long(), blk.sum(-1)), f"counts of level {l}"
        assert bool((blk[..., :-1] >= blk[..., 1:]).all()), f"children of level {l} not packed"
        dist = (child_c[:, : k * bf].reshape(t, k, bf, d) - cen[:, :, None]).norm(dim=-1)
        reach = torch.where(blk, dist + child_r[:, : k * bf].reshape(t, k, bf),
                            torch.full_like(dist, float("-inf"))).max(dim=-1).values
        has = cnt > 0
        assert bool((rad[has] >= reach[has] * (1 - 1e-5) - 1e-5).all()), f"radius of level {l}"
        child_c, child_r, child_ok = cen, torch.where(has, rad, torch.zeros_like(rad)), has


def test_build_and_growth_keep_the_tree_valid_at_full_size(gpu_device):
    """cfg 4's index (8 x 131072 keys, 4 levels): valid after the build, after a window that
    is grafted, after single appends and after a subtree rebuild."""
    from hira_amd import synth
    from hira_amd.indexer import HIPIndexer

    w = synth.WORKLOADS[4]
    keys, values = synth.make_kv(w)
    more, _ = synth.make_stream(w, 2048 + 40)
    kd, vd, md = keys.cuda(), values.cuda(), more.cuda()
    idx = HIPIndexer(w.num_levels, w.kmeans_iters, w.bf).build(kd, vd)
    _check_tree_on_device(idx, kd[0])
    idx.update(md[:, :, :2048], md[:, :, :2048])
    for i in range(2048, 2088):
        idx.update(md[:, :, i:i + 1], md[:, :, i:i + 1], sync=False)
    idx.rebuild_subtree(3)
    assert idx.num_keys == w.n + 2088
    _check_tree_on_device(idx, torch.cat([kd[0], md[0]], dim=1))


@pytest.mark.parametrize("n,heads", [(131072, 4), (200000, 8), (33000, 4)])
def test_lone_tree_is_scanned_by_many_workgroups(n, heads, gpu_device):
    """One tree alone on the chip: the launch plan gives it up to 128 workgroups (a head then has
    up to 128 partials to fold) or, at 33000 keys, workgroups of unequal tile counts.  The sparse
    output must equal softmax over exactly the k best keys (fp64 on the device, 2e-3 through the
    bf16 storage), and every key selected must equal dense attention."""
    from hira_amd.cache.threshold_finder import exact_topk
    from hira_amd.indexer import HIPIndexer
    from hira_amd.searcher import HIPSearcher

    g = torch.Generator().manual_seed(n)
    d = 128
    K = torch.randn(1, 1, n, d, generator=g).bfloat16().cuda()
    V = torch.randn(1, 1, n, d, generator=g).bfloat16().cuda()
    q = torch.randn(heads, d, generator=g).bfloat16().cuda()
    idx = HIPIndexer(3, 1, 32).build(K, V)
    k = n // 200
    tau = exact_topk(K[0], q, k)
    sc = torch.full((heads,), d ** -0.5)
    se = HIPSearcher()
    out = se.search_attention(q, tau, idx, scaling=sc)
    assert torch.equal(out, se.search_attention(q, tau, idx, scaling=sc))
    s = (q.double() @ K[0, 0].double().T)                      # (heads, n)
    top = s.topk(k, dim=-1)
    w = torch.softmax(top.values * d ** -0.5, dim=-1)
    ref = torch.einsum("hk,hkd->hd", w, V[0, 0].double()[top.indices])
    err = ((out.double() - ref).abs().max(dim=1).values / ref.abs().max(dim=1).values).max()
    assert float(err) <= 2e-3, float(err)
    dense = se.search_attention(q, torch.full((heads,), -3.0e38), idx, scaling=sc)
    refd = torch.softmax(s * d ** -0.5, dim=-1) @ V[0, 0].double()
    err = ((dense.double() - refd).abs().max(dim=1).values / refd.abs().max(dim=1).values).max()
    assert float(err) <= 2e-3, float(err)


def test_large_fp32_trees_on_the_vector_kernel(gpu_device):
    """fp32 keys (the vector-ALU kernel) at a size where a wavefront takes several steps of nodes
    so that a head has fewer partials to fold: the sparse output equals softmax over exactly the k
    best keys of every head (fp64 on the device, 1e-5)."""
    from hira_amd.cache.threshold_finder import exact_topk
    from hira_amd.indexer import HIPIndexer
    from hira_amd.searcher import HIPSearcher

    g = torch.Generator().manual_seed(5)
    t, grp, n, d = 4, 2, 65536, 128
    K = torch.randn(1, t, n, d, generator=g).cuda()
    V = torch.randn(1, t, n, d, generator=g).cuda()
    q = torch.randn(t * grp, d, generator=g).cuda()
    idx = HIPIndexer(3, 1, 32).build(K, V)
    k = 300
    tau = exact_topk(K[0], q, k)
    sc = torch.full((t * grp,), d ** -0.5)
    out = HIPSearcher().search_attention(q, tau, idx, scaling=sc)
    s = torch.einsum("tgd,tnd->tgn", q.view(t, grp, d).double(), K[0].double())
    top = s.topk(k, dim=-1)
    w = torch.softmax(top.values * d ** -0.5, dim=-1)
    vsel = torch.gather(V[0].double()[:, None].expand(t, grp, n, d), 2,
                        top.indices[..., None].expand(t, grp, k, d))
    ref = torch.einsum("tgk,tgkd->tgd", w, vsel).reshape(t * grp, d)
    err = ((out.double() - ref).abs().max(dim=1).values / ref.abs().max(dim=1).values).max()
    assert float(err) <= 1e-5, float(err)


FOLD_CASES = [
    # trees, keys per tree, heads a tree, keys kept per head, tiles per workgroup (0 = plan's choice)
    (8, 32768, 4, 328, 0),      # the benchmark's shape: 32 partials a head, single round
    (1, 131072, 4, 655, 0),     # a lone tree: 128 partials a head
    (1, 200000, 8, 1000, 0),    # 8 heads a tree, 98 workgroups of unequal tile counts
    (32, 32768, 4, 200, 0),     # more workgroups than compute units: several rounds of them
    (8, 16384, 4, 160, 1),      # one tile a workgroup by request: 32 partials, every wave one node
    (4, 8192, 16, 80, 0),       # 16 heads a tree
]


@pytest.mark.parametrize("t,n,g,keep,tpw", FOLD_CASES)
def test_fused_fold_equals_the_fold_of_a_second_launch(t, n, g, keep, tpw, gpu_device):
    """The search kernel's last workgroup of a tree folds the tree's attention partials inside the
    launch, behind a hand-off that rests on the completion of write-through stores; asked for
    (`separate_merge`), the partials are folded by a second launch instead, which sees them behind
    the kernel boundary.  Both must give the same output: a partial that the in-launch fold read
    too early (stale, or not yet there) would show as a difference far above rounding.  The two
    folds add the partials up in different orders, so the comparison is to 2e-6 of a head's
    largest output, not bit for bit; each path must repeat its own result bit for bit."""
    from hira_amd.cache.threshold_finder import exact_topk
    from hira_amd.indexer import HIPIndexer
    from hira_amd.searcher import HIPSearcher

    gen = torch.Generator().manual_seed(1000 * t + g)
    d, h = 128, t * g
    K = torch.randn(1, t, n, d, generator=gen).bfloat16().cuda()
    V = torch.randn(1, t, n, d, generator=gen).bfloat16().cuda()
    idx = HIPIndexer(3, 1, 32).build(K, V)
    sc = torch.full((h,), d ** -0.5)
    fused = HIPSearcher(kernel=2, nodes_per_wave=tpw)
    apart = HIPSearcher(kernel=2, nodes_per_wave=tpw, separate_merge=True)
    for step in range(3):   # fresh queries: the workspace's partials are overwritten every time
        q = torch.randn(h, d, generator=gen).bfloat16().cuda()
        tau = exact_topk(K[0], q, keep)
        a = fused.search_attention(q, tau, idx, scaling=sc).clone()
        b = apart.search_attention(q, tau, idx, scaling=sc).clone()
        scale = b.abs().max(dim=1, keepdim=True).values
        assert float(((a - b).abs() / scale).max()) <= 2e-6, (step, float(((a - b).abs() / scale).max()))
        assert torch.equal(a, fused.search_attention(q, tau, idx, scaling=sc))
        assert torch.equal(b, apart.search_attention(q, tau, idx, scaling=sc))
    # against the definition, once (the last step's queries, a few trees): softmax over exactly
    # the kept keys
    for i in range(min(t, 3)):
        qi = q[i * g:(i + 1) * g].double()
        s = qi @ K[0, i].double().T
        top = s.topk(keep, dim=-1)
        w = torch.softmax(top.values * d ** -0.5, dim=-1)
        ref = torch.einsum("hk,hkd->hd", w, V[0, i].double()[top.indices])
        got = a[i * g:(i + 1) * g].double()
        err = ((got - ref).abs().max(dim=1).values / ref.abs().max(dim=1).values).max()
        assert float(err) <= 2e-3, (i, float(err))
