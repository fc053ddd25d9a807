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
