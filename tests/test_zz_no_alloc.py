"""hira_search_noalloc (the search for callers that cannot allocate: its scratch is a buffer
inside the library's device image) against hira_search with a caller's workspace: the same
attention output bit for bit, on two calls in a row, the second over a smaller index; sizes
beyond the built-in buffer are refused."""
import ctypes as C

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _index(trees, n, d, bf, nl, seed):
    from hira_amd.indexer import HIPIndexer

    g = torch.Generator().manual_seed(seed)
    keys = torch.randn((1, trees, n, d), generator=g).to(torch.bfloat16)
    vals = torch.randn((1, trees, n, d), generator=g).to(torch.bfloat16)
    return HIPIndexer(nl, 1, bf).build(keys.cuda(), vals.cuda()), keys


def _both(idx, keys, h_q, seed, keep, kernel=0, queue=None):
    """One step through hira_search (workspace from the caller) and one through
    hira_search_noalloc; returns both outputs."""
    from hira_amd import _lib
    from hira_amd.cache.threshold_finder import exact_topk
    from hira_amd.searcher import HIPSearcher

    lib = _lib.lib()
    g = torch.Generator().manual_seed(seed)
    d = idx.dim
    q = torch.randn((h_q, d), generator=g).to(torch.bfloat16).cuda()
    tau = exact_topk(keys[0].cuda(), q, keep)
    se = HIPSearcher(kernel=kernel)
    scale = torch.full((h_q,), d ** -0.5)
    qk = qv = None
    if queue:
        qk = torch.randn((idx.num_trees, queue, d), generator=g).to(torch.bfloat16).cuda()
        qv = torch.randn((idx.num_trees, queue, d), generator=g).to(torch.bfloat16).cuda()
    want = se.search_attention(q, tau, idx, scaling=scale, queue_keys=qk, queue_values=qv).clone()
    qs, keep_alive = se._query_struct(q, tau, idx, None, scale)
    out = torch.full((h_q, idx.vdim), float("nan"), dtype=torch.float32, device="cuda")
    so = _lib.HiraSearchOut()
    so.attn_out = out.data_ptr()
    tree = idx.tree_struct()
    hq = None
    if queue:
        hq = _lib.HiraQueue(qk.data_ptr(), qv.data_ptr(), queue, queue)
    rc = lib.hira_search_noalloc(C.byref(tree), C.byref(qs), C.byref(hq) if hq else None,
                                 C.byref(so), C.byref(se.launch),
                                 torch.cuda.current_stream().cuda_stream)
    _lib.check(rc)
    torch.cuda.synchronize()
    del keep_alive
    return want, out


def test_noalloc_matches_workspace_search_twice_second_smaller(gpu_device):
    big, kbig = _index(8, 8192, 128, 32, 3, seed=1)
    small, ksmall = _index(2, 1500, 128, 32, 3, seed=2)
    want, got = _both(big, kbig, 32, seed=3, keep=80)
    assert bool(torch.isfinite(got).all()) and torch.equal(got, want)
    want, got = _both(small, ksmall, 8, seed=4, keep=20)       # fewer trees, heads and partials
    assert torch.equal(got, want)
    want, got = _both(big, kbig, 32, seed=5, keep=200, queue=5)  # and larger again, with a queue
    assert torch.equal(got, want)


def test_noalloc_vector_kernel_and_fp32(gpu_device):
    """The vector-ALU kernel folds through the same scratch (one head per tree: fused fold)."""
    from hira_amd.indexer import HIPIndexer

    g = torch.Generator().manual_seed(9)
    keys = torch.randn((1, 3, 700, 64), generator=g)
    vals = torch.randn((1, 3, 700, 64), generator=g)
    idx = HIPIndexer(2, 1, 8).build(keys.cuda(), vals.cuda())
    from hira_amd import _lib
    from hira_amd.cache.threshold_finder import exact_topk
    from hira_amd.searcher import HIPSearcher

    q = torch.randn((3, 64), generator=g).cuda()
    tau = exact_topk(keys[0].cuda(), q, 30)
    se = HIPSearcher()
    scale = torch.full((3,), 0.125)
    want = se.search_attention(q, tau, idx, scaling=scale).clone()
    qs, keep_alive = se._query_struct(q, tau, idx, None, scale)
    out = torch.empty((3, 64), dtype=torch.float32, device="cuda")
    so = _lib.HiraSearchOut()
    so.attn_out = out.data_ptr()
    tree = idx.tree_struct()
    _lib.check(_lib.lib().hira_search_noalloc(C.byref(tree), C.byref(qs), None, C.byref(so),
                                              C.byref(se.launch),
                                              torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert torch.equal(out, want)


def test_noalloc_refuses_what_does_not_fit(gpu_device):
    """64 sequences x 8 trees with 32 heads each and 16 workgroups per tree need more partials
    than the built-in buffer holds: a clear error, nothing launched."""
    from hira_amd import _lib
    from hira_amd.searcher import HIPSearcher

    idx, keys = _index(256, 4096, 128, 32, 3, seed=7)
    h_q = 256 * 8
    q = torch.zeros((h_q, 128), dtype=torch.bfloat16, device="cuda")
    tau = torch.zeros((h_q,), device="cuda")
    se = HIPSearcher(nodes_per_wave=1)
    qs, keep_alive = se._query_struct(q, tau, idx, None, None)
    out = torch.zeros((h_q, 128), dtype=torch.float32, device="cuda")
    so = _lib.HiraSearchOut()
    so.attn_out = out.data_ptr()
    tree = idx.tree_struct()
    rc = _lib.lib().hira_search_noalloc(C.byref(tree), C.byref(qs), None, C.byref(so),
                                        C.byref(se.launch), torch.cuda.current_stream().cuda_stream)
    assert rc == -3
    msg = _lib.lib().hira_last_error().decode()
    assert "scratch buffer" in msg, msg
    with pytest.raises(RuntimeError):
        _lib.check(rc)


def test_noalloc_under_graph_capture_after_a_warm_up(gpu_device):
    """One eager call resolves the scratch buffer's address; after it the call records nothing
    but the kernel launch, so it can be captured: the graph is replayed for three different
    queries, with eager work and synchronisations between the replays, and every replay equals
    hira_search with a caller's workspace bit for bit."""
    from hira_amd import _lib
    from hira_amd.cache.threshold_finder import exact_topk
    from hira_amd.searcher import HIPSearcher

    idx, keys = _index(4, 4096, 128, 32, 3, seed=11)
    h_q, d = 16, 128
    _both(idx, keys, h_q, seed=12, keep=40)                     # the warm-up call, eager
    lib, se = _lib.lib(), HIPSearcher()
    scale = torch.full((h_q,), d ** -0.5)
    q = torch.zeros((h_q, d), dtype=torch.bfloat16, device="cuda")      # fixed buffers the graph reads
    tau = torch.zeros((h_q,), dtype=torch.float32, device="cuda")
    out = torch.zeros((h_q, d), dtype=torch.float32, device="cuda")
    qs, keep_alive = se._query_struct(q, tau, idx, None, scale)
    assert qs.q == q.data_ptr() and qs.tau == tau.data_ptr()    # the launch reads the fixed buffers
    so = _lib.HiraSearchOut()
    so.attn_out = out.data_ptr()
    tree = idx.tree_struct()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            _lib.check(lib.hira_search_noalloc(C.byref(tree), C.byref(qs), None, C.byref(so),
                                               C.byref(se.launch),
                                               torch.cuda.current_stream().cuda_stream))
    torch.cuda.current_stream().wait_stream(side)
    g = torch.Generator().manual_seed(13)
    for step in range(3):
        qn = torch.randn((h_q, d), generator=g).to(torch.bfloat16).cuda()
        tn = exact_topk(keys[0].cuda(), qn, 30 + 25 * step)
        want = se.search_attention(qn, tn, idx, scaling=scale).clone()  # eager work between replays
        q.copy_(qn)
        tau.copy_(tn)
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), f"replay {step}"
    del keep_alive
