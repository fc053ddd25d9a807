"""GPU tests of hira_threshold (through threshold_finder on device tensors): the two sample
rules the reference names (cache/threshold_finder.py:1-14) against a float64 restatement, and
sample thresholds feeding the search."""
import numpy as np
import pytest
import torch

from oracle import hira_oracle as ho
from helpers import bf16_round, clustered_keys, random_query

pytestmark = pytest.mark.gpu

CASES = [
    # trees, samples, d, heads, dtype, k
    (2, 1000, 128, 8, torch.bfloat16, 10),
    (8, 1000, 128, 32, torch.bfloat16, 32),
    (1, 4096, 64, 4, torch.float32, 4096),    # k = all samples: the mean score
    (3, 37, 32, 3, torch.float32, 1),         # k = 1: the maximum; ragged sample count
    (2, 1, 256, 4, torch.bfloat16, 1),        # one sample
    (4, 513, 16, 16, torch.bfloat16, 100),    # just past a power of two
    (2, 1024, 64, 4, torch.float32, 16),      # the most that the few-of-many path takes
    (2, 65, 32, 8, torch.bfloat16, 7),        # a second wave holding a single score
    (1, 1500, 128, 4, torch.bfloat16, 12),    # two registers per sorting thread, ragged last pass
]


@pytest.mark.parametrize("case", CASES, ids=[f"t{c[0]}_s{c[1]}_d{c[2]}_h{c[3]}_k{c[5]}_"
                                             f"{'bf16' if c[4] == torch.bfloat16 else 'f32'}" for c in CASES])
def test_sample_thresholds_match_float64(case, gpu_device):
    from hira_amd.cache import threshold_finder as tf

    t, s, d, h, dtype, k = case
    print(f"case {case}", flush=True)
    rnd = bf16_round if dtype == torch.bfloat16 else (lambda x: x)
    x = rnd(clustered_keys(t, s, d, seed=3 + s, clusters=max(1, s // 40)))
    q = rnd(random_query(h, d, seed=11 + s))
    xd = torch.from_numpy(x).to(dtype).cuda()
    qd = torch.from_numpy(q).to(dtype).cuda()
    scale = float(np.abs(ho.sample_thresholds(x, q, "sample_max")).max()) + 1e-6
    got = tf.sample_max(xd, qd).cpu().numpy()
    assert np.abs(got - ho.sample_thresholds(x, q, "sample_max")).max() <= 1e-5 * scale
    got = tf.sample_mean_topk(xd, qd.view(1, h, 1, d), k).cpu().numpy()
    assert np.abs(got - ho.sample_thresholds(x, q, "sample_mean_topk", k)).max() <= 1e-5 * scale
    if k == 1:
        assert np.array_equal(got, tf.sample_max(xd, qd).cpu().numpy())
    # a head map that is not the default one (tests/test_cpp_kernels.py:529-565 of the reference)
    m = torch.from_numpy(np.random.default_rng(s).integers(0, t, size=h))
    got = tf.sample_mean_topk(xd, qd, k, m).cpu().numpy()
    assert np.abs(got - ho.sample_thresholds(x, q, "sample_mean_topk", k, m.numpy())).max() <= 1e-5 * scale


def test_sample_threshold_rejects_bad_input(gpu_device):
    from hira_amd.cache import threshold_finder as tf

    x = torch.randn(2, 100, 32, device="cuda")
    q = torch.randn(4, 32, device="cuda")
    with pytest.raises(ValueError):
        tf.sample_max(x, torch.randn(4, 16, device="cuda"))        # dims differ
    with pytest.raises(ValueError):
        tf.sample_max(x, torch.randn(3, 32, device="cuda"))        # 3 heads over 2 trees
    with pytest.raises(ValueError):
        tf.sample_max(torch.randn(2, 5000, 32, device="cuda"), q)  # too many samples
    with pytest.raises(ValueError):
        tf.sample_max(x.half(), q)                                   # dtype
    with pytest.raises(ValueError):
        tf.device_thresholds(x[:, :, :30].contiguous(), q[:, :30].contiguous(), "sample_max")  # 120-byte rows


def test_sample_threshold_feeds_the_search(gpu_device):
    """tau from a 1000-key sample, left on the device, then the search: the selected set is
    exactly {k : q.k >= tau} for that tau."""
    from hira_amd.cache import threshold_finder as tf
    from hira_amd.indexer.hip import HIPIndexer
    from hira_amd.searcher.hip import HIPSearcher
    from helpers import assert_same_selection

    t, n, d, h = 2, 6000, 128, 8
    keys = bf16_round(clustered_keys(t, n, d, seed=4, clusters=60))
    q = bf16_round(random_query(h, d, seed=5))
    K = torch.from_numpy(keys)[None].to(torch.bfloat16).cuda()
    idx = HIPIndexer(3, 1, 32).build(K)
    pick = torch.randperm(n, generator=torch.Generator().manual_seed(0))[:1000].cuda()
    samples = K[0][:, pick].contiguous()
    qd = torch.from_numpy(q).to(torch.bfloat16).cuda()
    tau = tf.sample_mean_topk(samples, qd, 20)
    out = HIPSearcher(index_space="position").search(qd, tau, idx)
    s = ho.scores(keys, q, ho.default_q2kv(h, t))
    assert_same_selection(out.cpu().numpy() != 0, s, tau.cpu().numpy())
    frac = float((out != 0).float().mean())
    assert 0.0 < frac < 0.2, frac


def test_cache_layer_uses_its_sample_rule(gpu_device):
    """With no threshold passed in, the attention function takes tau from the cache layer's key
    sample by the configured rule: output == softmax attention over {indexed keys with
    q.k >= tau} and the queued keys, tau recomputed on the host from the same sample."""
    from hira_amd.attention import hira_attention_forward
    from hira_amd.cache.hira_cache import HiraCacheLayer
    from hira_amd.cache.hira_config import DeviceMode, HiraConfig
    from helpers import rel_err

    cfg = HiraConfig(device_mode=DeviceMode.CUDA_ONLY, update_every=4, num_levels=3,
                     branching_factor=16, threshold_method="sample_mean_topk", sample_size=200,
                     threshold_topk=5)
    layer = HiraCacheLayer(cfg.device_mode, cfg.update_every, cfg.get_indexer_kwargs(),
                           cfg.get_searcher_kwargs(), cfg.get_threshold_kwargs())
    h_kv, h_q, d, n0 = 2, 8, 64, 1500
    keys = bf16_round(clustered_keys(h_kv, n0 + 6, d, seed=8, clusters=30))
    vals = bf16_round(np.random.default_rng(2).normal(size=(h_kv, n0 + 6, d)).astype(np.float32))
    K = torch.from_numpy(keys)[None].to(torch.bfloat16).cuda()
    V = torch.from_numpy(vals)[None].to(torch.bfloat16).cuda()
    out, _ = layer.update(K[:, :, :n0], V[:, :, :n0])
    assert out.samples.shape == (h_kv, 200, d) and out.threshold_method == "sample_mean_topk"
    samples = out.samples.float().cpu().numpy()
    q2kv = ho.default_q2kv(h_q, h_kv)
    sc = np.full(h_q, d ** -0.5, np.float32)
    compared = 0
    for step in range(6):
        n = n0 + step + 1
        out, _ = layer.update(K[:, :, n - 1:n], V[:, :, n - 1:n])
        q = bf16_round(random_query(h_q, d, seed=40 + step))
        qd = torch.from_numpy(q).to(torch.bfloat16).cuda().view(1, h_q, 1, d)
        att, _ = hira_attention_forward(None, qd, out, None, scaling=d ** -0.5)
        tau = ho.sample_thresholds(samples, q, "sample_mean_topk", 5)
        s = ho.scores(keys[:, :n], q, q2kv)
        mask = s >= tau[:, None]
        mask[:, layer.indexed_len:] = True          # the queue is always attended
        band = np.abs(s - tau[:, None]) <= 1e-5 * np.abs(tau[:, None])
        if band[:, : layer.indexed_len].any():      # a score within rounding of tau: either answer is right
            continue
        compared += 1
        ref = ho.attention(keys[:, :n], vals[:, :n], q, sc, mask, q2kv)
        # (2e-3 for the attention plus the rounding of the returned tensor to bf16)
        assert rel_err(att.float().cpu().numpy().reshape(h_q, d), ref) <= 2e-3 + 2.0 ** -8, step
        assert 0 < mask[:, : layer.indexed_len].mean() < 0.5
    assert compared >= 3


def test_decode_step_in_a_hip_graph(gpu_device):
    """Thresholds + search + attention captured once and replayed with new queries, with eager
    work and synchronisation between the replays: every replay equals the eager result."""
    from hira_amd.indexer.hip import HIPIndexer
    from hira_amd.searcher.hip import HIPSearcher

    t, n, d, h = 4, 5000, 128, 16
    keys = bf16_round(clustered_keys(t, n, d, seed=14, clusters=50))
    K = torch.from_numpy(keys)[None].to(torch.bfloat16).cuda()
    idx = HIPIndexer(3, 1, 32).build(K, K)
    pick = torch.randperm(n, generator=torch.Generator().manual_seed(1))[:500].cuda()
    samples = K[0][:, pick].contiguous()
    queue = K[0][:, :3].contiguous()
    se = HIPSearcher()
    scale = torch.full((h,), d ** -0.5)
    plan = se.plan_attention(idx, h, scaling=scale)
    q_in = torch.zeros((h, d), dtype=torch.bfloat16, device="cuda")
    out = torch.zeros((h, d), dtype=torch.float32, device="cuda")
    plan.run_sampled(q_in, samples, "sample_mean_topk", 8, out, queue_keys=queue, queue_values=queue)
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            plan.run_sampled(q_in, samples, "sample_mean_topk", 8, out, stream=stream.cuda_stream,
                             queue_keys=queue, queue_values=queue)
    eager_plan = se.plan_attention(idx, h, scaling=scale)
    for rep in range(4):
        q = torch.from_numpy(bf16_round(random_query(h, d, seed=70 + rep))).to(torch.bfloat16).cuda()
        q_in.copy_(q)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        want = torch.empty_like(out)
        tau = eager_plan.run_sampled(q, samples, "sample_mean_topk", 8, want, queue_keys=queue,
                                     queue_values=queue).clone()
        torch.cuda.synchronize()
        assert torch.equal(tau, plan.tau_buf), rep
        assert torch.equal(got, want), rep
        assert float(got.abs().max()) > 0
