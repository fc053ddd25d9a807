"""Host-side logic that needs no GPU: layout sizes, head maps, input coercion, config,
threshold rules, synthetic workloads."""
import numpy as np
import pytest
import torch

from hira_amd import synth
from hira_amd.cache import hira_config, threshold_finder
from hira_amd.indexer.hip import HIPIndexer, level_sizes
from hira_amd.searcher.hip import HIPSearcher
from oracle import hira_oracle as ho


def test_level_sizes_match_the_benchmark_shapes():
    assert level_sizes(4096, 16, 2) == [4096, 256]
    assert level_sizes(8192, 32, 3) == [8192, 256, 8]
    assert level_sizes(32768, 32, 3) == [32768, 1024, 32]
    assert level_sizes(131072, 32, 4) == [131072, 4096, 128, 4]
    assert level_sizes(203, 4, 4) == [256, 64, 16, 4]
    assert level_sizes(20, 32, 3) == [1024, 32, 1]
    assert level_sizes(100, 1, 2) == [100, 100]
    for n, bf, nl in [(203, 4, 4), (769, 8, 3), (5, 64, 2), (4096, 16, 2)]:
        assert level_sizes(n, bf, nl) == ho.fixed_fanout_sizes(n, bf, nl)


class _FakeIndexer:
    def __init__(self, batch, heads):
        self.batch, self.num_heads, self.num_trees = batch, heads, batch * heads
        self.device = torch.device("cpu")


def test_default_head_map_is_gqa_grouping():
    off, heads, gmax, group = HIPSearcher()._head_map(32, _FakeIndexer(1, 8), None)
    assert gmax == 4 and group == 4 and off.tolist() == list(range(0, 33, 4))
    assert heads.tolist() == list(range(32))
    # two sequences of 4 query / 2 KV heads: tree = b*H_kv + h // 2
    off, heads, gmax, group = HIPSearcher()._head_map(8, _FakeIndexer(2, 2), None)
    assert off.tolist() == [0, 2, 4, 6, 8] and heads.tolist() == list(range(8)) and group == 2


def test_explicit_head_map_and_its_errors():
    se = HIPSearcher()
    off, heads, gmax, group = se._head_map(4, _FakeIndexer(1, 2), torch.tensor([1, 0, 1, 0]))
    assert off.tolist() == [0, 2, 4] and heads.tolist() == [1, 3, 0, 2] and gmax == 2 and group == 0
    with pytest.raises(ValueError):
        se._head_map(4, _FakeIndexer(1, 2), torch.tensor([0, 1, 2, 0]))  # out of range
    with pytest.raises(ValueError):
        se._head_map(4, _FakeIndexer(1, 2), torch.tensor([0, 1]))        # wrong length
    with pytest.raises(TypeError):
        se._head_map(4, _FakeIndexer(1, 2), [0, 1, 0, 1])
    with pytest.raises(ValueError):
        se._head_map(3, _FakeIndexer(1, 2), None)                        # 3 heads over 2 trees


def test_input_coercion_errors_follow_the_reference_wrappers():
    """kernels/triton_search_wrappers.py:9-110 of the reference."""
    se = HIPSearcher
    assert se._coerce_query(torch.zeros(1, 4, 1, 16), 16).shape == (4, 16)
    assert se._coerce_query(torch.zeros(3, 4, 1, 16), 16).shape == (12, 16)
    with pytest.raises(TypeError):
        se._coerce_query([[0.0]], 1)
    with pytest.raises(ValueError):
        se._coerce_query(torch.zeros(1, 4, 2, 16), 16)
    with pytest.raises(ValueError):
        se._coerce_query(torch.zeros(4, 8), 16)
    with pytest.raises(ValueError):
        se._coerce_query(torch.zeros(16), 16)
    assert se._coerce_threshold(0.5, 3, "cpu").tolist() == [0.5] * 3
    assert se._coerce_threshold(torch.tensor(2.0), 2, "cpu").tolist() == [2.0, 2.0]
    with pytest.raises(ValueError):
        se._coerce_threshold(torch.zeros(2), 3, "cpu")
    assert se._coerce_scaling(None, 2, "cpu").tolist() == [1.0, 1.0]
    with pytest.raises(ValueError):
        se._coerce_scaling(torch.ones(5), 2, "cpu")
    with pytest.raises(TypeError):
        se._coerce_scaling(1.0, 2, "cpu")
    with pytest.raises(ValueError):
        HIPSearcher(index_space="token")


def test_indexer_constructor_contract():
    idx = HIPIndexer(num_levels=3, max_iterations=2, branching_factor=8)
    assert idx.depth == HIPIndexer.DEPTH.THREE_LEVELS and idx.children is None
    assert HIPIndexer(HIPIndexer.DEPTH.TWO_LEVELS, 1, 4).num_levels == 2
    assert HIPIndexer(5, 1, 4).depth == 5  # deeper than the reference's enum goes
    with pytest.raises(ValueError):
        idx.tree_struct()  # not built


def test_config_kwargs_and_loaders(tmp_path):
    """cache/hira_config.py:35-46 of the reference + the loaders it leaves unwritten."""
    cfg = hira_config.HiraConfig(device_mode=hira_config.DeviceMode.CUDA_ONLY, num_levels=3,
                                 max_iterations=2, branching_factor=32)
    assert cfg.get_indexer_kwargs() == {"num_levels": 3, "max_iterations": 2,
                                        "branching_factor": 32}
    assert cfg.get_searcher_kwargs() == {"block_c": 32}
    cpu = hira_config.HiraConfig(device_mode=hira_config.DeviceMode.CPU_ONLY)
    assert cpu.get_searcher_kwargs() == {"chunk_size": 8192}
    HIPIndexer(**cfg.get_indexer_kwargs())
    HIPSearcher(**cfg.get_searcher_kwargs())
    d = hira_config.HiraConfig.from_dict({"num_levels": 4, "update_every": 64})
    assert d.num_levels == 4 and d.update_every == 64 and d.branching_factor == 10
    with pytest.raises(ValueError):
        hira_config.HiraConfig.from_dict({"no_such_setting": 1})
    p = tmp_path / "c.yml"
    p.write_text("device_mode: cuda_only\nnum_levels: 3\nbranching_factor: 16\n")
    y = hira_config.HiraConfig.from_yaml(str(p))
    assert (y.device_mode, y.num_levels, y.branching_factor) == ("cuda_only", 3, 16)


def test_config_file_in_the_layout_of_the_reference_sample(tmp_path):
    """The one configuration file the reference ships (examples/configs/1_example_config.yml:1-8)
    groups the index's settings under ``indexing:`` and carries a ``cuda_memory_limit`` nothing
    reads; a file of that structure must load."""
    p = tmp_path / "sample.yml"
    p.write_text('device_mode: "cuda_only" # "cpu_only" or "cuda_only" or "cpu-cuda"\n\n'
                 'cuda_memory_limit: 4096  # MB\n\n'
                 'indexing:\n  num_levels: 3\n  max_iterations: 2 # k-means\n'
                 '  branching_factor: 32\n')
    with pytest.warns(UserWarning, match="cuda_memory_limit"):
        cfg = hira_config.HiraConfig.from_yaml(str(p))
    assert cfg.device_mode == "cuda_only"
    assert cfg.get_indexer_kwargs() == {"num_levels": 3, "max_iterations": 2,
                                        "branching_factor": 32}
    assert cfg.update_every == 1 and cfg.sample_size == 1000      # untouched defaults
    both = hira_config.HiraConfig.from_dict(
        {"update_every": 64, "indexing": {"num_levels": 4},
         "thresholds": {"threshold_method": "sample_max", "sample_size": 256}})
    assert (both.update_every, both.num_levels, both.threshold_method, both.sample_size) == \
        (64, 4, "sample_max", 256)
    for bad in ({"indexing": {"update_every": 2}},            # a setting in the wrong section
                {"indexing": {"num_level": 3}},               # a misspelt one
                {"indexing": 3},                              # a section that is no mapping
                {"num_levels": 3, "indexing": {"num_levels": 4}}):   # given twice
        with pytest.raises(ValueError):
            hira_config.HiraConfig.from_dict(bad)


def test_reference_import_paths_resolve_to_this_package():
    """The reference installs as ``hira`` (setup.py:14-15) and its modules import each other as
    ``hira.indexer``, ``hira.searcher``, ``hira.cache.*`` (cache/hira_cache.py:7-10,
    tests/test_hira_cache.py:17-19): the same paths give this package's modules, the very
    objects, so a patch through one name is seen through the other."""
    import importlib

    import hira
    import hira.indexer
    import hira.searcher
    import hira.cache.hira_cache as by_old_name
    import hira_amd.cache.hira_cache as by_new_name
    import hira_amd.indexer
    from hira.attention.hira_attention import hira_attention_forward
    from hira.cache.hira_cache import CacheOutput, HiraCache, HiraCacheLayer  # noqa: F401
    from hira.cache.hira_config import DeviceMode, HiraConfig
    from hira.cache.threshold_finder import THRESHOLD_METHODS
    from hira.indexer import BaseIndexer, CUDAIndexer
    from hira.indexer.cuda import CUDAIndexer as from_cuda_module
    from hira.searcher import BaseSearcher, CUDASearcher
    from hira.searcher.cuda import CUDASearcher as searcher_from_cuda_module

    assert hira.indexer is hira_amd.indexer and by_old_name is by_new_name
    assert CUDAIndexer is from_cuda_module is HIPIndexer and issubclass(CUDAIndexer, BaseIndexer)
    assert CUDASearcher is searcher_from_cuda_module is HIPSearcher
    assert issubclass(CUDASearcher, BaseSearcher)
    assert HiraConfig is hira_config.HiraConfig and DeviceMode.CUDA_ONLY == "cuda_only"
    assert THRESHOLD_METHODS is threshold_finder.THRESHOLD_METHODS
    assert callable(hira_attention_forward)
    assert by_new_name.__spec__.name == "hira_amd.cache.hira_cache"   # its own spec is kept
    with pytest.raises(ModuleNotFoundError):
        importlib.import_module("hira.no_such_module")


def test_threshold_rules():
    g = torch.Generator().manual_seed(0)
    keys = torch.randn((2, 500, 16), generator=g)
    q = torch.randn((4, 16), generator=g)
    s = torch.einsum("hnd,hd->hn", keys.repeat_interleave(2, 0), q)
    t = threshold_finder.exact_topk(keys, q, 25)
    assert ((s >= t[:, None]).sum(1) == 25).all()
    t2 = threshold_finder.exact_topk(keys, q.view(1, 4, 1, 16), 25, midpoint=False)
    assert torch.equal(t2, s.topk(25, dim=1).values[:, -1])
    assert torch.allclose(threshold_finder.sample_max(keys, q), s.max(1).values)
    assert torch.allclose(threshold_finder.sample_mean_topk(keys, q, 10),
                          s.topk(10, dim=1).values.mean(1))
    m = torch.tensor([1, 0, 1, 0])
    s2 = torch.einsum("hnd,hd->hn", keys[m], q)
    assert torch.allclose(threshold_finder.sample_max(keys, q, m), s2.max(1).values)
    assert set(threshold_finder.THRESHOLD_METHODS) >= {"sample_max", "sample_mean_topk"}
    # the float64 restatement the GPU tests check hira_threshold against: same rules via
    # numpy's sort, against torch's topk here; k = 1 is the maximum, k = all the mean score
    from oracle import hira_oracle as ho
    kn, qn = keys.numpy(), q.numpy()
    assert np.allclose(ho.sample_thresholds(kn, qn, "sample_max"), s.max(1).values.numpy(), rtol=1e-6)
    assert np.allclose(ho.sample_thresholds(kn, qn, "sample_mean_topk", 10),
                       s.topk(10, dim=1).values.mean(1).numpy(), rtol=1e-5, atol=1e-6)
    assert np.array_equal(ho.sample_thresholds(kn, qn, "sample_mean_topk", 1),
                          ho.sample_thresholds(kn, qn, "sample_max"))
    assert np.allclose(ho.sample_thresholds(kn, qn, "sample_mean_topk", 500), s.mean(1).numpy(),
                       rtol=1e-4, atol=1e-5)
    assert np.allclose(ho.sample_thresholds(kn, qn, "sample_max", q2kv=m.numpy()),
                       s2.max(1).values.numpy(), rtol=1e-6)


def test_synthetic_workloads_are_seeded_and_shaped():
    w = synth.WORKLOADS[0]
    k1, v1 = synth.make_kv(w)
    k2, _ = synth.make_kv(w)
    assert k1.shape == (1, 1, 4096, 128) and k1.dtype == torch.float32 and torch.equal(k1, k2)
    q = synth.make_queries(w, k1, 3)
    assert q.shape == (3, 1, 1, 128)
    w2 = synth.WORKLOADS[2]
    d = synth.head_dist(w2, 0, 3)
    assert d.massive.numel() == 8
    k, _ = synth.make_kv(w2, n=256)
    assert k.dtype == torch.bfloat16 and k.shape == (1, 8, 256, 128)
    big = k[0, 3].float().abs().mean(0)
    others = torch.ones(128, dtype=torch.bool)
    others[d.massive] = False
    assert big[d.massive].min() > 3 * big[others].mean()  # the 8 boosted channels stand out
    fr = synth.select_fractions(synth.WORKLOADS[3])
    assert fr.shape == (16,) and 0.005 <= float(fr.min()) and float(fr.max()) <= 0.05


def test_capture_file_in_the_reference_samplers_format(tmp_path):
    """benchmark_area/kv_sampling/collect_kv_data.py:393-397 writes keys (N, D) and queries
    (N, D); the loader deals them to the workload's trees, seeded."""
    w = synth.WORKLOADS[1]
    rng = np.random.default_rng(0)
    path = tmp_path / "capture.npz"
    np.savez_compressed(path, keys=rng.normal(size=(8 * 300 + 5, w.d)).astype(np.float32),
                        queries=rng.normal(size=(100, w.d)).astype(np.float32))
    w2, k, v, q = synth.load_capture(str(path), w, 7)
    assert w2.n == 300 and w2.name.endswith("+capture")
    assert k.shape == (1, 8, 300, w.d) and v.shape == k.shape and q.shape == (7, 1, 32, w.d)
    assert k.dtype == w.dtype
    _, k2, _, q2 = synth.load_capture(str(path), w, 7)
    assert torch.equal(k, k2) and torch.equal(q, q2)
    # every key of the index comes from the file, none twice
    pool = torch.from_numpy(np.load(path)["keys"]).to(w.dtype)
    rows = {tuple(r.tolist()) for r in k.reshape(-1, w.d)[:, :4].float()}
    assert rows <= {tuple(r.tolist()) for r in pool[:, :4].float()} and len(rows) == 8 * 300
    np.savez_compressed(tmp_path / "bad.npz", keys=np.zeros((10, 3), np.float32),
                        queries=np.zeros((10, 3), np.float32))
    with pytest.raises(ValueError):
        synth.load_capture(str(tmp_path / "bad.npz"), w, 1)


def test_bench_refuses_more_than_one_gpu():
    """The path is built and measured on one GPU: bench.py --gpus N > 1 says so and exits."""
    import subprocess
    import sys
    from pathlib import Path

    root = Path(__file__).resolve().parents[1]
    r = subprocess.run([sys.executable, str(root / "bench.py"), "--gpus", "2"], capture_output=True,
                       text=True, timeout=120)
    assert r.returncode == 2 and "ONE GPU" in (r.stdout + r.stderr)


def test_config_rejects_bad_settings():
    for bad in (dict(device_mode="gpu"), dict(update_every=0), dict(num_levels=0),
                dict(branching_factor=0), dict(max_iterations=-1), dict(threshold_method="median"),
                dict(sample_size=0), dict(threshold_topk=0)):
        with pytest.raises(ValueError):
            hira_config.HiraConfig(**bad)
    cfg = hira_config.HiraConfig(max_iterations=0, threshold_method="none")
    assert cfg.get_indexer_kwargs() == {"num_levels": 5, "max_iterations": 0, "branching_factor": 10}
    assert cfg.get_threshold_kwargs() == {"method": "none", "sample_size": 1000, "topk": 10}


def test_attention_refuses_masks_that_hide_keys():
    """A padded batch cannot be honoured by the sparse decode step (the index holds every cached
    position): the attention function raises instead of attending to pad keys."""
    from types import SimpleNamespace

    from hira_amd.attention.hira_attention import _hides_a_key, hira_attention_forward

    b, h, l, d = 2, 2, 5, 16
    q = torch.randn(b, h, l, d)
    cache = SimpleNamespace(indexer=object(), prefill_keys=torch.randn(b, h, l, d),
                            prefill_values=torch.randn(b, h, l, d))
    causal = torch.tril(torch.ones(l, l, dtype=torch.bool))[None, None].expand(b, 1, l, l)
    out, _ = hira_attention_forward(None, q, cache, None, attention_mask=causal)
    assert out.shape == (b, l, h, d)
    padded = causal.clone()
    padded[1, :, :, 0] = False                      # sequence 1 is left-padded by one position
    with pytest.raises(ValueError, match="padded"):
        hira_attention_forward(None, q, cache, None, attention_mask=padded)
    additive = torch.zeros(b, 1, l, l).masked_fill(~padded, float("-inf"))
    with pytest.raises(ValueError, match="padded"):
        hira_attention_forward(None, q, cache, None, attention_mask=additive)
    assert not _hides_a_key(None)
    assert not _hides_a_key(torch.ones(b, l, dtype=torch.long))
    assert _hides_a_key(torch.tensor([[0, 1, 1], [1, 1, 1]]))
    # decode: looked at on the first step of an index
    idx = SimpleNamespace()
    dec = SimpleNamespace(indexer=idx, searcher=None, prefill_keys=None)
    with pytest.raises(ValueError, match="padded"):
        hira_attention_forward(None, q[:, :, :1], dec, None, attention_mask=padded[:, :, -1:, :])


def test_unsynced_stretch_guards_the_pointers():
    """While a stretch of updates without read-back is open (a captured decode step holds the
    pointers) the index refuses to re-allocate, and the capacity bound counts from the exact
    sizes, not from the bound that stands in for them."""
    idx = HIPIndexer(3, 1, 4, device="cpu")
    idx.num_trees, idx.num_keys = 1, 64
    idx.size, idx.cap = [64, 16, 4], [64, 16, 4]
    idx._exact_size, idx._pending = [64, 16, 4], 0
    idx.size = [96, 24, 8]                      # bounds, as begin_unsynced leaves them
    assert idx._needed_caps(4)[2] == 4 + 2      # from the exact size 4, not from the bound 8
    idx._unsynced_room = 8
    idx.tiled = False
    with pytest.raises(RuntimeError, match="re-allocate"):
        idx._grow([128, 32, 8])
    idx._grow([64, 16, 4])                      # nothing to do: fine


def test_storage_dtype_policy():
    assert HIPIndexer.storage_dtype(torch.bfloat16) == torch.bfloat16
    assert HIPIndexer.storage_dtype(torch.float32) == torch.float32
    with pytest.warns(UserWarning, match="bfloat16"):
        assert HIPIndexer.storage_dtype(torch.float16) == torch.bfloat16
    assert HIPIndexer.storage_dtype(torch.float64) == torch.float32


def test_layout_rule_adds_the_shadow_only_for_long_trees_with_many_heads():
    """layout="auto": tiled where the MFMA kernel can scan, with the 8-bit shadow only from
    131072 keys a tree and 8 query heads per KV head on (where it measurably wins); explicit
    requests are honoured or refused."""
    import torch
    from hira_amd.indexer.hip import Q8_AUTO_MIN_HEADS, Q8_AUTO_MIN_KEYS, choose_layout

    bf16, f32 = torch.bfloat16, torch.float32
    assert (Q8_AUTO_MIN_KEYS, Q8_AUTO_MIN_HEADS) == (131072, 8)
    # (request, dtype, dim, vdim, levels, bf, n, heads per tree) -> (tiled, q8)
    assert choose_layout("auto", bf16, 128, 128, 4, 32, 131072, 8) == (True, True)
    assert choose_layout("auto", bf16, 128, 128, 4, 32, 131071, 8) == (True, False)
    assert choose_layout("auto", bf16, 128, 128, 4, 32, 1 << 20, 7) == (True, False)
    assert choose_layout("auto", bf16, 128, 128, 4, 32, 1 << 20, None) == (True, False)
    assert choose_layout("auto", bf16, 64, 64, 3, 16, 1 << 18, 16) == (True, True)
    assert choose_layout("auto", bf16, 256, 256, 3, 32, 1 << 18, 16) == (True, False)  # no shadow kernels
    assert choose_layout("auto", bf16, 128, 0, 3, 32, 1 << 18, 16) == (True, False)    # no values: scores only
    assert choose_layout("auto", bf16, 128, 128, 1, 32, 1 << 18, 16) == (False, False)
    assert choose_layout("auto", bf16, 128, 128, 3, 8, 1 << 18, 16) == (False, False)  # fan-out not in tiles
    assert choose_layout("auto", f32, 128, 128, 3, 32, 1 << 18, 16) == (False, False)
    assert choose_layout("q8", bf16, 128, 128, 2, 32, 100, None) == (True, True)
    assert choose_layout("tiled", bf16, 96, 96, 2, 8, 100, 16) == (True, False)
    assert choose_layout("row_major", bf16, 128, 128, 4, 32, 1 << 20, 16) == (False, False)
    import pytest
    with pytest.raises(ValueError):
        choose_layout("q8", bf16, 256, 256, 3, 32, 1000, 8)
    with pytest.raises(ValueError):
        choose_layout("q8", f32, 128, 128, 3, 32, 1000, 8)
    with pytest.raises(ValueError):
        choose_layout("tiled", f32, 128, 128, 3, 32, 1000, 8)
