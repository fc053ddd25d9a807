"""Cache glue with recording stand-ins for indexer and searcher (the approach of the
reference's tests/test_hira_cache.py:29-299): backend selection, prefill, queueing and
flush at update_every, lengths, reset, layer-count derivation."""
import pytest
import torch

import hira_amd.cache.hira_cache as hc
from hira_amd.cache.hira_config import DeviceMode, HiraConfig


class DummyIndexer:
    def __init__(self, **kw):
        self.kw, self.built, self.updates = kw, None, []

    def build(self, k, v):
        self.built = (k, v)
        return self

    def update(self, k, v):
        self.updates.append((k.clone(), v.clone()))
        return self


class DummySearcher:
    def __init__(self, **kw):
        self.kw = kw


@pytest.fixture
def patched(monkeypatch):
    monkeypatch.setattr(hc, "CUDAIndexer", DummyIndexer)
    monkeypatch.setattr(hc, "CUDASearcher", DummySearcher)


def _layer(update_every=4):
    return hc.HiraCacheLayer(DeviceMode.CUDA_ONLY, update_every,
                             {"num_levels": 3, "max_iterations": 1, "branching_factor": 8},
                             {"block_c": 8})


def test_backend_selection(patched):
    l = _layer()
    assert l.indexer_cls is DummyIndexer and l.searcher_cls is DummySearcher
    with pytest.raises(NotImplementedError):
        hc.HiraCacheLayer(DeviceMode.CPU_CUDA, 1, {}, {})
    with pytest.raises(NotImplementedError):
        hc.HiraCacheLayer(DeviceMode.CPU_ONLY, 1, {}, {})


def test_prefill_builds_and_returns_the_same_tensors(patched):
    l = _layer()
    k, v = torch.randn(1, 2, 10, 16), torch.randn(1, 2, 10, 16)
    out, none = l.update(k, v)
    assert none is None and isinstance(out, hc.CacheOutput)
    assert out.prefill_keys is k and out.prefill_values is v
    assert out.indexer.built[0] is k and out.indexer.kw["branching_factor"] == 8
    assert out.searcher.kw == {"block_c": 8}
    assert out.queued_keys.shape == (1, 2, 0, 16)
    assert l.get_seq_length() == 10


def test_decode_queues_then_flushes_every_update_every(patched):
    l = _layer(update_every=3)
    l.update(torch.randn(1, 2, 10, 16), torch.randn(1, 2, 10, 16))
    toks = [(torch.randn(1, 2, 1, 16), torch.randn(1, 2, 1, 16)) for _ in range(4)]
    o = l.update(*toks[0])[0]
    assert o.prefill_keys is None and o.queued_keys.shape[-2] == 1 and l.get_seq_length() == 11
    l.update(*toks[1])
    assert l.queued_len == 2 and not l.indexer.updates
    o = l.update(*toks[2])[0]  # third token reaches update_every: flush
    assert l.queued_len == 0 and o.queued_keys.shape[-2] == 0 and l.indexed_len == 13
    fk, fv = l.indexer.updates[0]
    assert torch.equal(fk, torch.cat([t[0] for t in toks[:3]], dim=-2))
    assert torch.equal(fv, torch.cat([t[1] for t in toks[:3]], dim=-2))
    l.update(*toks[3])
    assert l.get_seq_length() == 14 and l.queued_len == 1


def test_the_queue_is_one_buffer_allocated_once(patched):
    """Queued rows land in a buffer of update_every rows that is allocated with the index (the
    reference concatenates per token, cache/hira_cache.py:121-140); what the layer hands out are
    views of it, and values may be narrower than keys.  A step of more tokens than fit grows it."""
    l = _layer(update_every=5)
    l.update(torch.randn(1, 2, 10, 16), torch.randn(1, 2, 10, 8))
    store = l._queue_k
    assert store.shape == (1, 2, 5, 16) and l._queue_v.shape == (1, 2, 5, 8)
    toks = [(torch.randn(1, 2, 1, 16), torch.randn(1, 2, 1, 8)) for _ in range(4)]
    for i, t in enumerate(toks):
        o = l.update(*t)[0]
        assert l._queue_k is store and o.queue_store[0] is store
        assert o.queued_keys.shape == (1, 2, i + 1, 16) and o.queued_values.shape == (1, 2, i + 1, 8)
        assert o.queued_keys.data_ptr() == store.data_ptr()
    assert torch.equal(o.queued_keys, torch.cat([t[0] for t in toks], dim=-2))
    assert torch.equal(o.queued_values, torch.cat([t[1] for t in toks], dim=-2))
    # six tokens at once: more than the buffer holds; they reach update_every and are flushed
    many = (torch.randn(1, 2, 6, 16), torch.randn(1, 2, 6, 8))
    o = l.update(*many)[0]
    assert l.queued_len == 0 and o.queued_keys.shape[-2] == 0 and l.indexed_len == 20
    fk, fv = l.indexer.updates[0]
    assert torch.equal(fk, torch.cat([t[0] for t in toks] + [many[0]], dim=-2))
    assert torch.equal(fv, torch.cat([t[1] for t in toks] + [many[1]], dim=-2))
    assert l._queue_k.shape[-2] >= 10


def test_mask_sizes_lengths_and_reset(patched):
    l = _layer()
    assert l.get_seq_length() == 0 and l.get_max_cache_shape() == -1 and l.get_max_length() == -1
    l.update(torch.randn(1, 2, 7, 16), torch.randn(1, 2, 7, 16))
    assert l.get_mask_sizes(torch.arange(1)) == (8, 0)   # the reference passes cache_position
    assert l.get_mask_sizes(1) == (8, 0)                 # newer transformers pass query_length
    first = l.indexer
    l.reset()
    assert not l.is_initialized and l.get_seq_length() == 0 and l.indexer is not first


class _Cfg:
    def __init__(self, **kw):
        self.__dict__.update(kw)

    def get_text_config(self, decoder=True):
        return self


def test_cache_layer_count_derivation(patched):
    hcfg = HiraConfig(device_mode=DeviceMode.CUDA_ONLY, update_every=2, num_levels=3,
                      branching_factor=8)
    assert len(hc.HiraCache(_Cfg(num_hidden_layers=4), hcfg).layers) == 4
    assert len(hc.HiraCache(_Cfg(num_hidden_layers=4, sliding_window=128), hcfg).layers) == 4
    assert len(hc.HiraCache(_Cfg(num_hidden_layers=6, num_kv_shared_layers=2), hcfg).layers) == 4
    assert len(hc.HiraCache(_Cfg(num_hidden_layers=9, layer_types=["full_attention"] * 3),
                            hcfg).layers) == 3
    c = hc.HiraCache(_Cfg(num_hidden_layers=2), hcfg)
    out, none = c.update(torch.randn(1, 2, 5, 16), torch.randn(1, 2, 5, 16), layer_idx=1)
    assert none is None and isinstance(out, hc.CacheOutput)
    assert c.layers[1].get_seq_length() == 5 and c.layers[0].get_seq_length() == 0
    assert c.layers[0].update_every == 2


def test_key_sample_follows_the_index(patched):
    """The sample for the threshold rules: taken from the prompt, then kept uniform over the
    indexed keys as queued keys are flushed into the index (never a key that is still queued)."""
    l = hc.HiraCacheLayer(DeviceMode.CUDA_ONLY, 4, {}, {},
                          {"method": "sample_mean_topk", "sample_size": 16, "topk": 3})
    d = 8
    allk = torch.arange(2 * 400, dtype=torch.float32).reshape(1, 2, 400, 1).repeat(1, 1, 1, d)
    out, _ = l.update(allk[:, :, :10], allk[:, :, :10])       # prompt shorter than the sample
    assert out.samples.shape == (2, 10, d) and out.threshold_topk == 3
    for i in range(10, 400):
        out, _ = l.update(allk[:, :, i:i + 1], allk[:, :, i:i + 1])
        ids = out.samples[0, :, 0].long()
        assert out.samples.shape[1] == min(16, l.indexed_len)
        assert int(ids.max()) < l.indexed_len                   # nothing from the queue
        assert len(set(ids.tolist())) == ids.numel()            # no key twice
        assert torch.equal(out.samples[1, :, 0].long() - 400, ids)  # same positions per head
    assert int((ids >= 200).sum()) >= 3 and int((ids < 200).sum()) >= 3  # old and new keys
    assert hc.HiraCacheLayer(DeviceMode.CUDA_ONLY, 4, {}, {}).update(allk, allk)[0].samples is None
