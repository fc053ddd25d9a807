"""End to end through transformers: a small random-weight Llama decodes with HiraCache and the
registered attention function (prefill: dense attention + index build; decode: search + sparse
attention over the index and the queue, the queue folded into the index every few tokens).
With a threshold that selects every key the logits must equal those of the same weights with
transformers' own cache and attention (cache/hira_cache.py:96-153, attention/hira_attention.py
of the reference describe this wiring; its examples need downloaded weights)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _models(dtype, head_dim):
    from transformers import LlamaConfig, LlamaForCausalLM

    from hira_amd.attention import register_hira_attention

    torch.manual_seed(0)
    kw = dict(vocab_size=512, hidden_size=256, intermediate_size=512, num_hidden_layers=2,
              num_attention_heads=8, num_key_value_heads=2, head_dim=head_dim,
              max_position_embeddings=4096)
    cfg = LlamaConfig(**kw)
    ref = LlamaForCausalLM(cfg).to("cuda").to(dtype).eval()
    model = LlamaForCausalLM(LlamaConfig(**kw, attn_implementation=register_hira_attention("hira")))
    model.load_state_dict(ref.state_dict())
    model = model.to("cuda").to(dtype).eval()
    assert model.config._attn_implementation == "hira"
    return cfg, ref, model


def _set(model, **attrs):
    for m in model.modules():
        if hasattr(m, "layer_idx"):
            for k, v in attrs.items():
                setattr(m, k, v)


@pytest.mark.parametrize("dtype,head_dim,bf,tol,batch", [(torch.float32, 32, 8, 1e-4, 1),
                                                        (torch.float32, 32, 8, 1e-4, 3),  # the reference: B = 1 only
                                                        (torch.bfloat16, 64, 16, 6e-2, 2)])
def test_llama_decode_matches_dense_when_every_key_is_selected(dtype, head_dim, bf, tol, batch, gpu_device):
    from hira_amd.cache.hira_cache import HiraCache
    from hira_amd.cache.hira_config import DeviceMode, HiraConfig

    cfg, ref, model = _models(dtype, head_dim)
    _set(model, hira_threshold=-3.0e38)
    hc = HiraConfig(device_mode=DeviceMode.CUDA_ONLY, update_every=4, num_levels=3,
                    branching_factor=bf, threshold_method="none")
    cache = HiraCache(cfg, hc)
    ids = torch.randint(0, 512, (batch, 300), device="cuda", generator=torch.Generator("cuda").manual_seed(1))
    with torch.no_grad():
        o_ref = ref(ids, use_cache=True)
        o = model(ids, past_key_values=cache, use_cache=True)
        scale = float(o_ref.logits.float().abs().max())
        assert float((o.logits.float() - o_ref.logits.float()).abs().max()) <= tol * scale
        pk = o_ref.past_key_values
        tok = o_ref.logits[:, -1:].argmax(-1)
        for step in range(10):
            print(f"decode step {step}", flush=True)
            o_ref = ref(tok, past_key_values=pk, use_cache=True)
            o = model(tok, past_key_values=cache, use_cache=True)
            assert cache.get_seq_length() == 301 + step
            err = float((o.logits.float() - o_ref.logits.float()).abs().max())
            assert err <= tol * scale, (step, err, scale)
            tok = o_ref.logits[:, -1:].argmax(-1)
    layer = cache.layers[0]
    assert layer.indexed_len == 308 and layer.queued_len == 2   # two flushes of four, two queued


def test_llama_generate_greedy_tokens_match(gpu_device):
    from hira_amd.cache.hira_cache import HiraCache
    from hira_amd.cache.hira_config import DeviceMode, HiraConfig

    cfg, ref, model = _models(torch.float32, 32)
    _set(model, hira_threshold=-3.0e38)
    hc = HiraConfig(device_mode=DeviceMode.CUDA_ONLY, update_every=3, num_levels=2,
                    branching_factor=16, threshold_method="none")
    ids = torch.randint(0, 512, (1, 200), device="cuda", generator=torch.Generator("cuda").manual_seed(2))
    with torch.no_grad():
        want = ref.generate(ids, max_new_tokens=12, do_sample=False)
        got = model.generate(ids, max_new_tokens=12, do_sample=False,
                             past_key_values=HiraCache(cfg, hc))
    assert torch.equal(want, got)


def test_llama_decode_with_sample_thresholds_is_sparse_and_finite(gpu_device):
    """The configured rule (mean of the 5 best of a 128-key sample) drives the decode: the
    logits are finite and differ from dense attention's (keys were left out)."""
    from hira_amd.cache.hira_cache import HiraCache
    from hira_amd.cache.hira_config import DeviceMode, HiraConfig

    cfg, ref, model = _models(torch.bfloat16, 64)
    hc = HiraConfig(device_mode=DeviceMode.CUDA_ONLY, update_every=4, num_levels=3,
                    branching_factor=16, threshold_method="sample_mean_topk", sample_size=128,
                    threshold_topk=5)
    cache = HiraCache(cfg, hc)
    ids = torch.randint(0, 512, (1, 600), device="cuda", generator=torch.Generator("cuda").manual_seed(3))
    with torch.no_grad():
        o_ref = ref(ids, use_cache=True)
        o = model(ids, past_key_values=cache, use_cache=True)
        assert cache.layers[0].samples.shape == (2, 128, 64)
        pk = o_ref.past_key_values
        tok = o_ref.logits[:, -1:].argmax(-1)
        diff = 0.0
        for step in range(6):
            o_ref = ref(tok, past_key_values=pk, use_cache=True)
            o = model(tok, past_key_values=cache, use_cache=True)
            assert torch.isfinite(o.logits).all()
            diff = max(diff, float((o.logits.float() - o_ref.logits.float()).abs().max()))
            tok = o_ref.logits[:, -1:].argmax(-1)
    assert diff > 0.0
