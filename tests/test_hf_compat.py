"""The model shells against HF transformers' own Llama / Qwen2 implementations (a library, not the
reference): same config object, same state dict.  The rotary tables are checked on the CPU; the
logits need the GPU (the attention has no CPU path) and use prompts shorter than one group, so that
all keys are still unquantized and the two models compute the same function up to half precision."""
import pytest
import torch

transformers = pytest.importorskip("transformers")

from polarquant_amd.modeling_common import RotaryEmbedding, rope_parameters  # noqa: E402


def _hf_rotary(cfg):
    from transformers.models.llama.modeling_llama import LlamaRotaryEmbedding
    return LlamaRotaryEmbedding(config=cfg)


LLAMA3_SCALING = {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                  "original_max_position_embeddings": 8192}


def _llama_config(scaling=None, theta=500000.0):
    kw = dict(hidden_size=512, num_attention_heads=4, num_key_value_heads=2, num_hidden_layers=2, intermediate_size=768,
              vocab_size=1000, head_dim=128, max_position_embeddings=131072, rms_norm_eps=1e-5, attn_implementation="eager")
    try:        # transformers 5: one rope_parameters dict
        rp = dict(scaling or {"rope_type": "default"})
        rp["rope_theta"] = theta
        cfg = transformers.LlamaConfig(rope_parameters=rp, **kw)
        if getattr(cfg, "rope_parameters", None) is None:
            raise TypeError
    except TypeError:
        cfg = transformers.LlamaConfig(rope_theta=theta, rope_scaling=scaling, **kw)
    return cfg


@pytest.mark.parametrize("scaling", [None, LLAMA3_SCALING, {"rope_type": "linear", "factor": 4.0}])
def test_rotary_tables_match_hf(scaling):
    cfg = _llama_config(scaling)
    theta, sc = rope_parameters(cfg)
    assert theta == 500000.0 and (sc is None) == (scaling is None)
    mine = RotaryEmbedding(128, theta, sc)
    hf = _hf_rotary(cfg)
    assert torch.allclose(mine.inv_freq, hf.inv_freq, rtol=1e-6, atol=0)
    pos = torch.tensor([[0, 1, 17, 4095, 8191, 8192, 100000]])
    x = torch.zeros(1, 1, 1, dtype=torch.float16)
    c0, s0 = mine(x, pos)
    c1, s1 = hf(x, pos)
    assert torch.equal(c0, c1) and torch.equal(s0, s1)


def test_rope_parameters_of_plain_and_legacy_configs():
    from polarquant_amd.modeling_common import PolarConfig

    class Legacy:       # transformers < 5 layout
        rope_theta = 1e6
        rope_scaling = None
    assert rope_parameters(PolarConfig()) == (500000.0, None)
    assert rope_parameters(Legacy()) == (1e6, None)
    with pytest.raises(NotImplementedError):
        RotaryEmbedding(128, 1e4, {"rope_type": "yarn", "factor": 2.0})


def _logits_close(a, b, tol):
    a, b = a.float().cpu(), b.float().cpu()
    scale = b.abs().max().item()
    err = (a - b).abs().max().item()
    assert err <= tol * scale, "max |diff| %.3e against logits up to %.3e" % (err, scale)


@pytest.mark.gpu
@pytest.mark.parametrize("family", ["llama", "llama3-scaled", "qwen2"])
def test_shell_computes_what_hf_computes_before_any_key_is_quantized(gpu, family):
    torch.manual_seed(11)
    if family == "qwen2":
        from polarquant_amd.modeling_qwen_polar import Qwen2PolarForCausalLM as Mine
        kw = dict(hidden_size=896, num_attention_heads=7, num_key_value_heads=1, num_hidden_layers=2, intermediate_size=768,
                  vocab_size=1000, max_position_embeddings=32768, rms_norm_eps=1e-6, attn_implementation="eager",
                  tie_word_embeddings=False)
        try:
            cfg = transformers.Qwen2Config(rope_parameters={"rope_type": "default", "rope_theta": 1e6}, **kw)
        except TypeError:
            cfg = transformers.Qwen2Config(rope_theta=1e6, **kw)
        hf = transformers.Qwen2ForCausalLM(cfg)
    else:
        from polarquant_amd.modeling_llama_polar import LlamaPolarForCausalLM as Mine
        cfg = _llama_config(LLAMA3_SCALING if family == "llama3-scaled" else None)
        hf = transformers.LlamaForCausalLM(cfg)
    hf = hf.eval()
    with torch.no_grad():       # default init leaves biases at 0 and norms at 1: make every parameter matter
        for n, p in hf.named_parameters():
            if p.ndim == 1:
                p.add_(0.1 * torch.randn_like(p))
    mine = Mine(cfg)
    missing = mine.load_state_dict(hf.state_dict(), strict=True)
    assert not missing.missing_keys and not missing.unexpected_keys
    mine = mine.half().to(gpu).eval()
    B, L, steps = 2, 90, 6          # 96 tokens in the end: all keys stay in the unquantized window
    ids = torch.randint(0, 1000, (B, L + steps))
    with torch.no_grad():
        ref = hf(ids).logits                                   # fp32, CPU, one causal pass
        out = mine(ids[:, :L].to(gpu), None, None)
        _logits_close(out.logits, ref[:, :L], 2e-2)
        cache = out.past_key_values
        for s in range(steps):
            out = mine(ids[:, L + s:L + s + 1].to(gpu), None, cache)
            cache = out.past_key_values
            _logits_close(out.logits[:, -1], ref[:, L + s], 2e-2)
        assert cache[0][-1] == L + steps and cache[0][1] is None       # no group was quantized


@pytest.mark.gpu
def test_left_padded_batch_matches_hf_at_the_real_tokens(gpu):
    """Two layers, so that whatever the padded positions produce in layer 0 meets the mask in layer 1."""
    from polarquant_amd.modeling_llama_polar import LlamaPolarForCausalLM
    torch.manual_seed(12)
    cfg = _llama_config()
    hf = transformers.LlamaForCausalLM(cfg).eval()
    mine = LlamaPolarForCausalLM(cfg)
    mine.load_state_dict(hf.state_dict(), strict=True)
    mine = mine.half().to(gpu).eval()
    B, L, steps, pad = 2, 70, 5, 9
    ids = torch.randint(0, 1000, (B, L + steps))
    mask = torch.ones(B, L + steps, dtype=torch.int64)
    mask[1, :pad] = 0
    with torch.no_grad():
        ref = hf(ids, attention_mask=mask).logits
        out = mine(ids[:, :L].to(gpu), mask[:, :L].to(gpu), None)
        assert torch.isfinite(out.logits[0]).all() and torch.isfinite(out.logits[1, pad:]).all()
        _logits_close(out.logits[0], ref[0, :L], 2e-2)
        _logits_close(out.logits[1, pad:], ref[1, pad:L], 2e-2)
        cache = out.past_key_values
        for s in range(steps):
            out = mine(ids[:, L + s:L + s + 1].to(gpu), mask[:, :L + s + 1].to(gpu), cache)
            cache = out.past_key_values
            _logits_close(out.logits[:, -1], ref[:, L + s], 2e-2)
