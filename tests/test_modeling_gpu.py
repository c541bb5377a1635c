"""The drop-in attention classes and model shell on the GPU, checked against the CPU
oracle's restatement of the reference forward (prefill split, decode step, flush)."""
import math

import pytest
import torch

from oracle import polar_oracle as po
from polarquant_amd.modeling_common import PolarConfig
from polarquant_amd.modeling_llama_polar import (GenerationConfig, LlamaPolarForCausalLM, LlamaPolarGroupAttention,
                                                 PolarCache, generate)
from polarquant_amd.modeling_qwen_polar import Qwen2PolarForCausalLM, Qwen2PolarGroupAttention

pytestmark = pytest.mark.gpu


def _tiny(n_heads=4, n_kv=2, layers=2, **kw):
    return PolarConfig(hidden_size=n_heads * 128, num_attention_heads=n_heads, num_key_value_heads=n_kv,
                       num_hidden_layers=layers, intermediate_size=512, vocab_size=1000, rope_theta=1e4,
                       eos_token_id=[999999], **kw)


def _rope(cfg, start, n, dtype, dev):
    inv = 1.0 / (cfg.rope_theta ** (torch.arange(0, 128, 2, dtype=torch.float32) / 128))
    ang = torch.arange(start, start + n, dtype=torch.float32)[:, None] * inv[None]
    emb = torch.cat([ang, ang], -1)[None]
    return emb.cos().to(dtype).to(dev), emb.sin().to(dtype).to(dev)


@pytest.mark.parametrize("cls,n_heads,n_kv,rb,tb", [(LlamaPolarGroupAttention, 4, 2, 4, 4), (Qwen2PolarGroupAttention, 7, 1, 3, 3)])
@pytest.mark.parametrize("L", [1, 5, 200, 256])      # 1: a one-token prompt is a prefill here (the reference fails on it)
def test_attention_forward_matches_reference_restatement(gpu, cls, n_heads, n_kv, rb, tb, L):
    """Prefill then decode across a residual flush.  The post-RoPE q/k/v of every call are captured
    on the GPU and replayed through the oracle's forward: cache contents must be bit-identical
    (codes, metadata, residual keys, values, kv_seq_len) and outputs within the fp16 tolerance."""
    torch.manual_seed(0)
    cfg = _tiny(n_heads, n_kv, rbits=rb, tbits=tb)
    att = cls(cfg, 0).half().to(gpu)
    assert (att.q_proj.bias is not None) == (cls is Qwen2PolarGroupAttention)
    att.capture = []
    B, steps = 2, 140
    mask = torch.ones(B, L, dtype=torch.int64)
    mask[1, :min(3, L - 1)] = 0                              # left padding on sequence 1
    x = (torch.randn(B, L + steps, cfg.hidden_size) * 0.5).half().to(gpu)
    with torch.no_grad():
        out, cache = att(x[:, :L], attention_mask=mask.to(gpu), past_key_value=None, position_embeddings=_rope(cfg, 0, L, torch.float16, gpu))
    assert isinstance(cache, tuple) and len(cache) == 8 and cache[-1] == L
    q, k, v = [t.cpu() for t in att.capture[-1]]
    ref_cache = po.prefill_cache(k, v, rb, tb)
    _check_cache(cache, ref_cache)
    o_proj = att.o_proj.weight.detach().float().cpu()
    for i in range(steps):
        mask = torch.cat([mask, torch.ones(B, 1, dtype=torch.int64)], -1)
        with torch.no_grad():
            out, cache = att(x[:, L + i:L + i + 1], attention_mask=mask.to(gpu), past_key_value=cache,
                             position_embeddings=_rope(cfg, L + i, 1, torch.float16, gpu))
        q, k, v = [t.cpu() for t in att.capture[-1]]
        ref_attn, ref_cache = po.decode_step(q, k, v, ref_cache, mask, rb, tb)
        ref_out = ref_attn.reshape(B, 1, -1).float() @ o_proj.T
        assert out.shape == (B, 1, cfg.hidden_size)
        err = (out.float().cpu() - ref_out).abs().max().item()
        assert err < 2e-2 * max(1.0, ref_out.abs().max().item()), (i, err)
        if i in (0, 1, steps // 2, steps - 1) or (L + i + 1) % 128 in (0, 1):
            _check_cache(cache, ref_cache)


def _check_cache(got, ref):
    assert got[-1] == ref[-1]
    for j, (g, r) in enumerate(zip(got[:-1], ref[:-1])):
        assert (g is None) == (r is None), "tuple element %d" % j
        if g is not None:
            g = g.cpu()
            assert g.shape == r.shape and g.dtype == r.dtype, "tuple element %d" % j
            if g.dtype in (torch.uint8, torch.int32):
                assert torch.equal(g, r), "codes differ (tuple element %d)" % j
            else:
                assert bool((g.float() == r.float()).all()), "tuple element %d differs" % j


def test_plain_reference_tuple_is_accepted(gpu):
    """A cache tuple built elsewhere in the reference's format (plain tuple, no arena) can be passed in."""
    torch.manual_seed(1)
    cfg = _tiny()
    att = LlamaPolarGroupAttention(cfg, 0).half().to(gpu)
    att.capture = []
    x = torch.randn(1, 301, cfg.hidden_size).half().to(gpu)
    with torch.no_grad():
        _, cache = att(x[:, :300], None, None, _rope(cfg, 0, 300, torch.float16, gpu))
        plain = tuple(t.clone() if torch.is_tensor(t) else t for t in cache)
        assert not isinstance(plain, PolarCache)
        o1, c1 = att(x[:, 300:], None, cache, _rope(cfg, 300, 1, torch.float16, gpu))
        o2, c2 = att(x[:, 300:], None, plain, _rope(cfg, 300, 1, torch.float16, gpu))
    assert torch.equal(o1, o2) and c1[-1] == c2[-1] == 301


@pytest.mark.parametrize("cls,cfg", [(LlamaPolarForCausalLM, _tiny()), (Qwen2PolarForCausalLM, _tiny(7, 1, rbits=3, tbits=3, attention_bias=True))])
def test_generate_greedy_matches_cpu_replay(gpu, cls, cfg):
    """Greedy generation across a flush; every decode step's logits are replayed on the CPU with
    the oracle attention (fp32 weights) and must agree."""
    torch.manual_seed(2)
    model = cls(cfg).half().to(gpu).eval()
    B, L, new = 2, 250, 12
    ids = torch.randint(0, cfg.vocab_size, (B, L))
    gen = GenerationConfig(eos_token_id=[999999])
    out = generate(model, ids.to(gpu), torch.ones(B, L, dtype=torch.int64, device=gpu), gen, max_new_tokens=new)
    assert out.shape == (B, new) and out.dtype == torch.long
    assert model.kv_cache_bytes_per_token() == cfg.num_hidden_layers * cfg.num_key_value_heads * (64 + 4 + 256)
    # replay: same model, step by step, capturing q/k/v per layer and checking the layer outputs
    for layer in model.model.layers:
        layer.self_attn.capture = []
    with torch.no_grad():
        o = model(ids.to(gpu), None, None, num_logits_to_keep=1)
        caches = o.past_key_values
        assert caches[0][-1] == L and len(caches) == cfg.num_hidden_layers
        ref_caches = []
        for layer in model.model.layers:
            q, k, v = [t.cpu() for t in layer.self_attn.capture[-1]]
            ref_caches.append(po.prefill_cache(k, v, cfg.rbits, cfg.tbits))
        tok = o.logits.argmax(-1)
        assert torch.equal(tok.cpu(), out[:, :1].cpu())
        for s in range(1, new):
            o = model(tok, None, caches, num_logits_to_keep=1)
            caches = o.past_key_values
            for li, layer in enumerate(model.model.layers):
                q, k, v = [t.cpu() for t in layer.self_attn.capture[-1]]
                _, ref_caches[li] = po.decode_step(q, k, v, ref_caches[li], None, cfg.rbits, cfg.tbits)
                _check_cache(caches[li], ref_caches[li])
            tok = o.logits.argmax(-1)
            assert torch.equal(tok.cpu(), out[:, s:s + 1].cpu())
        assert caches[0][-1] == L + new - 1


def test_cache_arena_grows_past_its_initial_capacity(gpu):
    """cache_capacity is only a hint: decoding past it reallocates (doubling) and keeps every cached token."""
    torch.manual_seed(3)
    cfg = _tiny(cache_capacity=128)
    att = LlamaPolarGroupAttention(cfg, 0).half().to(gpu)
    att.capture = []
    L, steps = 100, 400                      # ends at 500 tokens: 3 groups + 116 residual, capacity grown twice
    x = (torch.randn(1, L + steps, cfg.hidden_size) * 0.5).half().to(gpu)
    with torch.no_grad():
        _, cache = att(x[:, :L], None, None, _rope(cfg, 0, L, torch.float16, gpu))
        q, k, v = [t.cpu() for t in att.capture[-1]]
        ref_cache = po.prefill_cache(k, v)
        cap0 = cache.arena.vcap
        for i in range(steps):
            out, cache = att(x[:, L + i:L + i + 1], None, cache, _rope(cfg, L + i, 1, torch.float16, gpu))
            q, k, v = [t.cpu() for t in att.capture[-1]]
            _, ref_cache = po.decode_step(q, k, v, ref_cache)
    assert cache.arena.vcap > cap0 and cache[-1] == L + steps
    _check_cache(cache, ref_cache)


def test_decode_with_bf16_model(gpu):
    torch.manual_seed(4)
    cfg = _tiny()
    att = LlamaPolarGroupAttention(cfg, 0).bfloat16().to(gpu)
    att.capture = []
    L = 130
    x = (torch.randn(2, L + 3, cfg.hidden_size) * 0.5).bfloat16().to(gpu)
    with torch.no_grad():
        _, cache = att(x[:, :L], None, None, _rope(cfg, 0, L, torch.bfloat16, gpu))
        q, k, v = [t.cpu() for t in att.capture[-1]]
        ref_cache = po.prefill_cache(k, v)
        _check_cache(cache, ref_cache)
        for i in range(3):
            out, cache = att(x[:, L + i:L + i + 1], None, cache, _rope(cfg, L + i, 1, torch.bfloat16, gpu))
            q, k, v = [t.cpu() for t in att.capture[-1]]
            ref_attn, ref_cache = po.decode_step(q, k, v, ref_cache)
            ref_out = ref_attn.reshape(2, 1, -1).float() @ att.o_proj.weight.detach().float().cpu().T
            assert (out.float().cpu() - ref_out).abs().max().item() < 5e-2 * max(1.0, ref_out.abs().max().item())
    assert cache[1].dtype == torch.uint8 and cache[2].dtype == torch.bfloat16


@pytest.mark.parametrize("L", [1, 5, 200, 256])
def test_mixed_attention_forward_matches_reference_restatement(gpu, L):
    """LlamaPolarMixedGroupAttention (polar keys + 4-bit values): prefill, then decode across a
    flush of the shared residual window.  Captured post-RoPE q/k/v are replayed through the oracle's
    Mixed forward: the 11-slot cache must be bit-identical (key codes and metadata, packed value
    words, value scale and zero-point, residual keys and values, kv_seq_len), outputs within tolerance."""
    from polarquant_amd.modeling_llama_polar import LlamaPolarMixedGroupAttention
    torch.manual_seed(5)
    cfg = _tiny(8, 2)
    att = LlamaPolarMixedGroupAttention(cfg, 0).half().to(gpu)
    assert att.vbits == 4
    att.capture = []
    B, steps = 2, 140
    mask = torch.ones(B, L, dtype=torch.int64)
    mask[1, :min(3, L - 1)] = 0
    x = (torch.randn(B, L + steps, cfg.hidden_size) * 0.5).half().to(gpu)
    with torch.no_grad():
        out, cache = att(x[:, :L], attention_mask=mask.to(gpu), past_key_value=None, position_embeddings=_rope(cfg, 0, L, torch.float16, gpu))
    assert isinstance(cache, tuple) and len(cache) == 11 and cache[-1] == L
    q, k, v = [t.cpu() for t in att.capture[-1]]
    ref_cache = po.prefill_cache_mixed(k, v)
    _check_cache(cache, ref_cache)
    o_proj = att.o_proj.weight.detach().float().cpu()
    for i in range(steps):
        mask = torch.cat([mask, torch.ones(B, 1, dtype=torch.int64)], -1)
        with torch.no_grad():
            out, cache = att(x[:, L + i:L + i + 1], attention_mask=mask.to(gpu), past_key_value=cache,
                             position_embeddings=_rope(cfg, L + i, 1, torch.float16, gpu))
        q, k, v = [t.cpu() for t in att.capture[-1]]
        ref_attn, ref_cache = po.decode_step_mixed(q, k, v, ref_cache, mask)
        ref_out = ref_attn.reshape(B, 1, -1).float() @ o_proj.T
        err = (out.float().cpu() - ref_out).abs().max().item()
        assert err < 2e-2 * max(1.0, ref_out.abs().max().item()), (i, err)
        if i in (0, 1, steps // 2, steps - 1) or (L + i + 1) % 128 in (0, 1):
            _check_cache(cache, ref_cache)
    # a plain 11-tuple (no arena) is accepted too
    plain = tuple(t.clone() if torch.is_tensor(t) else t for t in cache)
    with torch.no_grad():
        o1, c1 = att(x[:, -1:], None, cache, _rope(cfg, L + steps, 1, torch.float16, gpu))
        o2, c2 = att(x[:, -1:], None, plain, _rope(cfg, L + steps, 1, torch.float16, gpu))
    assert torch.equal(o1, o2) and c1[-1] == c2[-1] == L + steps + 1


@pytest.mark.parametrize("L", [700, 1400])
def test_snapkv_attention_matches_reference_restatement(gpu, L):
    """LlamaSnapKVAttention: prompt eviction (when L > 1152) + polar cache + decode across a flush.
    The kept set is checked against the oracle's pooled scores (every kept token scores at least the
    oracle's threshold up to half-precision noise; the sets overlap almost entirely), then the oracle
    is given the product's indices and the caches must be bit-identical; decode outputs within tolerance
    and positions continue from the full prompt length."""
    from polarquant_amd.modeling_llama_polar import LlamaSnapKVAttention
    torch.manual_seed(8)
    cfg = _tiny(8, 2)
    att = LlamaSnapKVAttention(cfg, 0).half().to(gpu)
    assert (att.window_size, att.kernel_size, att.max_capacity_prompt) == (128, 7, 1152)
    att.capture = []
    steps = 140
    x = (torch.randn(1, L + steps, cfg.hidden_size) * 0.5).half().to(gpu)
    with torch.no_grad():
        out, cache = att(x[:, :L], None, None, _rope(cfg, 0, L, torch.float16, gpu))
    q, k, v = [t.cpu() for t in att.capture[-1]]
    assert len(cache) == 8 and cache[-1] == L and cache[6].shape[2] == min(L, 1152)
    idx = None
    if L > 1152:
        idx = att.last_selection.cpu()
        s = po.snapkv_scores(q, k).float()
        kth = s.topk(1024, dim=-1).values[..., -1:]
        ref_idx = po.snapkv_select(q, k)
        for h in range(2):
            got, want = set(idx[0, h].tolist()), set(ref_idx[0, h].tolist())
            assert len(got) == 1024 and len(got & want) >= 1000, len(got & want)
            assert bool((s[0, h, idx[0, h]] >= kth[0, h] - 2e-3 * s[0, h].max()).all())
    else:
        assert att.last_selection is None
    ref_cache = po.prefill_cache_snapkv(q, k, v, indices=idx)
    _check_cache(cache, ref_cache)
    o_proj = att.o_proj.weight.detach().float().cpu()
    for i in range(steps):
        with torch.no_grad():
            out, cache = att(x[:, L + i:L + i + 1], None, cache, _rope(cfg, L + i, 1, torch.float16, gpu))
        q, k, v = [t.cpu() for t in att.capture[-1]]
        ref_attn, ref_cache = po.decode_step(q, k, v, ref_cache)
        ref_out = ref_attn.reshape(1, 1, -1).float() @ o_proj.T
        err = (out.float().cpu() - ref_out).abs().max().item()
        assert err < 2e-2 * max(1.0, ref_out.abs().max().item()), (i, err)
        if i in (0, 1, steps - 1) or cache[0] is None or cache[0].shape[2] == 1:
            _check_cache(cache, ref_cache)
    assert cache[-1] == L + steps and cache[6].shape[2] == min(L, 1152) + steps
    # a plain tuple (no arena) whose length slot exceeds its cached tokens is accepted as well
    plain = tuple(t.clone() if torch.is_tensor(t) else t for t in cache)
    with torch.no_grad():
        o1, c1 = att(x[:, -1:], None, cache, _rope(cfg, L + steps, 1, torch.float16, gpu))
        o2, c2 = att(x[:, -1:], None, plain, _rope(cfg, L + steps, 1, torch.float16, gpu))
    assert torch.equal(o1, o2) and c1[-1] == c2[-1] == L + steps + 1
    with pytest.raises(AssertionError):
        att(x[:, -1:].repeat(2, 1, 1), None, c1, _rope(cfg, 0, 1, torch.float16, gpu))      # batch 1 only at decode time


def test_model_shell_selects_the_variants(gpu):
    from polarquant_amd.modeling_llama_polar import LlamaPolarMixedGroupAttention, LlamaSnapKVAttention
    assert isinstance(LlamaPolarForCausalLM(_tiny(layers=1, vbits=4)).model.layers[0].self_attn, LlamaPolarMixedGroupAttention)
    assert isinstance(LlamaPolarForCausalLM(_tiny(layers=1, snapkv=True)).model.layers[0].self_attn, LlamaSnapKVAttention)
    assert type(LlamaPolarForCausalLM(_tiny(layers=1)).model.layers[0].self_attn) is LlamaPolarGroupAttention
    # greedy generation through the SnapKV variant: positions run on from the full prompt length
    torch.manual_seed(9)
    cfg = _tiny(layers=2, snapkv=True)
    model = LlamaPolarForCausalLM(cfg).half().to(gpu).eval()
    ids = torch.randint(0, cfg.vocab_size, (1, 1300), device=gpu)
    out = generate(model, ids, torch.ones_like(ids), GenerationConfig(eos_token_id=[999999]), max_new_tokens=5)
    assert out.shape == (1, 5)
