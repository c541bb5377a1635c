"""The decode step captured in a HIP graph against the eager drop-in modules: same tokens, same
logits, same cache, on every replay, across residual flushes, with eager work between replays."""
import pytest
import torch

from polarquant_amd.graph_decode import PolarGraphDecoder
from polarquant_amd.modeling_common import PolarConfig
from polarquant_amd.modeling_llama_polar import LlamaPolarForCausalLM
from polarquant_amd.modeling_qwen_polar import Qwen2PolarForCausalLM

pytestmark = pytest.mark.gpu


def _tiny(n_heads=4, n_kv=2, layers=2, **kw):
    return PolarConfig(hidden_size=n_heads * 128, num_attention_heads=n_heads, num_key_value_heads=n_kv,
                       num_hidden_layers=layers, intermediate_size=512, vocab_size=1000, rope_theta=1e4,
                       eos_token_id=[999999], **kw)


def _same_cache(a, b):
    assert a[-1] == b[-1]
    for x, y in zip(a[:-1], b[:-1]):
        assert (x is None) == (y is None)
        if x is not None:
            assert x.shape == y.shape and torch.equal(x, y)


@pytest.mark.parametrize("cls,cfg,dtype", [
    (LlamaPolarForCausalLM, _tiny(), torch.float16),
    (Qwen2PolarForCausalLM, _tiny(7, 1, rbits=3, tbits=3, attention_bias=True), torch.bfloat16),
    (LlamaPolarForCausalLM, _tiny(8, 2, vbits=4), torch.float16),          # Mixed variant: 4-bit values, 11-slot cache
])
def test_graph_decoder_matches_eager_model(gpu, cls, cfg, dtype):
    """Four decoders in lock step over 140 tokens (two residual flushes): the eager drop-in model;
    the static-state step with the eager modules' own elementwise ops (unfused); the static-state
    step with the fused HIP elementwise kernels, run eagerly; and that same step replayed from a
    captured graph.
    Graph replay vs eager fused step: bit-identical logits on every replay and identical caches
    (same kernels, same launch shapes).  Unfused static step vs drop-in model: the split count is
    fixed for the capacity instead of chosen per call, so partial sums associate differently: logits
    agree to rounding, the first layer's cache (which no attention output feeds) exactly.  Fused vs
    drop-in model: the norms may differ in the last bit, so logits agree to rounding."""
    torch.manual_seed(11)
    model = cls(cfg).to(dtype).to(gpu).eval()
    B, L, new = 2, 250, 140                      # flushes at 256 and 384 tokens
    ids = torch.randint(0, cfg.vocab_size, (B, L), device=gpu)
    dec_g = PolarGraphDecoder(model, max_len=L + new + 8, use_graph=True)
    dec_e = PolarGraphDecoder(model, max_len=L + new + 8, use_graph=False)
    dec_u = PolarGraphDecoder(model, max_len=L + new + 8, use_graph=False, fused_ops=False)
    dec_l = PolarGraphDecoder(model, max_len=L + new + 8, use_graph=False, small_m_gemm=False)   # library GEMMs
    with torch.no_grad():
        ref = model(input_ids=ids, attention_mask=None, past_key_values=None, num_logits_to_keep=1)
        for d in (dec_g, dec_e, dec_u, dec_l):
            assert torch.equal(d.prefill(ids), ref.logits)
        cache = ref.past_key_values
        tok = ref.logits.argmax(-1)
        for s in range(new):
            ref = model(input_ids=tok, attention_mask=None, past_key_values=cache, num_logits_to_keep=1)
            cache = ref.past_key_values
            got_u = dec_u.step(tok).clone()
            got_e = dec_e.step(tok).clone()
            got_l = dec_l.step(tok).clone()
            got_g = dec_g.step(tok).clone()
            torch.cuda.synchronize()
            assert torch.equal(got_g, got_e), "graph replay %d differs from the eager step" % s
            rl = ref.logits.float()
            for got in (got_u, got_e, got_l):
                err = (got.float() - rl).abs().max().item()
                assert err <= 2e-2 * max(1.0, rl.abs().max().item()), (s, err)
                # the token the static step would pick is (nearly) the model's best
                pick = rl.gather(-1, got.argmax(-1, keepdim=True)).squeeze(-1)
                assert bool((rl.max(-1).values - pick <= 2 * err + 1e-6).all()), s
            if s % 16 == 0 or s in (5, 6, 7, 133, 134, 135, new - 1):
                for a, b in zip(dec_g.cache(), dec_e.cache()):
                    _same_cache(a, b)
                _same_cache(dec_u.cache()[0], cache[0])
            tok = ref.logits.argmax(-1)
        assert dec_g.kv_len == L + new == cache[0][-1]
        assert dec_g.graph is not None and dec_e.graph is None


@pytest.mark.parametrize("mixed", [False, True])
def test_graph_decoder_with_left_padded_prompt(gpu, mixed):
    """The prompt's padding mask is carried as a static mask over the whole capacity: graph replay, eager
    static step and the drop-in model (which grows its mask by one column per token) agree across a flush."""
    torch.manual_seed(21)
    cfg = _tiny(8, 2, vbits=4) if mixed else _tiny()
    model = LlamaPolarForCausalLM(cfg).half().to(gpu).eval()
    B, L, new = 3, 120, 20                        # flush at 128 tokens
    ids = torch.randint(0, cfg.vocab_size, (B, L), device=gpu)
    mask = torch.ones(B, L, dtype=torch.int64, device=gpu)
    mask[1, :7] = 0
    mask[2, :50] = 0
    dec_g = PolarGraphDecoder(model, max_len=L + new + 8, use_graph=True)
    dec_e = PolarGraphDecoder(model, max_len=L + new + 8, use_graph=False)
    with torch.no_grad():
        ref = model(input_ids=ids, attention_mask=mask, past_key_values=None, num_logits_to_keep=1)
        for d in (dec_g, dec_e):
            assert torch.equal(d.prefill(ids, mask), ref.logits)
        cache, tok = ref.past_key_values, ref.logits.argmax(-1)
        for s in range(new):
            mask = torch.cat([mask, torch.ones_like(tok)], dim=-1)
            ref = model(input_ids=tok, attention_mask=mask, past_key_values=cache, num_logits_to_keep=1)
            cache = ref.past_key_values
            got_e, got_g = dec_e.step(tok).clone(), dec_g.step(tok).clone()
            torch.cuda.synchronize()
            assert torch.equal(got_g, got_e), s
            rl = ref.logits.float()
            err = (got_g.float() - rl).abs().max().item()
            assert err <= 2e-2 * max(1.0, rl.abs().max().item()), (s, err)
            tok = ref.logits.argmax(-1)
        # the mask matters: without it the padded sequences' logits move
        dec_n = PolarGraphDecoder(model, max_len=L + new + 8, use_graph=False)
        dec_n.prefill(ids, None)
        assert not torch.allclose(dec_n.step(tok)[2].float(), dec_e.step(tok)[2].float(), atol=1e-3)


def test_fused_prompt_pass_agrees_with_the_eager_model_to_rounding(gpu):
    """fused_prefill: norms and SiLU * up of the prompt pass through the fused kernels (more rows than one
    launch of the activation kernel takes are split).  Logits of the prompt and of later steps agree with the
    eager model to rounding; the cache bookkeeping is the same."""
    torch.manual_seed(23)
    cfg = _tiny()
    model = LlamaPolarForCausalLM(cfg).half().to(gpu).eval()
    B, L, new = 2, 300, 12
    ids = torch.randint(0, cfg.vocab_size, (B, L), device=gpu)
    dec = PolarGraphDecoder(model, max_len=L + new + 8, fused_prefill=True)
    with torch.no_grad():
        ref = model(input_ids=ids, attention_mask=None, past_key_values=None, num_logits_to_keep=1)
        got = dec.prefill(ids)
        rl = ref.logits.float()
        assert (got.float() - rl).abs().max().item() <= 2e-2 * max(1.0, rl.abs().max().item())
        cache, tok = ref.past_key_values, ref.logits.argmax(-1)
        assert dec.kv_len == L and dec.arenas[0].n_groups == cache[0][1].shape[2] == 2
        for s in range(new):
            ref = model(input_ids=tok, attention_mask=None, past_key_values=cache, num_logits_to_keep=1)
            cache = ref.past_key_values
            got = dec.step(tok)
            rl = ref.logits.float()
            assert (got.float() - rl).abs().max().item() <= 2e-2 * max(1.0, rl.abs().max().item()), s
            tok = ref.logits.argmax(-1)


def test_silu_mul_splits_more_rows_than_one_launch_takes(gpu):
    from polarquant_amd.decode_ops import silu_mul
    g = torch.Generator().manual_seed(3)
    gate = torch.randn(70000, 64, generator=g).half().to(gpu)
    up = torch.randn(70000, 64, generator=g).half().to(gpu)
    y = silu_mul(gate, up)
    ref = (torch.nn.functional.silu(gate.float()).half().float() * up.float()).half()
    assert (y.float() - ref.float()).abs().max().item() <= 2e-3 * ref.float().abs().max().item()
    assert torch.equal(y[65535:], silu_mul(gate[65535:].contiguous(), up[65535:].contiguous()))


def test_generate_with_the_graph_decoder(gpu):
    """`generate(..., graph_decoder=True)`: the reference's loop with the steps replayed from the graph.  Same tokens
    as driving the decoder by hand; against the eager loop the tokens agree until a near-tie (checked: every token
    picked is within rounding of the eager model's best at that step); stops when every sequence has hit a stop id."""
    from polarquant_amd.modeling_common import GenerationConfig, generate
    torch.manual_seed(31)
    cfg = _tiny()
    model = LlamaPolarForCausalLM(cfg).half().to(gpu).eval()
    B, L, new = 2, 125, 12                         # flush at 128 tokens
    ids = torch.randint(0, cfg.vocab_size, (B, L), device=gpu)
    mask = torch.ones(B, L, dtype=torch.int64, device=gpu)
    mask[1, :9] = 0
    gc = GenerationConfig(eos_token_id=[999999])
    got = generate(model, ids, mask, gc, max_new_tokens=new, graph_decoder=True)
    assert got.shape == (B, new)
    dec = PolarGraphDecoder(model, max_len=L + new + 1)
    with torch.no_grad():
        tok = dec.prefill(ids, mask).argmax(-1)
        by_hand = [tok]
        for _ in range(new - 1):
            tok = dec.step(tok).argmax(-1)
            by_hand.append(tok)
    assert torch.equal(got, torch.cat(by_hand, dim=-1))
    # the eager model, fed the graph decoder's tokens, would have picked (nearly) the same at every step
    with torch.no_grad():
        m, cache, tok = mask, None, ids
        for s in range(new):
            out = model(input_ids=tok, attention_mask=m, past_key_values=cache, num_logits_to_keep=1)
            cache, rl = out.past_key_values, out.logits.float()
            tok = got[:, s:s + 1]
            pick = rl.gather(-1, tok.unsqueeze(-1)).squeeze(-1)
            assert bool((rl.max(-1).values - pick <= 4e-2 * max(1.0, rl.abs().max().item())).all()), s
            m = torch.cat([m, torch.ones_like(tok)], dim=-1)
    # stop ids: every sequence's first token is a stop id -> one token comes back
    first = got[:, 0].tolist()
    short = generate(model, ids, mask, GenerationConfig(eos_token_id=first), max_new_tokens=new, graph_decoder=True)
    assert short.shape == (B, 1) and torch.equal(short, got[:, :1])
    # sampling draws from the same filtered distribution: valid ids, right shape
    torch.manual_seed(5)
    smp = generate(model, ids, None, GenerationConfig(eos_token_id=[999999], top_k=5), do_sample=True, max_new_tokens=4,
                   graph_decoder=True)
    assert smp.shape == (B, 4) and int(smp.min()) >= 0 and int(smp.max()) < cfg.vocab_size


def test_generate_with_the_graph_decoder_on_the_mixed_variant(gpu):
    """4-bit values (11-slot cache) and a Qwen-shaped model with biases through `generate(..., graph_decoder=True)`:
    same tokens as the decoder driven by hand, every pick within rounding of the eager model's best."""
    from polarquant_amd.modeling_common import GenerationConfig, generate
    for cls, cfg, dtype in ((LlamaPolarForCausalLM, _tiny(8, 2, vbits=4), torch.float16),
                            (Qwen2PolarForCausalLM, _tiny(7, 1, rbits=3, tbits=3, attention_bias=True), torch.bfloat16)):
        torch.manual_seed(37)
        model = cls(cfg).to(dtype).to(gpu).eval()
        B, L, new = 2, 250, 10                     # flush at 256 tokens
        ids = torch.randint(0, cfg.vocab_size, (B, L), device=gpu)
        got = generate(model, ids, None, GenerationConfig(eos_token_id=[999999]), max_new_tokens=new, graph_decoder=True)
        assert got.shape == (B, new)
        dec = PolarGraphDecoder(model, max_len=L + new + 1)
        with torch.no_grad():
            tok = dec.prefill(ids).argmax(-1)
            by_hand = [tok]
            for _ in range(new - 1):
                tok = dec.step(tok).argmax(-1)
                by_hand.append(tok)
            assert torch.equal(got, torch.cat(by_hand, dim=-1))
            cache, tok = None, ids
            for s in range(new):
                out = model(input_ids=tok, attention_mask=None, past_key_values=cache, num_logits_to_keep=1)
                cache, rl = out.past_key_values, out.logits.float()
                tok = got[:, s:s + 1]
                pick = rl.gather(-1, tok.unsqueeze(-1)).squeeze(-1)
                assert bool((rl.max(-1).values - pick <= 4e-2 * max(1.0, rl.abs().max().item())).all()), (cls.__name__, s)


def test_graph_decoder_rejects_overflow(gpu):
    torch.manual_seed(12)
    cfg = _tiny(layers=1)
    model = LlamaPolarForCausalLM(cfg).half().to(gpu).eval()
    ids = torch.randint(0, cfg.vocab_size, (1, 10), device=gpu)
    dec = PolarGraphDecoder(model, max_len=12, use_graph=False)
    dec.prefill(ids)
    tok = torch.zeros(1, 1, dtype=torch.long, device=gpu)
    dec.step(tok)
    dec.step(tok)
    with pytest.raises(AssertionError):
        dec.step(tok)
