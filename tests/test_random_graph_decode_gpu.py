"""Seeded random differential test of the graph decoder: random tiny models (head layout, bit widths, layers, dtype,
plain / Qwen / Mixed), batch, prompt length, left padding and number of new tokens.  The captured graph's replays must be
bit-identical to the same step run eagerly, and both must follow the drop-in model (which chooses its split per call, so
sums associate differently) to rounding, across the flushes of the residual window wherever they fall."""
import os
import random

import pytest
import torch

from polarquant_amd.graph_decode import PolarGraphDecoder
from polarquant_amd.modeling_common import PolarConfig
from polarquant_amd.modeling_llama_polar import LlamaPolarForCausalLM
from polarquant_amd.modeling_qwen_polar import Qwen2PolarForCausalLM

pytestmark = pytest.mark.gpu
# more seeds: PQ_RANDOM_GRAPH_CASES=100; another stretch of them: PQ_RANDOM_GRAPH_FIRST=1000
SEEDS = range(int(os.environ.get("PQ_RANDOM_GRAPH_FIRST", "0")),
              int(os.environ.get("PQ_RANDOM_GRAPH_FIRST", "0")) + int(os.environ.get("PQ_RANDOM_GRAPH_CASES", "4")))
BITS = [(4, 4), (3, 3), (4, 2), (2, 4), (3, 5), (2, 6), (1, 7)]


@pytest.mark.parametrize("seed", SEEDS)
def test_random_graph_decoder_case(gpu, seed):
    rnd = random.Random(52000 + seed)
    n_kv = rnd.choice([1, 2, 4])
    n_heads = n_kv * rnd.randint(1, 8 if n_kv < 4 else 4)
    mixed = rnd.random() < 0.3
    qwen = not mixed and rnd.random() < 0.3
    rb, tb = rnd.choice(BITS)
    dtype = torch.bfloat16 if seed % 4 == 3 else torch.float16
    layers = rnd.randint(1, 2)
    B = rnd.choice([1, 2, 3, 8, 9])              # 9: more rows than the fused q|k|v projection takes
    L = rnd.choice([rnd.randint(1, 127), 128, rnd.randint(129, 300)])
    new = rnd.randint(1, 140)
    padded = rnd.random() < 0.4 and L > 1
    print("case", dict(seed=seed, heads=(n_heads, n_kv), bits=(rb, tb), mixed=mixed, qwen=qwen, dtype=str(dtype), layers=layers,
                       B=B, L=L, new=new, padded=padded), flush=True)
    torch.manual_seed(seed)
    kw = dict(vbits=4) if mixed else (dict(attention_bias=True) if qwen else {})
    cfg = PolarConfig(hidden_size=n_heads * 128, num_attention_heads=n_heads, num_key_value_heads=n_kv,
                      num_hidden_layers=layers, intermediate_size=256, vocab_size=500, rope_theta=1e4, eos_token_id=[999999],
                      rbits=rb, tbits=tb, **kw)
    model = (Qwen2PolarForCausalLM if qwen else LlamaPolarForCausalLM)(cfg).to(dtype).to(gpu).eval()
    ids = torch.randint(0, cfg.vocab_size, (B, L), device=gpu)
    mask = None
    if padded:
        mask = torch.ones(B, L, dtype=torch.int64, device=gpu)
        for b in range(B):
            mask[b, :rnd.randint(0, min(L - 1, 60))] = 0
    dec_g = PolarGraphDecoder(model, max_len=L + new + 8, use_graph=True)
    dec_e = PolarGraphDecoder(model, max_len=L + new + 8, use_graph=False)
    with torch.no_grad():
        ref = model(input_ids=ids, attention_mask=mask, past_key_values=None, num_logits_to_keep=1)
        for d in (dec_g, dec_e):
            assert torch.equal(d.prefill(ids, mask), ref.logits)
        cache, tok = ref.past_key_values, ref.logits.argmax(-1)
        for s in range(new):
            if mask is not None:
                mask = torch.cat([mask, torch.ones_like(tok)], dim=-1)
            ref = model(input_ids=tok, attention_mask=mask, past_key_values=cache, num_logits_to_keep=1)
            cache = ref.past_key_values
            got_e, got_g = dec_e.step(tok).clone(), dec_g.step(tok).clone()
            torch.cuda.synchronize()
            assert torch.equal(got_g, got_e), "graph replay %d differs from the eager step" % s
            rl = ref.logits.float()
            assert torch.isfinite(got_g.float()).all()
            err = (got_g.float() - rl).abs().max().item()
            assert err <= 2e-2 * max(1.0, rl.abs().max().item()), (s, err)
            tok = ref.logits.argmax(-1)
        for a, b in zip(dec_g.cache(), dec_e.cache()):
            assert a[-1] == b[-1] == L + new
            for x, y in zip(a[:-1], b[:-1]):
                assert (x is None) == (y is None)
                if x is not None:
                    assert x.shape == y.shape and torch.equal(x, y)
