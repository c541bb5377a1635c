"""Seeded random differential test of the drop-in attention classes: random head layout, bit widths, dtype, batch,
prompt length, left padding and number of decode steps (so that flushes of the residual window fall at random places),
plain or Mixed (4-bit values) variant.  Every call's post-RoPE q / k / v are captured on the GPU and replayed through the
oracle's restatement of the reference forward: the cache tuple must be bit-identical, the outputs within tolerance."""
import os
import random

import pytest
import torch

from oracle import polar_oracle as po
from polarquant_amd.modeling_common import PolarConfig
from polarquant_amd.modeling_llama_polar import LlamaPolarGroupAttention, LlamaPolarMixedGroupAttention
from polarquant_amd.modeling_qwen_polar import Qwen2PolarGroupAttention

pytestmark = pytest.mark.gpu
# more seeds: PQ_RANDOM_MODEL_CASES=200; another stretch of them: PQ_RANDOM_MODEL_FIRST=1000
SEEDS = range(int(os.environ.get("PQ_RANDOM_MODEL_FIRST", "0")),
              int(os.environ.get("PQ_RANDOM_MODEL_FIRST", "0")) + int(os.environ.get("PQ_RANDOM_MODEL_CASES", "8")))
BITS = [(4, 4), (3, 3), (4, 2), (5, 3), (2, 4), (3, 5), (2, 6), (1, 7)]


def _rope(theta, start, n, dtype, dev):
    inv = 1.0 / (theta ** (torch.arange(0, 128, 2, dtype=torch.float32) / 128))
    ang = torch.arange(start, start + n, dtype=torch.float32)[:, None] * inv[None]
    emb = torch.cat([ang, ang], -1)[None]
    return emb.cos().to(dtype).to(dev), emb.sin().to(dtype).to(dev)


def _same_cache(got, ref, where):
    assert got[-1] == ref[-1], where
    for j, (g, r) in enumerate(zip(got[:-1], ref[:-1])):
        assert (g is None) == (r is None), (where, "tuple element %d" % j)
        if g is not None:
            g = g.cpu()
            assert g.shape == r.shape and g.dtype == r.dtype, (where, "tuple element %d" % j)
            if g.dtype in (torch.uint8, torch.int32):
                assert torch.equal(g, r), (where, "codes differ (tuple element %d)" % j)
            else:
                assert bool((g.float() == r.float()).all()), (where, "tuple element %d differs" % j)


@pytest.mark.parametrize("seed", SEEDS)
def test_random_attention_class_case(gpu, seed):
    rnd = random.Random(31000 + seed)
    n_kv = rnd.choice([1, 2, 4])
    n_heads = n_kv * rnd.randint(1, 8 if n_kv < 4 else 4)
    mixed = rnd.random() < 0.35
    rb, tb = (4, 4) if mixed and rnd.random() < 0.5 else rnd.choice(BITS)
    dtype = torch.bfloat16 if seed % 5 == 4 else torch.float16
    B = rnd.randint(1, 3)
    L = rnd.choice([1, rnd.randint(2, 127), 128, rnd.randint(129, 400)])
    steps = rnd.randint(1, 150)
    pads = [rnd.randint(0, min(5, L - 1)) if rnd.random() < 0.5 else 0 for _ in range(B)]
    qwen = not mixed and rnd.random() < 0.3
    print("case", dict(seed=seed, heads=(n_heads, n_kv), bits=(rb, tb), mixed=mixed, qwen=qwen, dtype=str(dtype), B=B, L=L,
                       steps=steps, pads=pads), flush=True)
    torch.manual_seed(seed)
    cfg = PolarConfig(hidden_size=n_heads * 128, num_attention_heads=n_heads, num_key_value_heads=n_kv,
                      num_hidden_layers=1, intermediate_size=256, vocab_size=100, rope_theta=1e4, eos_token_id=[999999],
                      rbits=rb, tbits=tb)
    cls = LlamaPolarMixedGroupAttention if mixed else (Qwen2PolarGroupAttention if qwen else LlamaPolarGroupAttention)
    att = cls(cfg, 0).to(dtype).to(gpu)
    att.capture = []
    mask = torch.ones(B, L, dtype=torch.int64)
    for b, p in enumerate(pads):
        mask[b, :p] = 0
    use_mask = any(pads) or rnd.random() < 0.5
    x = (torch.randn(B, L + steps, cfg.hidden_size) * 0.5).to(dtype).to(gpu)
    prefill = po.prefill_cache_mixed if mixed else po.prefill_cache
    step_fn = po.decode_step_mixed if mixed else po.decode_step
    bits = (rb, tb)
    with torch.no_grad():
        out, cache = att(x[:, :L], attention_mask=mask.to(gpu) if use_mask else None, past_key_value=None,
                         position_embeddings=_rope(cfg.rope_theta, 0, L, dtype, gpu))
    assert cache[-1] == L and len(cache) == (11 if mixed else 8)
    q, k, v = [t.cpu() for t in att.capture[-1]]
    ref_cache = prefill(k, v, *bits)
    _same_cache(cache, ref_cache, "after the prompt")
    o_proj = att.o_proj.weight.detach().float().cpu()
    tol = 2e-2 if dtype == torch.float16 else 5e-2
    for i in range(steps):
        mask = torch.cat([mask, torch.ones(B, 1, dtype=torch.int64)], -1)
        with torch.no_grad():
            out, cache = att(x[:, L + i:L + i + 1], attention_mask=mask.to(gpu) if use_mask else None, past_key_value=cache,
                             position_embeddings=_rope(cfg.rope_theta, L + i, 1, dtype, gpu))
        q, k, v = [t.cpu() for t in att.capture[-1]]
        ref_attn, ref_cache = step_fn(q, k, v, ref_cache, mask if use_mask else None, *bits)
        ref_out = ref_attn.reshape(B, 1, -1).float() @ o_proj.T
        assert torch.isfinite(out.float()).all()
        err = (out.float().cpu() - ref_out).abs().max().item()
        assert err < tol * max(1.0, ref_out.abs().max().item()), (i, err)
        if i in (0, steps - 1) or (L + i + 1) % 128 in (0, 1):
            _same_cache(cache, ref_cache, "after decode step %d" % i)
