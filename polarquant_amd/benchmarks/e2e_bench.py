"""End-to-end greedy decode with the polar-key attention (workload configs[4]):
random-init Llama-3-8B architecture (32 layers, hidden 4096, 32 q / 8 KV heads, FFN 14336,
vocab 128256), bf16 weights ~N(0, 0.02), batch 8, prompt 16384 random ids, 256 new tokens.
Reports prefill seconds, decode tokens/s and KV-cache bytes per token.  Mirrors the
reference's throughput script (benchmark/benchmark_throughput.py:15-113): one timed prefill,
then the timed greedy loop with EOS made unreachable.

    python -m polarquant_amd.benchmarks.e2e_bench [--batch 8] [--prompt 16384] [--new 256] [--layers 32] [--graph] [--values4] [--fused-prefill]
                                                  [--fp16-kv same_kernel|sdpa_splitk] [--check-tokens 8]

--graph replays the decode step from a captured HIP graph (polarquant_amd/graph_decode.py)
instead of driving ~40 launches per layer from Python.
--fp16-kv runs the script's other side, the un-quantized model: the same shells and graph with fp16 / bf16 key and
value caches (polarquant_amd/benchmarks/fp16_kv_decoder.py), so that the polar figure has a ratio.
--check-tokens n (with --graph): after the timed loop, the first n greedy steps are redone by the eager model (module
by module, as the reference drives it) on the graph decoder's own tokens, and the two are compared step by step.
"""
from __future__ import annotations

import argparse
import json
import time

import torch

from ..modeling_common import PolarConfig
from ..modeling_llama_polar import LlamaPolarForCausalLM


def build_model(cfg: PolarConfig, device, dtype=torch.bfloat16):
    torch.manual_seed(0)
    with torch.device(device):
        prev = torch.get_default_dtype()
        torch.set_default_dtype(dtype)
        try:
            model = LlamaPolarForCausalLM(cfg)
        finally:
            torch.set_default_dtype(prev)
    g = torch.Generator(device=device).manual_seed(1234)
    with torch.no_grad():
        for name, p in model.named_parameters():
            if p.dim() >= 2:
                p.normal_(0.0, 0.02, generator=g)
    return model.eval()


def _check_against_eager(model, ids, first_logits, graph_tokens, graph_logits):
    """The eager model (the drop-in classes driven module by module) on the same prompt, fed the GRAPH decoder's tokens
    step by step (so that one near-tie cannot send the two runs down different paths): how many of the greedy choices
    agree, how far the logits are apart, and whether everything is finite."""
    mask = torch.ones_like(ids)
    out = model(input_ids=ids, attention_mask=mask, past_key_values=None, num_logits_to_keep=1)
    cache = out.past_key_values
    cos = lambda a, b: float(torch.nn.functional.cosine_similarity(a.float().flatten(1), b.float().flatten(1), dim=1).min())
    agree = int((out.logits.argmax(-1) == first_logits.argmax(-1)).sum())
    total = first_logits.shape[0]
    diff = float((out.logits.float() - first_logits.float()).abs().max())
    worst_cos = cos(out.logits, first_logits)
    finite = bool(torch.isfinite(first_logits.float()).all())
    for tok, lg in zip(graph_tokens, graph_logits):
        mask = torch.cat([mask, torch.ones_like(tok)], dim=-1)
        out = model(input_ids=tok, attention_mask=mask, past_key_values=cache, num_logits_to_keep=1)
        cache = out.past_key_values
        agree += int((out.logits.argmax(-1) == lg.argmax(-1)).sum())
        total += lg.shape[0]
        diff = max(diff, float((out.logits.float() - lg.float()).abs().max()))
        worst_cos = min(worst_cos, cos(out.logits, lg))
        finite = finite and bool(torch.isfinite(lg.float()).all())
    scale = float(first_logits.float().abs().max())
    return {"greedy_tokens_agreeing_with_the_eager_model": "%d of %d" % (agree, total), "steps_compared": len(graph_tokens) + 1,
            "max_abs_logit_diff": round(diff, 5), "max_abs_logit": round(scale, 4),
            "min_cosine_of_a_sequence's_logit_vectors": round(worst_cos, 6), "logits_finite": finite,
            "how": "eager model (module by module, Python-driven) fed the graph decoder's own tokens; all %d layers" % len(model.model.layers)}


def run(batch=8, prompt=16384, new=256, layers=32, graph=False, values4=False, fused_prefill=False, separate_rope=False,
        fp16_kv=None, check_tokens=0):
    """One timed prefill and the timed greedy loop -> dict of figures (see the module docstring)."""
    dev = torch.device("cuda:0")
    torch.cuda.reset_peak_memory_stats()
    cfg = PolarConfig.llama3_8b(num_hidden_layers=layers, cache_capacity=prompt + new + 128,
                                eos_token_id=[128256 + 10], vbits=4 if values4 else 16)
    model = build_model(cfg, dev)
    g = torch.Generator(device=dev).manual_seed(1004)
    ids = torch.randint(0, cfg.vocab_size, (batch, prompt), generator=g, device=dev)
    mask = torch.ones_like(ids)
    with torch.no_grad():
        sanity = None
        if graph or fp16_kv:
            if fp16_kv:
                from .fp16_kv_decoder import Fp16KVGraphDecoder
                dec = Fp16KVGraphDecoder(model, max_len=prompt + new + 128, attention=fp16_kv)
            else:
                from ..graph_decode import PolarGraphDecoder
                dec = PolarGraphDecoder(model, max_len=prompt + new + 128, fused_prefill=fused_prefill,
                                        fused_qkv_rope=not separate_rope)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            logits = dec.prefill(ids)
            torch.cuda.synchronize()
            t_prefill = time.perf_counter() - t0
            first_logits = logits.clone()
            kept_tok, kept_logits = [], []
            tok = logits.argmax(-1)
            kept_tok.append(tok)
            lg = dec.step(tok)                       # capture happens on the first step: not timed
            kept_logits.append(lg.clone())
            tok = lg.argmax(-1)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for i in range(new - 2):
                if i + 1 < check_tokens:             # (clones of a [B, 1, vocab] tensor: microseconds, the first steps only)
                    kept_tok.append(tok)
                lg = dec.step(tok)
                if i + 1 < check_tokens:
                    kept_logits.append(lg.clone())
                tok = lg.argmax(-1)
            torch.cuda.synchronize()
            t_decode = time.perf_counter() - t0
            steps = new - 2
            cache = dec.cache()
            peak = torch.cuda.max_memory_allocated()        # before the check below builds the eager model's own cache
            if check_tokens and not fp16_kv:
                n = min(check_tokens, len(kept_logits))
                sanity = _check_against_eager(model, ids, first_logits, kept_tok[:n], kept_logits[:n])
        else:
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            out = model(input_ids=ids, attention_mask=mask, past_key_values=None, num_logits_to_keep=1)
            torch.cuda.synchronize()
            t_prefill = time.perf_counter() - t0
            cache = out.past_key_values
            tok = out.logits.argmax(-1)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(new - 1):
                mask = torch.cat([mask, torch.ones_like(tok)], dim=-1)
                out = model(input_ids=tok, attention_mask=mask, past_key_values=cache, num_logits_to_keep=1)
                cache = out.past_key_values
                tok = out.logits.argmax(-1)
            torch.cuda.synchronize()
            t_decode = time.perf_counter() - t0
            steps = new - 1
            peak = torch.cuda.max_memory_allocated()
    kv = model.kv_cache_bytes_per_token()
    fp16_bytes = cfg.num_hidden_layers * cfg.num_key_value_heads * 2 * 128 * 2
    if fp16_kv:
        return {
            "workload": "configs[4] with an un-quantized KV cache (model dtype keys and values, attention: %s): greedy decode, "
                        "random-init Llama-3-8B architecture, bf16, batch %d, prompt %d, %d new tokens" % (fp16_kv, batch, prompt, new),
            "layers": layers, "graph": True, "attention": fp16_kv, "prefill_s": round(t_prefill, 3), "decode_s": round(t_decode, 3),
            "decode_ms_per_step": round(1e3 * t_decode / steps, 3), "decode_tokens_per_s": round(batch * steps / t_decode, 1),
            "kv_cache_bytes_per_token": fp16_bytes, "kv_seq_len": cache[0][-1],
            "peak_memory_GiB": round(peak / 2 ** 30, 2),
        }
    res = {
        "workload": "configs[4]: greedy decode, random-init Llama-3-8B architecture, bf16, batch %d, prompt %d, %d new tokens"
                    % (batch, prompt, new),
        "layers": layers, "graph": bool(graph), "values": "4-bit" if values4 else "half", "prefill_s": round(t_prefill, 3), "decode_s": round(t_decode, 3),
        "decode_ms_per_step": round(1e3 * t_decode / steps, 3),
        "decode_tokens_per_s": round(batch * steps / t_decode, 1),
        "kv_cache_bytes_per_token": kv, "fp16_kv_cache_bytes_per_token": fp16_bytes,
        "kv_seq_len": cache[0][-1], "quantized_groups": cache[0][1].shape[2],
        "peak_memory_GiB": round(peak / 2 ** 30, 2),
    }
    if sanity is not None:
        res["sanity"] = sanity
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt", type=int, default=16384)
    ap.add_argument("--new", type=int, default=256)
    ap.add_argument("--layers", type=int, default=32)
    ap.add_argument("--graph", action="store_true")
    ap.add_argument("--values4", action="store_true", help="4-bit values as well (the reference's Mixed variant)")
    ap.add_argument("--fused-prefill", action="store_true", help="with --graph: fused norm / SiLU kernels in the prompt pass too")
    ap.add_argument("--separate-rope", action="store_true", help="with --graph: q|k|v projection and RoPE + append as two launches")
    ap.add_argument("--fp16-kv", choices=["same_kernel", "sdpa_splitk"], default=None,
                    help="the un-quantized baseline: model-dtype key and value caches, graph decode")
    ap.add_argument("--check-tokens", type=int, default=0, help="with --graph: compare the first n greedy steps with the eager model")
    args = ap.parse_args()
    print(json.dumps(run(args.batch, args.prompt, args.new, args.layers, args.graph, args.values4, args.fused_prefill,
                         args.separate_rope, args.fp16_kv, args.check_tokens)))


if __name__ == "__main__":
    main()
