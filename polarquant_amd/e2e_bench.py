"""End-to-end greedy decode with the polar-key attention (workload configs[4]):
random-init Llama-3-8B architecture (32 layers, hidden 4096, 32 q / 8 KV heads, FFN 14336,
vocab 128256), bf16 weights ~N(0, 0.02), batch 8, prompt 16384 random ids, 256 new tokens.
Reports prefill seconds, decode tokens/s and KV-cache bytes per token.  Mirrors the
reference's throughput script (benchmark/benchmark_throughput.py:15-113): one timed prefill,
then the timed greedy loop with EOS made unreachable.

    python -m polarquant_amd.e2e_bench [--batch 8] [--prompt 16384] [--new 256] [--layers 32] [--graph] [--values4] [--fused-prefill]

--graph replays the decode step from a captured HIP graph (polarquant_amd/graph_decode.py)
instead of driving ~40 launches per layer from Python.
"""
from __future__ import annotations

import argparse
import json
import time

import torch

from .modeling_common import PolarConfig
from .modeling_llama_polar import LlamaPolarForCausalLM


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


def run(batch=8, prompt=16384, new=256, layers=32, graph=False, values4=False, fused_prefill=False, separate_rope=False):
    """One timed prefill and the timed greedy loop -> dict of figures (see the module docstring)."""
    dev = torch.device("cuda:0")
    cfg = PolarConfig.llama3_8b(num_hidden_layers=layers, cache_capacity=prompt + new + 128,
                                eos_token_id=[128256 + 10], vbits=4 if values4 else 16)
    model = build_model(cfg, dev)
    g = torch.Generator(device=dev).manual_seed(1004)
    ids = torch.randint(0, cfg.vocab_size, (batch, prompt), generator=g, device=dev)
    mask = torch.ones_like(ids)
    with torch.no_grad():
        if graph:
            from .graph_decode import PolarGraphDecoder
            dec = PolarGraphDecoder(model, max_len=prompt + new + 128, fused_prefill=fused_prefill,
                                    fused_qkv_rope=not separate_rope)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            logits = dec.prefill(ids)
            torch.cuda.synchronize()
            t_prefill = time.perf_counter() - t0
            tok = logits.argmax(-1)
            tok = dec.step(tok).argmax(-1)          # capture happens on the first step: not timed
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(new - 2):
                tok = dec.step(tok).argmax(-1)
            torch.cuda.synchronize()
            t_decode = time.perf_counter() - t0
            steps = new - 2
            cache = dec.cache()
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
    kv = model.kv_cache_bytes_per_token()
    fp16_kv = cfg.num_hidden_layers * cfg.num_key_value_heads * 2 * 128 * 2
    return {
        "workload": "configs[4]: greedy decode, random-init Llama-3-8B architecture, bf16, batch %d, prompt %d, %d new tokens"
                    % (batch, prompt, new),
        "layers": layers, "graph": bool(graph), "values": "4-bit" if values4 else "half", "prefill_s": round(t_prefill, 3), "decode_s": round(t_decode, 3),
        "decode_ms_per_step": round(1e3 * t_decode / steps, 3),
        "decode_tokens_per_s": round(batch * steps / t_decode, 1),
        "kv_cache_bytes_per_token": kv, "fp16_kv_cache_bytes_per_token": fp16_kv,
        "kv_seq_len": cache[0][-1], "quantized_groups": cache[0][1].shape[2],
        "peak_memory_GiB": round(torch.cuda.max_memory_allocated() / 2 ** 30, 2),
    }


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
    args = ap.parse_args()
    print(json.dumps(run(args.batch, args.prompt, args.new, args.layers, args.graph, args.values4, args.fused_prefill,
                         args.separate_rope)))


if __name__ == "__main__":
    main()
