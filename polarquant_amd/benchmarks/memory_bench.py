"""Peak-memory protocol of the reference (benchmark/benchmark_memory.py:12-77, 84-94): a prompt of `input_length`
random ids, `output_length` greedily generated tokens with the stop token made unreachable, and the peak of the
allocator over prompt pass + generation, in GB (1e9 bytes), per batch size.  The model is the random-init Llama-3-8B
architecture in fp16 (no weights can be fetched here; memory does not depend on their values).

    python -m polarquant_amd.benchmarks.memory_bench [--batch_size 1 4 16] [--input_length 256] [--output_length 4096]
                                          [--layers 32] [--values4] [--eager]

One JSON line per batch size: peak memory, the part of it that is weights, and the cache's size by the per-token
formula next to what an fp16 cache of the same shape would take.  The steps after the prompt replay a captured HIP
graph unless --eager is given (the reference drives every launch from Python; the memory is the same, the time is not).
"""
from __future__ import annotations

import argparse
import json
import time

import torch

from .e2e_bench import build_model
from ..modeling_common import GenerationConfig, PolarConfig, generate


def run(batch_size: int, input_length: int, output_length: int, layers: int = 32, values4: bool = False, eager: bool = False):
    dev = torch.device("cuda:0")
    cfg = PolarConfig.llama3_8b(num_hidden_layers=layers, cache_capacity=input_length + output_length + 128,
                                eos_token_id=[128256 + 10], vbits=4 if values4 else 16)
    model = build_model(cfg, dev, dtype=torch.float16)
    weights = sum(p.numel() * p.element_size() for p in model.parameters())
    g = torch.Generator(device=dev).manual_seed(7)
    prompts = torch.randint(0, 10000, (batch_size, input_length), generator=g, device=dev)      # :85
    gen = GenerationConfig(eos_token_id=[cfg.vocab_size + 10])                                    # :149
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    torch.cuda.reset_peak_memory_stats()                                                          # :25
    t0 = time.perf_counter()
    out = generate(model, prompts, None, gen, max_new_tokens=output_length, graph_decoder=not eager)
    torch.cuda.synchronize()
    seconds = time.perf_counter() - t0
    peak = torch.cuda.max_memory_allocated()                                                      # :75
    tokens = input_length + out.shape[1]
    per_token = model.kv_cache_bytes_per_token()
    fp16_per_token = layers * cfg.num_key_value_heads * 2 * 128 * 2
    del model, out
    torch.cuda.empty_cache()
    return {"batch_size": batch_size, "input_length": input_length, "output_length": output_length, "layers": layers,
            "values": "4-bit" if values4 else "half", "peak_memory_GB": round(peak / 1e9, 2), "weights_GB": round(weights / 1e9, 2),
            "kv_cache_GB": round(batch_size * tokens * per_token / 1e9, 3),
            "fp16_kv_cache_GB": round(batch_size * tokens * fp16_per_token / 1e9, 3),
            "kv_cache_bytes_per_token": per_token, "seconds": round(seconds, 1)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--batch_size", type=int, nargs="*", default=[1, 4, 16])
    ap.add_argument("--input_length", type=int, default=256)
    ap.add_argument("--output_length", type=int, default=4096)
    ap.add_argument("--layers", type=int, default=32)
    ap.add_argument("--values4", action="store_true")
    ap.add_argument("--eager", action="store_true")
    args = ap.parse_args()
    for b in args.batch_size:
        print(json.dumps(run(b, args.input_length, args.output_length, args.layers, args.values4, args.eager)), flush=True)


if __name__ == "__main__":
    main()
