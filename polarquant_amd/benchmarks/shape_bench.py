"""Fused decode attention at head layouts and sizes other than the benchmark configurations: the default kernels (a
scorer / accumulator pair of wavefronts per slice) beside the kernels with one wavefront per slice.

    python -m polarquant_amd.benchmarks.shape_bench

One JSON line per shape: batch, query heads, KV heads, context, bits, dtype -> us per step (attention + merge) of
both forms and their fractions of the 8 TB/s HBM peak on algorithmic bytes.  Uniform batches, one residual key,
random keys quantized on the GPU, values N(0,1).
"""
from __future__ import annotations

import json

import torch

from .. import workloads as wl
from ..attention import polar_decode_attention
from ..quantize import quantize_and_pack_nbit

SHAPES = [
    # B, N, Nk, L, rbits, tbits, dtype
    (4, 32, 32, 32768, 4, 4, torch.float16),       # MHA (Llama-2-7B heads)
    (16, 16, 8, 32768, 4, 4, torch.float16),       # 2 heads per KV head
    (16, 32, 8, 32768, 4, 4, torch.bfloat16),      # configs[1]'s shape in bfloat16
    (16, 28, 4, 32768, 3, 3, torch.float16),       # 7 heads per KV head, uniform lengths
    (16, 64, 8, 32768, 4, 4, torch.float16),       # 8 heads per KV head, 16 angle bins: the largest table
    (8, 32, 8, 4096, 4, 4, torch.float16),         # short contexts
    (64, 32, 8, 2048, 4, 4, torch.float16),
    (128, 32, 8, 2048, 4, 4, torch.float16),       # one slice per plane: the default kernels write the output, no merge
    (256, 32, 8, 1024, 4, 4, torch.float16),
]


def main():
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(5)
    for B, N, Nk, L, rb, tb, dt in SHAPES:
        ng = L // 128
        keys = torch.randn(B, Nk, L, 128, generator=g, device=dev).to(dt)
        quant = quantize_and_pack_nbit(keys, rb, tb)
        del keys
        v = torch.randn(B, Nk, L + 1, 128, generator=g, device=dev).to(dt)
        kres = torch.randn(B, Nk, 128, 128, generator=g, device=dev).to(dt)
        q = torch.randn(B, N, 1, 128, generator=g, device=dev).to(dt)
        nbytes = wl.algorithmic_bytes(Nk, N, [L] * B, [1] * B, rb, tb)
        row = dict(batch=B, heads=N, kv_heads=Nk, context=L, bits="%d/%d" % (rb, tb), dtype=str(dt)[6:], algorithmic_bytes=int(nbytes))
        outs = []
        for name, single in (("pairs", False), ("one_wavefront", True)):
            call = lambda: polar_decode_attention(q, *quant, kres, v, ng, 1, rbits=rb, tbits=tb, single_wavefront=single)
            outs.append(call().float())
            ms = min(wl.time_events(call, 30, 5) for _ in range(2))
            row[name + "_us"] = round(ms * 1e3, 1)
            row[name + "_frac_of_hbm_peak"] = round(nbytes / (ms * 1e-3) / 8e12, 3)
        row["max_abs_diff_between_the_two"] = float((outs[0] - outs[1]).abs().max())
        print(json.dumps(row), flush=True)
        del quant, v, kres, q, outs
        torch.cuda.empty_cache()


if __name__ == "__main__":
    main()
