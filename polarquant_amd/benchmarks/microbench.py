"""Score-op micro-benchmark with the reference's protocol and shapes
(benchmark/benchmark_matmul.py:89-153): N = Nk = 32 heads, D = 64 pairs, codes for all 32
heads, random codes and randn metadata, B in {1,2,4,8}, L in {4k..128k}; prints ms per call
of the polar score op next to an fp16 torch.matmul QK^T on the same GPU.

    python -m polarquant_amd.benchmarks.microbench [--iters 50]
"""
from __future__ import annotations

import argparse
import json

import torch

from ..kernel4group import attention_decode_forward_triton_impl

LENGTHS = (4096, 8192, 16384, 32768, 65536, 131072)
BATCHES = (1, 2, 4, 8)


def _time(fn, iters, warmup=5):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(iters):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / iters


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--iters", type=int, default=50)
    args = ap.parse_args()
    dev = torch.device("cuda:0")
    out = {"unit": "ms/call", "lengths": list(LENGTHS), "rows": {}}
    for B in BATCHES:
        row = []
        for L in LENGTHS:
            q = torch.randn(B, 32, 1, 128, dtype=torch.float16, device=dev)
            k = torch.randn(B, 32, L, 128, dtype=torch.float16, device=dev)
            row.append(round(_time(lambda: torch.matmul(q, k.transpose(2, 3)), args.iters), 3))
            del k
        out["rows"]["fp16 matmul B=%d" % B] = row
    for rb, tb in ((4, 4), (3, 3)):
        for B in BATCHES:
            row = []
            for L in LENGTHS:
                Nb = L // 128
                codes = torch.randint(0, 250 if tb == 4 else 64, (B, 32, Nb, 128, 64), dtype=torch.uint8, device=dev)
                meta = [torch.randn(B, 32, Nb, 1, 64, dtype=torch.float16, device=dev) for _ in range(4)]
                q = torch.randn(B, 32, 1, 128, dtype=torch.float16, device=dev)
                row.append(round(_time(lambda: attention_decode_forward_triton_impl(q, codes, *meta, rbits=rb, tbits=tb),
                                       args.iters), 3))
                del codes, meta
            out["rows"]["polar %d/%d B=%d" % (rb, tb, B)] = row
    print(json.dumps(out))


if __name__ == "__main__":
    main()
