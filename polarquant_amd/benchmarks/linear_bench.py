"""Linear layers of one decode step at Llama-3-8B's shapes (bf16, 8 rows): `pq_linear_small_m` against
`torch.nn.functional.linear` (hipBLASLt), each timed as a captured graph of back-to-back calls over
distinct weight matrices (more than the 256 MB of last-level cache in total), the way the decode step
meets them: every layer has its own weights and nothing is re-read between layers.

    python -m polarquant_amd.benchmarks.linear_bench [--rows 8]
"""
from __future__ import annotations

import argparse
import json

import torch
import torch.nn.functional as F

from ..decode_ops import linear_small_m

SHAPES = (("q|k|v", 6144, 4096, False), ("o_proj", 4096, 4096, False), ("gate, up, silu*up", 14336, 4096, True),
          ("down_proj", 4096, 14336, False))


def _graph_time_us(fn, n_calls: int) -> float:
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for i in range(n_calls):
            fn(i)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for i in range(n_calls):
            fn(i)
    graph.replay()
    torch.cuda.synchronize()
    reps = max(2, 200 // n_calls)
    t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0.record()
    for _ in range(reps):
        graph.replay()
    t1.record()
    torch.cuda.synchronize()
    return t0.elapsed_time(t1) / (reps * n_calls) * 1e3


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--rows", type=int, default=8)
    args = ap.parse_args()
    dev, dt = torch.device("cuda:0"), torch.bfloat16
    for name, n, k, gated in SHAPES:
        mats = 2 if gated else 1
        n_buf = max(2, int(600e6 // (n * k * 2 * mats)) + 1)
        ws = [torch.randn(n, k, device=dev, dtype=dt) * 0.02 for _ in range(n_buf)]
        us = [torch.randn(n, k, device=dev, dtype=dt) * 0.02 for _ in range(n_buf)] if gated else None
        x = torch.randn(args.rows, 1, k, device=dev, dtype=dt)
        if gated:
            lib = _graph_time_us(lambda i: F.silu(F.linear(x, ws[i])) * F.linear(x, us[i]), n_buf)
            own = _graph_time_us(lambda i: linear_small_m(x, ws[i], up_weight=us[i]), n_buf)
        else:
            lib = _graph_time_us(lambda i: F.linear(x, ws[i]), n_buf)
            own = _graph_time_us(lambda i: linear_small_m(x, ws[i]), n_buf)
        nbytes = n * k * 2 * mats
        print(json.dumps({"layer": name, "N": n, "K": k, "rows": args.rows, "weight_bytes": nbytes,
                          "library_us": round(lib, 2), "pq_linear_small_m_us": round(own, 2),
                          "hbm_gbps": round(nbytes / own / 1e3, 1), "frac_of_hbm_peak": round(nbytes / own / 1e3 / 8000.0, 4)}), flush=True)
        del ws, us


if __name__ == "__main__":
    main()
