"""The other benchmark configurations on one GPU, same kernels and timing as bench.py
(which carries the headline, configs[1], and calls `measure` here for the rest):

  configs[0]  score op, Llama-2-7B shape (batch 1, 32 heads MHA, context 4096)
  configs[2]  ragged continuous-batch decode attention, Qwen2.5-7B shape (batch 64, GQA 7, 3/3 bits)
  configs[3]  prompt quantization (append) of 131072 keys x 8 KV heads, then one decode step over them

    python -m polarquant_amd.benchmarks.config_bench [--configs 0 2 3] [--values4] [--packed]

Prints one JSON line per measurement: µs per call, algorithmic bytes, GB/s and fraction of the
8 TB/s HBM peak.  --values4 adds the decode step with 4-bit values (Mixed variant) for the
uniform-length configurations.
"""
from __future__ import annotations

import argparse
import json
import time

import torch

from .. import workloads as wl
from ..attention import polar_decode_attention, polar_decode_attention_v4
from ..kernel4group import attention_decode_forward_triton_impl
from ..quantize import quantize_and_pack_nbit
from ..values import quantize_values

HBM_PEAK_GBPS = 8000.0


def _entry(op, ms, nbytes, **extra):
    gbps = nbytes / (ms * 1e-3) / 1e9
    return dict(op=op, us=round(ms * 1e3, 2), algorithmic_bytes=int(nbytes), hbm_gbps=round(gbps, 1),
                frac_of_hbm_peak=round(gbps / HBM_PEAK_GBPS, 4), **extra)


def measure(idx: int, dev, values4: bool = False, steps: int = 100, packed: bool = False, single_wavefront: bool = False,
            n_sets: int = 2, eager_gpu_append: bool = False):
    """Time configs[idx] -> (list of measurement dicts, the workload).  The workload keeps what a caller
    needs to check the timed calls' results against a CPU checker: w["scores"] (configs[0]), w["out"] (decode
    attention output), w["append_out"] (configs[3]: codes and metadata the timed quantizer calls wrote) and
    w["keys"] (configs[0] and configs[3]); all of them belong to input set 0.
    n_sets: independent input sets the timed calls rotate over (configs[2] and [3]; configs[0] always uses 8):
    one set of these configurations is 340-390 MB, not much more than the 256 MB Infinity Cache, so a loop over a
    single set could be served partly from that cache.
    eager_gpu_append (configs[3]): the prompt quantization is timed a second time in PQ_EAGER_GPU mode, the
    arithmetic eager torch applies to the reference's lines on device tensors; its output is kept in
    w["append_out_eager_gpu"]."""
    w = wl.build_workload(idx, dev, keep_keys=(idx in (0, 3)), packed=packed)
    sh = w["shape"]
    B, N, Nk = sh.batch, sh.n_heads, sh.n_kv_heads
    res = []
    if idx == 0:
        # 9 MB of inputs would sit in the 256 MB Infinity Cache: rotate over 8 independent copies
        sets = [(w["q"].clone(), w["codes"].clone(), [m.clone() for m in w["meta"]]) for _ in range(8)]
        turn = [0]

        def score():
            q, c, m = sets[turn[0] & 7]
            turn[0] += 1
            return attention_decode_forward_triton_impl(q, c, *m, rbits=sh.rbits, tbits=sh.tbits)
        ms = wl.time_events(score, 4 * steps, steps)
        # the reference's own protocol (benchmark/benchmark_matmul.py:108-118): synchronize, host clock, call,
        # synchronize, host clock; mean over the calls
        total, calls = 0.0, 1000
        for _ in range(calls):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            score()
            torch.cuda.synchronize()
            total += time.perf_counter() - t0
        nbytes = w["codes"].numel() + 4 * w["meta"][0].numel() * 2 + B * N * sh.context * 4 + w["q"].numel() * 2
        res.append(_entry("scores (pq_decode_scores)", ms, nbytes, us_host_clock_per_synchronized_call=round(total / calls * 1e6, 2),
                          input_sets_rotated=8))
        w["scores"] = attention_decode_forward_triton_impl(w["q"], w["codes"], *w["meta"], rbits=sh.rbits, tbits=sh.tbits)
        return res, w
    n_sets = max(1, n_sets)
    sets = [w] + [wl.build_workload(idx, dev, keep_keys=(idx == 3), packed=packed, variant=i) for i in range(1, n_sets)]
    turn = [0]

    def next_set():
        x = sets[turn[0] % n_sets]
        turn[0] += 1
        return x
    if sh.ragged:
        lens = w["lengths"]
        lq, rs = ((lens // 128) * 128).tolist(), (lens % 128).tolist()
        total_groups = int((lens // 128).sum())
    else:
        lq, rs, total_groups = [w["n_groups"] * 128] * B, [w["n_resid"]] * B, None
    nbytes = wl.algorithmic_bytes(Nk, N, lq, rs, sh.rbits, sh.tbits, code_bytes_per_pair=0.75 if packed else 1.0)
    out = torch.empty(B, N, 1, 128, dtype=w["q"].dtype, device=dev)

    def attend(x=None, o=out):
        x = x or next_set()
        polar_decode_attention(
            x["q"], x["codes"], *x["meta"], x["kres"], x["v"], x["n_groups"], x["n_resid"], rbits=sh.rbits, tbits=sh.tbits,
            n_groups_per_seq=x["groups_per_seq"], n_resid_per_seq=x["resid_per_seq"], total_groups=total_groups, out=o,
            single_wavefront=single_wavefront)
    ms = wl.time_events(attend, steps, 10)
    res.append(_entry("decode attention (pq_decode_attn)" + (", packed 6-bit codes" if packed else "")
                      + (", one wavefront per slice" if single_wavefront else ""), ms, nbytes,
                      tokens=int(sum(lq) + sum(rs)), input_sets_rotated=n_sets))
    attend(w)                                   # leave set 0's result in `out` for the caller's check
    w["out"] = out
    if values4 and not sh.ragged:
        L = w["n_groups"] * 128
        v4 = []
        for x in sets:
            vq = quantize_values(x["v"][:, :, :L])
            vres = torch.zeros(B, Nk, 128, 128, dtype=x["v"].dtype, device=dev)
            vres[:, :, :x["n_resid"]] = x["v"][:, :, L:L + x["n_resid"]]
            v4.append((x, vq, vres))

        def attend4():
            x, vq, vres = v4[turn[0] % n_sets]
            turn[0] += 1
            polar_decode_attention_v4(x["q"], x["codes"], *x["meta"], x["kres"], vres, *vq, x["n_groups"], x["n_resid"],
                                      rbits=sh.rbits, tbits=sh.tbits)
        ms4 = wl.time_events(attend4, steps, 10)
        res.append(_entry("decode attention, 4-bit values (pq_decode_attn_v4)", ms4,
                          wl.algorithmic_bytes(Nk, N, lq, rs, sh.rbits, sh.tbits, value_bits=4), input_sets_rotated=n_sets))

        def quant4():
            x, vq, _ = v4[turn[0] % n_sets]
            turn[0] += 1
            quantize_values(x["v"][:, :, :L], out=vq)
        msq = wl.time_events(quant4, max(steps // 2, 5), 3)
        res.append(_entry("value quantization (pq_quantize_values)", msq, B * Nk * L * (256 + 64 + 4), input_sets_rotated=n_sets))
        del v4
    if idx == 3:
        aouts = [(torch.empty_like(x["codes"]), *[torch.empty_like(m) for m in x["meta"]]) for x in sets]

        def append(eager_gpu=False):
            i = turn[0] % n_sets
            turn[0] += 1
            quantize_and_pack_nbit(sets[i]["keys"], sh.rbits, sh.tbits, out=aouts[i], eager_gpu=eager_gpu)
        k = w["keys"]
        append_bytes = k.numel() * 2 + aouts[0][0].numel() + 4 * aouts[0][1].numel() * 2
        ms = wl.time_events(append, max(steps // 2, 6), 6)
        res.append(_entry("append / prompt quantization (pq_quantize_groups)", ms, append_bytes, input_sets_rotated=n_sets))
        if eager_gpu_append:
            ms = wl.time_events(lambda: append(True), max(steps // 2, 6), 6)
            res.append(_entry("append / prompt quantization, PQ_EAGER_GPU (the reference's lines as eager torch evaluates them on "
                              "device tensors)", ms, append_bytes, input_sets_rotated=n_sets))
            w["append_out_eager_gpu"] = quantize_and_pack_nbit(k, sh.rbits, sh.tbits, eager_gpu=True)
        quantize_and_pack_nbit(k, sh.rbits, sh.tbits, out=aouts[0])       # set 0, default mode, for the caller's check
        w["append_out"] = aouts[0]
    return res, w


def run(idx: int, dev, values4: bool, steps: int, packed: bool = False, single_wavefront: bool = False):
    res, _ = measure(idx, dev, values4, steps, packed, single_wavefront)
    for r in res:
        print(json.dumps(dict(config=idx, **r)), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--configs", type=int, nargs="*", default=[0, 2, 3])
    ap.add_argument("--values4", action="store_true")
    ap.add_argument("--packed", action="store_true", help="also run the 3/3-bit configuration with packed 6-bit code rows")
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--single-wavefront", action="store_true", help="decode attention with one wavefront per slice (PQ_SINGLE_WAVEFRONT) instead of the scorer / accumulator pairs")
    ap.add_argument("--no-ramp", action="store_true", help="no clock ramp before the timed regions (counter-collection runs under the profiler)")
    args = ap.parse_args()
    if args.no_ramp:
        wl.RAMP_SECONDS = 0.0
    dev = torch.device("cuda:0")
    for idx in args.configs:
        run(idx, dev, args.values4, args.steps, single_wavefront=args.single_wavefront)
        torch.cuda.empty_cache()
        if args.packed and wl.CONFIGS[idx].rbits + wl.CONFIGS[idx].tbits <= 6:
            run(idx, dev, False, args.steps, packed=True, single_wavefront=args.single_wavefront)
            torch.cuda.empty_cache()


if __name__ == "__main__":
    main()
