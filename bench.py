#!/usr/bin/env python3
"""Headline benchmark: fused polar decode attention, Llama-3-8B shape, batch 16, 32k context.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One "step" is one pass of the hot path over one batch: the fused decode
attention of one layer (quantized-key scores + residual key + softmax + P.V)
for 16 sequences x 32 query heads over 32768 cached tokens (4-bit radius /
4-bit angle codes, fp16 values), inputs resident in HBM.  Prints ONE JSON line.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
METRIC = "polar decode-attn µs/step + HBM GB/s (% of peak); Llama-3-8B shape b16 32k"

# HBM bytes per launch of the dominant kernel at this workload, from two
# `rocprofv3 --pmc` runs (FETCH_SIZE, WRITE_SIZE) scaled by what the same counters
# read for a copy kernel of known size; see profiles/attn_pair_kernel_cfg1_pmc.md.
MEASURED_TRAFFIC_BYTES = int(675343 * 2.0 * 1024 + 2112.58 * 1024)
TRAFFIC_SOURCE = ("constant, not read in this run: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of 2026-11-26 with the attention "
                  "kernel as of the commit 'Table build independent of the table's LDS alignment', re-measured unchanged "
                  "(675 341 / 2 112.55 counts) after the commit 'Device-side cut of balanced slices in 32-bit arithmetic' "
                  "(profiles/attn_pair_kernel_cfg1_pmc.md)")


def build_cfg1(dev, dtype=torch.float16, keep_keys_of=None):
    from polarquant_amd import workloads as wl
    return wl.build_workload(1, dev, dtype, keep_keys_of=keep_keys_of)


def build_workload(idx, dev, dtype=torch.float16, keep_keys=False, packed=False):
    from polarquant_amd import workloads as wl
    return wl.build_workload(idx, dev, dtype, keep_keys, packed)


def time_events(fn, steps, warmup):
    from polarquant_amd import workloads as wl
    return wl.time_events(fn, steps, warmup)


def kernel_duration_ms(launch, steps, warmup=4):
    """Average duration of one launch in a back-to-back series of `steps` launches between one pair
    of events on the launching stream."""
    return time_events(launch, steps, warmup)


def bracketed_step_ms(first, second, steps, warmup=4):
    """A second timed region of `steps` steps in which the step's two launches are issued separately
    (`first`, then `second`: the same kernels, stream and order as the fused call) with an event before,
    between and after them.  -> (ms per step over the region, mean ms of `first`, mean ms of `second`).
    All three come from the same events, so first + second <= step by construction; the gap between a
    step's end and the next step's start belongs to neither kernel."""
    from polarquant_amd import workloads as wl
    wl.ramp_clocks(lambda: (first(), second()))
    for _ in range(warmup):
        first()
        second()
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(steps)]
    torch.cuda.synchronize()
    for a, b, c in evs:
        a.record()
        first()
        b.record()
        second()
        c.record()
    torch.cuda.synchronize()
    k = sum(a.elapsed_time(b) for a, b, _ in evs) / steps
    m = sum(b.elapsed_time(c) for _, b, c in evs) / steps
    return evs[0][0].elapsed_time(evs[-1][2]) / steps, k, m


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(w):
    """The reference path on the host cores: dequantize-then-matmul scores, /sqrt(d),
    fp32 softmax, P.V (oracle restatement of modeling_llama_polar.py:66-99 and
    kernel4group.py:151-155), on every sequence of the batch in turn (a loop over batch
    elements, summed): the median of three runs per sequence."""
    from oracle import polar_oracle as po
    sh = w["shape"]
    threads = torch.get_num_threads()
    per_seq, ref0 = [], None
    for b in range(sh.batch):
        cq = w["q"][b:b + 1].cpu()
        quant = [w["codes"][b:b + 1].cpu()] + [m[b:b + 1].cpu() for m in w["meta"]]
        kres = w["kres"][b:b + 1, :, :w["n_resid"]].cpu()
        v = w["v"][b:b + 1].cpu()
        if b == 0:
            po.decode_attention(cq, kres, *quant, v, None, sh.rbits, sh.tbits)        # warm-up
        times = []
        for _ in range(3):
            t0 = time.perf_counter()
            ref = po.decode_attention(cq, kres, *quant, v, None, sh.rbits, sh.tbits)
            times.append(time.perf_counter() - t0)
        per_seq.append(sorted(times)[1])
        if b == 0:
            ref0 = ref
    return ref0, {
        "value": round(sum(per_seq) * 1e6, 1), "unit": "us/step", "cores": threads, "cpu": cpu_model(), "kind": "port",
        "per_sequence_us_min_max": [round(min(per_seq) * 1e6, 1), round(max(per_seq) * 1e6, 1)],
        "sample": "all %d sequences (8 KV heads x 32768 tokens each), one after the other, median of 3 runs each, summed: the "
                  "torch-CPU restatement of the reference path (dequantize, matmul, softmax, P.V) on all host threads"
                  % sh.batch,
    }


def code_flips(w):
    """Codes and metadata the HIP quantizer wrote for sequence 0 against the CPU restatement of the
    reference's quantizer (modeling_llama_polar.py:135-157) on the same keys: a differing code is a
    bin-edge flip (a rounding or arctangent difference), a differing metadata word a min/max or scale
    that came out in another half-precision value.  Both counts are meant to be 0."""
    from oracle import polar_oracle as po
    sh = w["shape"]
    ref = po.quantize_and_pack_nbit(w["keys"][0:1].cpu(), sh.rbits, sh.tbits)
    got = [w["codes"][0:1].cpu()] + [m[0:1].cpu() for m in w["meta"]]
    return {"codes": ref[0].numel(), "flips": int((ref[0] != got[0]).sum()),
            "metadata_words": sum(m.numel() for m in ref[1:]),
            "metadata_words_differing": sum(int((a.view(torch.int16) != b.view(torch.int16)).sum()) for a, b in zip(ref[1:], got[1:])),
            "sample": "sequence 0 of %d: %d KV heads x %d keys" % (sh.batch, sh.n_kv_heads, sh.context)}


def fp16_baselines(w, steps, warmup):
    """Un-quantized fp16 decode attention on the same GPU: (i) the reference's eager
    path (benchmark/models/modeling_llama_exp.py:42-52: cat + repeat_kv + matmul,
    softmax, matmul), (ii) torch's fused scaled_dot_product_attention, and (iii) the same
    fused kernel driven as a split-K decode: the context cut into S slices that become extra
    heads (views, no copy), the GQA group's queries as the slice's query rows, and the S
    partial outputs combined by their log-sum-exp.  (ii) runs one workgroup per head over the
    whole context, which leaves most of the GPU idle at one query token; (iii) is what a tuned
    fp16 decode built from library kernels reaches here."""
    import torch.nn.functional as F
    sh = w["shape"]
    B, N, Nk, L = sh.batch, sh.n_heads, sh.n_kv_heads, sh.context
    dev = w["q"].device
    g = torch.Generator(device=dev).manual_seed(1)
    kc = torch.empty(B, Nk, L, 128, dtype=torch.float16, device=dev)
    for b in range(B):
        kc[b] = torch.randn(Nk, L, 128, generator=g, device=dev).half()
    vc = w["v"][:, :, :L].contiguous()
    q, kn, vn = w["q"], w["kres"][:, :, :1].contiguous(), w["v"][:, :, L:L + 1].contiguous()
    rep = N // Nk

    def repeat_kv(x):
        b, h, s, d = x.shape
        return x[:, :, None].expand(b, h, rep, s, d).reshape(b, h * rep, s, d)

    def eager():
        k = torch.cat([kc, kn], dim=2)
        v = torch.cat([vc, vn], dim=2)
        a = torch.matmul(q, repeat_kv(k).transpose(2, 3)) / math.sqrt(128)
        a = torch.softmax(a, dim=-1, dtype=torch.float32).to(q.dtype)
        return torch.matmul(a, repeat_kv(v))

    kf, vf = torch.cat([kc, kn], dim=2), torch.cat([vc, vn], dim=2)

    def sdpa():
        return F.scaled_dot_product_attention(q, kf, vf, enable_gqa=True)

    def sdpa_splitk(S):
        k2, v2 = kc.view(B, Nk * S, L // S, 128), vc.view(B, Nk * S, L // S, 128)
        q2 = q.view(B, Nk, 1, rep, 128).expand(B, Nk, S, rep, 128).reshape(B, Nk * S, rep, 128)
        o, lse = torch.ops.aten._scaled_dot_product_flash_attention(q2, k2, v2, 0.0, False, False)[:2]
        wgt = torch.softmax(lse.view(B, Nk, S, rep).float(), dim=2)
        return (o.view(B, Nk, S, rep, 128).float() * wgt[..., None]).sum(2).to(q.dtype).view(B, N, 1, 128)

    out = {}
    try:
        want = F.scaled_dot_product_attention(q, kc, vc, enable_gqa=True).float()
        best = None
        for S in (16, 32, 64):
            if L % S:
                continue
            assert float((sdpa_splitk(S).float() - want).abs().max()) < 1e-3
            us = time_events(lambda: sdpa_splitk(S), steps, warmup) * 1e3
            if best is None or us < best[0]:
                best = (us, S)
        out["fp16_sdpa_splitk_us"], out["fp16_sdpa_splitk_slices"] = round(best[0], 1), best[1]
        del want
    except Exception as e:                      # noqa: BLE001 - report, do not fail the bench
        out["fp16_sdpa_splitk_error"] = str(e)[:200]
    try:
        out["fp16_eager_us"] = round(time_events(eager, max(3, steps // 4), 2) * 1e3, 1)
    except Exception as e:                      # noqa: BLE001 - report, do not fail the bench
        out["fp16_eager_error"] = str(e)[:200]
    try:
        out["fp16_sdpa_us"] = round(time_events(sdpa, steps, warmup) * 1e3, 1)
    except Exception as e:                      # noqa: BLE001
        out["fp16_sdpa_error"] = str(e)[:200]
    return out


def _roof(entry):
    return {"bound": "hbm", "achieved": entry["hbm_gbps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": entry["frac_of_hbm_peak"]}


def _flips(got, ref):
    return {"codes": ref[0].numel(), "flips": int((ref[0] != got[0]).sum()),
            "metadata_words": sum(m.numel() for m in ref[1:]),
            "metadata_words_differing": sum(int((a.view(torch.int16) != b.view(torch.int16)).sum()) for a, b in zip(ref[1:], got[1:]))}


def _attn_parity(got, ref64):
    err = (got.double().reshape(ref64.shape) - ref64).abs()
    return {"max_abs_err": float(err.max()), "within_rtol1e-2_atol1e-3": bool((err <= 1e-3 + 1e-2 * ref64.abs()).all())}


def other_configs(dev, steps):
    """configs[0], [2] and [3] with the same kernels and timing (HIP events around `steps` calls, inputs in
    HBM), each with its algorithmic bytes, fraction of the 8 TB/s peak, and a check of the timed calls' own
    results against the CPU oracle on a sampled plane."""
    from oracle import polar_oracle as po            # the checker, after the timing
    from polarquant_amd.benchmarks import config_bench as cb
    out = {}

    res, w = cb.measure(0, dev, steps=steps)
    sh = w["shape"]
    quant = [w["codes"].cpu()] + [m.cpu() for m in w["meta"]]
    qc = w["q"].cpu()
    ref = po.decode_scores(qc, *quant, sh.rbits, sh.tbits, dtype=torch.float64)
    got = w["scores"].cpu().double()
    adiff = (got - ref).abs()
    rel = (adiff / ref.abs().amax(-1, keepdim=True)).max()
    # element by element: scores that are off by more than 1e-3 of THEIR OWN magnitude (only scores near zero, where the
    # terms of the sum cancel, can be), how large the largest of them is, and the absolute error there
    off = adiff > 1e-3 * ref.abs()
    elementwise = {"scores": ref.numel(), "off_by_more_than_1e-3_of_own_magnitude": int(off.sum()),
                   "largest_abs_score_among_them": float(ref.abs()[off].max()) if bool(off.any()) else 0.0,
                   "largest_abs_err_among_them": float(adiff[off].max()) if bool(off.any()) else 0.0,
                   "row_max_abs_score_median": float(ref.abs().amax(-1).median()),
                   "max_abs_err": float(adiff.max())}
    fl = _flips(quant, po.quantize_and_pack_nbit(w["keys"].cpu(), sh.rbits, sh.tbits))
    # the reference's CPU-runnable case on the host cores: dequantize-then-matmul scores in fp32
    # (models/kernel4group.py:151-155 restated by the oracle), median of 5 runs
    po.decode_scores(qc, *quant, sh.rbits, sh.tbits)
    times = []
    for _ in range(5):
        t0 = time.perf_counter()
        po.decode_scores(qc, *quant, sh.rbits, sh.tbits)
        times.append(time.perf_counter() - t0)
    cpu0 = {"value": round(sorted(times)[2] * 1e6, 1), "unit": "us/call", "cores": torch.get_num_threads(), "cpu": cpu_model(),
            "kind": "port", "sample": "the whole configuration (1 x 32 heads x 4096 tokens), median of 5 runs: the torch-CPU "
                                      "restatement of the reference's dequantize-then-matmul score path"}
    out["cfg0_scores"] = dict(res[0], workload="configs[0]: score op, batch 1, 32 heads (MHA), context 4096, 4/4 bits",
                              roofline=_roof(res[0]), cpu_baseline=cpu0,
                              parity={"scores_max_err_rel_to_row_max_vs_fp64_oracle": float(rel), "within_1e-3": bool(rel < 1e-3),
                                      "elementwise_vs_fp64_oracle": elementwise,
                                      "quantizer_vs_cpu_oracle": fl, "sample": "all 32 heads x 4096 tokens"})
    del w, quant, ref, got, adiff, off
    torch.cuda.empty_cache()

    res, w = cb.measure(2, dev, steps=steps)
    sh = w["shape"]
    b = int(w["lengths"].argmax())
    L = int(w["lengths"][b]); ng, nr = L // 128, L % 128
    quant = [w["codes"][b:b + 1, :, :ng].cpu()] + [m[b:b + 1, :, :ng].cpu() for m in w["meta"]]
    kres = w["kres"][b:b + 1, :, :nr].cpu() if nr else None
    ref = po.decode_attention_exact(w["q"][b:b + 1].cpu(), kres, *quant, w["v"][b:b + 1, :, :L].cpu(), None, sh.rbits, sh.tbits)
    out["cfg2_decode"] = dict(res[0], workload="configs[2]: ragged decode attention, batch 64, 28 q / 4 KV heads, lengths uniform in "
                                               "[512, 8192], 3/3 bits (one byte per code), fp16 V",
                              roofline=_roof(res[0]),
                              parity=dict(_attn_parity(w["out"][b:b + 1].cpu(), ref), sample="sequence %d (the longest, %d tokens), all 28 heads, vs the fp64 oracle" % (b, L)))
    del w, quant, ref
    torch.cuda.empty_cache()

    res, w = cb.measure(3, dev, steps=steps, eager_gpu_append=True)
    sh = w["shape"]
    quant = [w["codes"][:, :1].cpu()] + [m[:, :1].cpu() for m in w["meta"]]
    rep = sh.n_heads // sh.n_kv_heads
    ref = po.decode_attention_exact(w["q"][:, :rep].cpu(), w["kres"][:, :1, :w["n_resid"]].cpu(), *quant, w["v"][:, :1].cpu(), None, sh.rbits, sh.tbits)
    out["cfg3_decode"] = dict(res[0], workload="configs[3]: decode attention, batch 1, context 131072, 32 q / 8 KV heads, 4/4 bits, split over the context",
                              roofline=_roof(res[0]),
                              parity=dict(_attn_parity(w["out"][:, :rep].cpu(), ref), sample="KV head 0 (query heads 0-3), all 131072 tokens, vs the fp64 oracle"))
    got = [w["append_out"][0][:, :1].cpu()] + [m[:, :1].cpu() for m in w["append_out"][1:]]
    fl = _flips(got, po.quantize_and_pack_nbit(w["keys"][:, :1].cpu(), sh.rbits, sh.tbits))
    out["cfg3_append"] = dict(res[1], workload="configs[3]: prompt quantization of 131072 fp16 post-RoPE keys x 8 KV heads (read keys, write codes and metadata)",
                              roofline=_roof(res[1]),
                              parity=dict(fl, sample="KV head 0, all 131072 keys, vs the CPU oracle's quantizer"))
    # the same append in PQ_EAGER_GPU mode, against the reference's lines evaluated by eager torch ON THE DEVICE (all 8 KV
    # heads, one at a time to bound the temporaries); and the default mode's distance from that evaluation, for the record
    from oracle.device_eager import quantize_and_pack_nbit_eager
    fe = {"codes": 0, "flips": 0, "metadata_words": 0, "metadata_words_differing": 0}
    fd = dict(fe)
    for h in range(sh.n_kv_heads):
        dref = [t.cpu() for t in quantize_and_pack_nbit_eager(w["keys"][:, h:h + 1].contiguous(), sh.rbits, sh.tbits)]
        for acc, src in ((fe, w["append_out_eager_gpu"]), (fd, w["append_out"])):
            one = _flips([t[:, h:h + 1].cpu() for t in src], dref)
            for key in acc:
                acc[key] += one[key]
    out["cfg3_append_eager_gpu"] = dict(res[2], workload="configs[3]'s prompt quantization in PQ_EAGER_GPU mode (fp32 wrap, the device "
                                                         "library's atan2f): codes as the reference's lines give them when they run on GPU tensors",
                                        roofline=_roof(res[2]),
                                        parity=dict(fe, sample="all 8 KV heads x 131072 keys, vs the reference's lines as eager torch ops on device tensors",
                                                    default_mode_vs_the_same=fd))
    del w, quant, ref, got
    torch.cuda.empty_cache()

    # configs[4]: the end-to-end greedy decode loop (random-init Llama-3-8B architecture, bf16, all 32 layers, batch 8,
    # prompt 16384, 256 new tokens), the step replayed from a HIP graph; a 2-layer run of the same loop splits the step
    # into its per-layer part and the embedding / lm_head part.  Sanity of the timed run itself: its first 8 greedy steps
    # against the eager model.  Beside it the un-quantized model (same shells and graph, bf16 K and V caches), as the
    # reference's throughput script has it (benchmark/benchmark_throughput.py:93-113).
    try:
        from polarquant_amd.benchmarks import e2e_bench
        r32 = e2e_bench.run(batch=8, prompt=16384, new=256, layers=32, graph=True, check_tokens=8)
        torch.cuda.empty_cache()
        r2 = e2e_bench.run(batch=8, prompt=16384, new=66, layers=2, graph=True)
        per_layer = (r32["decode_ms_per_step"] - r2["decode_ms_per_step"]) / 30
        out["cfg4_e2e"] = {
            "workload": r32["workload"], "layers": 32,
            "prefill_s": r32["prefill_s"], "decode_ms_per_step": r32["decode_ms_per_step"],
            "decode_tokens_per_s": r32["decode_tokens_per_s"],
            "decode_ms_per_layer": round(per_layer, 4),
            "decode_ms_embedding_and_lm_head": round(r32["decode_ms_per_step"] - 32 * per_layer, 4),
            "kv_cache_bytes_per_token": r32["kv_cache_bytes_per_token"],
            "fp16_kv_cache_bytes_per_token": r32["fp16_kv_cache_bytes_per_token"],
            "peak_memory_GiB": r32["peak_memory_GiB"],
            "sanity": r32.get("sanity"),
        }
        for mode in ("same_kernel", "sdpa_splitk"):
            torch.cuda.empty_cache()
            try:
                rb = e2e_bench.run(batch=8, prompt=16384, new=256, layers=32, fp16_kv=mode)
                out["cfg4_e2e"]["fp16_kv_" + mode] = {
                    "workload": rb["workload"], "decode_ms_per_step": rb["decode_ms_per_step"],
                    "decode_tokens_per_s": rb["decode_tokens_per_s"], "peak_memory_GiB": rb["peak_memory_GiB"],
                    "polar_speedup": round(rb["decode_ms_per_step"] / r32["decode_ms_per_step"], 3)}
            except Exception as e:              # noqa: BLE001 - report, do not fail the bench
                out["cfg4_e2e"]["fp16_kv_" + mode] = {"error": str(e)[:300]}
    except Exception as e:                      # noqa: BLE001 - report, do not fail the bench
        out["cfg4_e2e"] = {"error": str(e)[:300]}
    torch.cuda.empty_cache()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-baselines", action="store_true", help="skip the CPU and fp16 baselines")
    ap.add_argument("--splits", type=int, default=0, help="override the context split count")
    ap.add_argument("--no-values4", action="store_true", help="skip the 4-bit-value (Mixed variant) measurement")
    ap.add_argument("--no-configs", action="store_true", help="skip configs[0], [2], [3] and [4]")
    ap.add_argument("--no-ramp", action="store_true", help="no clock ramp before the timed regions (counter-collection runs under the profiler)")
    ap.add_argument("--copy-calib", action="store_true",
                    help="also run 3 plain 1 GiB device copies (torch clone): under `rocprofv3 --pmc FETCH_SIZE|WRITE_SIZE` "
                         "their counter values give the scale factor for the attention kernel's")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this path runs on ONE GPU (no sharding, no collectives); --gpus %d is not supported"
              % args.gpus, file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)

    from polarquant_amd import _ffi, workloads as wl
    if args.no_ramp:
        wl.RAMP_SECONDS = 0.0
    from polarquant_amd.attention import plan_splits, polar_decode_attention, workspace_for
    from polarquant_amd.kernel4group import _stream_ptr

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    lib = _ffi.lib()
    # two independent copies of the workload, used alternately: no step can find its inputs in a
    # cache left by the previous one (the Infinity Cache holds 256 MB; one copy is 1.36 GB)
    w = build_cfg1(dev, keep_keys_of=None if args.no_baselines else 1)
    w_alt = build_cfg1(dev)
    sh = w["shape"]
    B, N, Nk = sh.batch, sh.n_heads, sh.n_kv_heads
    n_splits = args.splits or plan_splits(B, Nk, w["n_groups"], dev)
    ws = workspace_for(B, N, n_splits, dev)
    out = torch.empty(B, N, 1, 128, dtype=torch.float16, device=dev)
    sm_scale = 1.0 / math.sqrt(128)

    sets = [w, w_alt]
    turn = [0]

    def step():
        x = sets[turn[0] & 1]
        turn[0] += 1
        polar_decode_attention(x["q"], x["codes"], *x["meta"], x["kres"], x["v"], x["n_groups"], x["n_resid"],
                               rbits=sh.rbits, tbits=sh.tbits, n_splits=n_splits, out=out)

    commons = [[x["q"].data_ptr(), x["codes"].data_ptr(), *[m.data_ptr() for m in x["meta"]], x["codes"].shape[2],
                x["n_groups"], None, x["kres"].data_ptr(), x["kres"].shape[2], x["n_resid"], None,
                x["v"].data_ptr(), x["v"].shape[2], None, 0, sm_scale, B, N, Nk, sh.rbits, sh.tbits, _ffi.PQ_F16,
                n_splits, 0, ws.data_ptr(), ws.numel() * 4, 0] for x in sets]

    def partials_only():
        rc = lib.pq_decode_attn_partials(*commons[turn[0] & 1], None, _stream_ptr(dev))
        turn[0] += 1
        assert rc == 0, rc

    if args.copy_calib:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(3)
        for _ in range(3):
            dst = src.clone()
        torch.cuda.synchronize()
        del src, dst

    def merge_only():
        rc = lib.pq_decode_attn_merge(ws.data_ptr(), ws.numel() * 4, B, N, n_splits, _ffi.PQ_F16, out.data_ptr(), _stream_ptr(dev))
        assert rc == 0, rc

    ms = time_events(step, args.steps, args.warmup)
    ms2, k_ms, m_ms = bracketed_step_ms(partials_only, merge_only, args.steps)

    # what a plain read-once kernel is delivered on this GPU: the V tensors of the two input sets
    # (1 GiB each) streamed alternately, one wavefront per SIMD and two per SIMD, best of the two
    sink = torch.zeros(1, dtype=torch.int32, device=dev)
    stream_gbps = 0.0
    for n_waves in (1024, 2048):
        got = [0]

        def stream_once():
            v = sets[turn[0] & 1]["v"]
            turn[0] += 1
            got[0] = _ffi.bench_lib().pq_stream_read(v.data_ptr(), v.numel() * 2, n_waves, sink.data_ptr(), _stream_ptr(dev))
            assert got[0] > 0
        s_ms = time_events(stream_once, 20, 4)
        stream_gbps = max(stream_gbps, got[0] / (s_ms * 1e-3) / 1e9)

    # the attention kernel's own HBM reads without its arithmetic: same grid, loads, order and prefetch depth
    n_tok = w["n_groups"] * 128
    replica = [0]

    def replica_once():
        x = sets[turn[0] & 1]
        turn[0] += 1
        replica[0] = _ffi.bench_lib().pq_attn_load_replica(x["codes"].data_ptr(), x["v"].data_ptr(), B * Nk, x["codes"].shape[2] * 128,
                                              x["v"].shape[2], n_tok, n_splits, sink.data_ptr(), _stream_ptr(dev))
        assert replica[0] > 0
    replica_once()
    replica_once()
    r_ms = kernel_duration_ms(replica_once, 20)

    # the same step with one wavefront per slice (PQ_SINGLE_WAVEFRONT), the form the kernel had before the
    # scorer / accumulator pairs
    def step_single():
        x = sets[turn[0] & 1]
        turn[0] += 1
        polar_decode_attention(x["q"], x["codes"], *x["meta"], x["kres"], x["v"], x["n_groups"], x["n_resid"],
                               rbits=sh.rbits, tbits=sh.tbits, n_splits=n_splits, out=out, single_wavefront=True)
    single_ms = time_events(step_single, 30, 5)

    alg_bytes = wl.algorithmic_bytes(Nk, N, [w["n_groups"] * 128] * B, [w["n_resid"]] * B, sh.rbits, sh.tbits)
    achieved = alg_bytes / (k_ms * 1e-3) / 1e9
    result = {
        "metric": METRIC, "value": round(ms * 1e3, 2), "unit": "us/step", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "clock_ramp_seconds_before_warmup": wl.RAMP_SECONDS, "ms_per_step": round(ms, 5),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "configs[1]: fused polar decode attention, Llama-3-8B shape (32 q heads / 8 KV heads, "
                               "head_dim 128), batch 16, context 32768, 4-bit radius / 4-bit angle, 128-token groups, "
                               "fp16 V, one decode step of one layer",
                   "n_splits": n_splits, "algorithmic_bytes": alg_bytes, "input_sets_rotated": 2},
        "hbm_gbps": round(alg_bytes / (ms * 1e-3) / 1e9, 1),
        "pct_of_hbm_peak": round(100 * alg_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 2),
        "roofline": {"bound": "hbm", "kernel": "attn_pair_kernel<F16,4,4>", "achieved": round(achieved, 1),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "kernel_us": round(k_ms * 1e3, 2), "merge_kernel_us": round(m_ms * 1e3, 2),
                     "step_us_in_the_bracketed_region": round(ms2 * 1e3, 2),
                     "traffic": MEASURED_TRAFFIC_BYTES, "traffic_source": TRAFFIC_SOURCE,
                     "plain_stream_read_gbps": round(stream_gbps, 1),
                     "frac_of_plain_stream_read": round(achieved / stream_gbps, 4),
                     "load_only_replica_us": round(r_ms * 1e3, 2),
                     "load_only_replica_gbps": round(replica[0] / (r_ms * 1e-3) / 1e9, 1)},
        "single_wavefront_us_per_step": round(single_ms * 1e3, 2),
    }
    # the same step with the values of the quantized groups in 4 bits (the reference's Mixed variant)
    if not args.no_values4:
        from polarquant_amd.attention import polar_decode_attention_v4
        from polarquant_amd.values import quantize_values
        L = w["n_groups"] * 128
        v4sets = []
        for x in sets:
            vq = quantize_values(x["v"][:, :, :L])
            vres = torch.zeros(B, Nk, 128, 128, dtype=torch.float16, device=dev)
            vres[:, :, :1] = x["v"][:, :, L:L + 1]
            v4sets.append((vq, vres))
        out4 = torch.empty_like(out)

        def step4():
            i = turn[0] & 1
            x, (vq, vres) = sets[i], v4sets[i]
            turn[0] += 1
            polar_decode_attention_v4(x["q"], x["codes"], *x["meta"], x["kres"], vres, *vq, x["n_groups"], x["n_resid"],
                                      rbits=sh.rbits, tbits=sh.tbits, out=out4)

        ms4 = time_events(step4, args.steps, args.warmup)
        bytes4 = wl.algorithmic_bytes(Nk, N, [L] * B, [w["n_resid"]] * B, sh.rbits, sh.tbits, value_bits=4)
        result["values4"] = {
            "workload": "same step, values of the quantized groups in 4 bits (Mixed variant): 136 B instead of 324 B per token and KV head",
            "us_per_step": round(ms4 * 1e3, 2), "algorithmic_bytes": bytes4,
            "hbm_gbps": round(bytes4 / (ms4 * 1e-3) / 1e9, 1), "frac_of_hbm_peak": round(bytes4 / (ms4 * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
            "speedup_vs_fp16_values": round(ms / ms4, 3),
            "max_abs_diff_vs_fp16_values": float((out4.float() - out.float()).abs().max()),
        }
        del v4sets
    turn[0] = 0
    step()                                   # leave set 0's result in `out` for the parity check
    torch.cuda.synchronize()
    if not args.no_baselines:
        w_alt = None
        del sets[1:]
        torch.cuda.empty_cache()
        ref, cpu = cpu_baseline(w)
        result["cpu_baseline"] = cpu
        result["code_flips_vs_cpu_sample"] = code_flips(w)
        w["keys"] = None
        got = out[0:1].cpu()
        err = (got.double() - ref.double()).abs()
        result["parity_vs_cpu_sample"] = {"max_abs_err": float(err.max()),
                                          "within_rtol1e-2_atol1e-3": bool((err <= 1e-3 + 1e-2 * ref.double().abs()).all())}
        fp = fp16_baselines(w, args.steps, args.warmup)
        result.update(fp)
        for key in ("fp16_eager_us", "fp16_sdpa_us", "fp16_sdpa_splitk_us"):
            if key in fp:
                result["speedup_vs_" + key[:-3]] = round(fp[key] / (ms * 1e3), 2)
        # what no fp16 kernel can beat on this GPU: its K + V + q/out bytes at the rate a plain read-once kernel is delivered
        fp16_bytes = 2 * B * Nk * (sh.context + 1) * 128 * 2 + 2 * B * N * 128 * 2
        result["fp16_stream_bound_us"] = round(fp16_bytes / stream_gbps / 1e3, 1)
        result["speedup_vs_fp16_stream_bound"] = round(result["fp16_stream_bound_us"] / (ms * 1e3), 2)
        if "values4" in result:
            result["values4"]["speedup_vs_fp16_stream_bound"] = round(result["fp16_stream_bound_us"] / result["values4"]["us_per_step"], 2)
            if "fp16_sdpa_splitk_us" in fp:
                result["values4"]["speedup_vs_fp16_sdpa_splitk"] = round(fp["fp16_sdpa_splitk_us"] / result["values4"]["us_per_step"], 2)
    else:
        result["cpu_baseline"] = None
    if not args.no_configs:
        w = w_alt = None
        sets.clear()
        torch.cuda.empty_cache()
        result["configs"] = other_configs(dev, max(args.steps, 20))
    print(json.dumps(result))


if __name__ == "__main__":
    main()
