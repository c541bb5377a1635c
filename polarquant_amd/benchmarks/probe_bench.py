"""Timing-only probes of the decode-attention kernels: a build of the library in which a part of a kernel is
compiled out (its results are wrong on purpose), timed on a benchmark configuration beside the real kernel.

    python -m polarquant_amd.build --probe no_values
    python -m polarquant_amd.benchmarks.probe_bench --probe no_values [--config 1]

no_values: the 4-bit-value step (pq_decode_attn_v4) without its value path (no value loads, no nibble unpacking, no
matrix products, no zero-point term; codes, tables, scores, mask and the softmax sums remain): the floor the score side
alone sets for that kernel.  Two input sets are rotated, as in bench.py.

    python -m polarquant_amd.build --probe direct_bins
    python -m polarquant_amd.benchmarks.probe_bench --probe direct_bins [--config 3]

direct_bins: the key quantizer (pq_quantize_groups) as another algorithm would start out: fp32 estimates of angle and
radius binned directly, with the test for elements near a bin edge but without the exact route those elements (and the
candidates for each pair's extremes) would then take.  Its codes are wrong near bin edges; the time is the floor of that
algorithm.  The report also counts how many codes differ from the shipping kernel's.
"""
from __future__ import annotations

import argparse
import json
import os
import sys

import torch

from .. import _ffi
from ..build import PROBE_LIB

SHIPPING_LIB = _ffi.LIB_PATH


def _direct_bins(args):
    """Prompt quantization of configs[3]'s keys (two key sets rotated) with whichever library was selected."""
    from .. import workloads as wl
    from ..quantize import quantize_and_pack_nbit
    dev = torch.device("cuda:0")
    cfg = args.config if args.config != 1 else 3
    sets = [wl.build_workload(cfg, dev, keep_keys=True, variant=v) for v in (0, 1)]
    sh = sets[0]["shape"]
    keys = [w["keys"][:, :, :w["n_groups"] * 128] for w in sets]
    outs = [quantize_and_pack_nbit(k, sh.rbits, sh.tbits) for k in keys]
    turn = [0]

    def step():
        i = turn[0] & 1
        turn[0] += 1
        quantize_and_pack_nbit(keys[i], sh.rbits, sh.tbits, out=outs[i])
    ms = wl.time_events(step, args.steps, 10)
    # the same keys through the shipping library, loaded beside whichever one is being timed
    import ctypes
    timed = _ffi.lib()
    ship = ctypes.CDLL(SHIPPING_LIB)
    for name, (res, argtypes) in _ffi.SIGNATURES.items():
        fn = getattr(ship, name)
        fn.restype, fn.argtypes = res, argtypes
    _ffi._LIB = ship
    same = quantize_and_pack_nbit(keys[0], sh.rbits, sh.tbits)[0]
    _ffi._LIB = timed
    torch.cuda.synchronize()
    flips = int((outs[0][0] != same).sum())
    print(json.dumps({"library": "shipping" if args.shipping else "probe direct_bins", "config": cfg,
                      "op": "pq_quantize_groups", "us_per_call": round(ms * 1e3, 2), "input_sets_rotated": 2,
                      "codes_differing_from_the_shipping_kernel's": flips, "codes": int(same.numel())}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--probe", choices=["no_values", "direct_bins"], default="no_values")
    ap.add_argument("--config", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--shipping", action="store_true", help="time the shipping library instead (the figure to compare with)")
    args = ap.parse_args()
    if not args.shipping:
        if not os.path.exists(PROBE_LIB):
            sys.exit("probe_bench: build the probe first: python -m polarquant_amd.build --probe " + args.probe)
        _ffi.LIB_PATH = PROBE_LIB
    from .. import workloads as wl
    if args.probe == "direct_bins":
        return _direct_bins(args)
    from ..attention import polar_decode_attention_v4
    from ..values import quantize_values
    dev = torch.device("cuda:0")
    sets = []
    for variant in (0, 1):
        w = wl.build_workload(args.config, dev, variant=variant)
        L = w["n_groups"] * 128
        vq = quantize_values(w["v"][:, :, :L])
        vres = torch.zeros(w["v"].shape[0], w["v"].shape[1], 128, 128, dtype=w["v"].dtype, device=dev)
        vres[:, :, :w["n_resid"]] = w["v"][:, :, L:L + w["n_resid"]]
        w["v"] = None
        sets.append((w, vq, vres))
    sh = sets[0][0]["shape"]
    turn = [0]

    def step():
        w, vq, vres = sets[turn[0] & 1]
        turn[0] += 1
        polar_decode_attention_v4(w["q"], w["codes"], *w["meta"], w["kres"], vres, *vq, w["n_groups"], w["n_resid"],
                                  rbits=sh.rbits, tbits=sh.tbits)
    ms = wl.time_events(step, args.steps, 10)
    print(json.dumps({"library": "shipping" if args.shipping else "probe " + args.probe, "config": args.config,
                      "op": "pq_decode_attn_v4", "us_per_step": round(ms * 1e3, 2), "input_sets_rotated": 2}))


if __name__ == "__main__":
    main()
