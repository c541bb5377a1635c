"""Where a wavefront of the one-wavefront-per-slice decode-attention kernel (PQ_SINGLE_WAVEFRONT, and the form the
kernels for 4-bit values have) spends its time, phase by phase: the measurement that led to the scorer / accumulator
pairs of the default kernels, whose two wavefronts overlap what is added up here.

Needs the measuring build of the library (`python -m polarquant_amd.build --phase-timers`), whose attention
kernel brackets its phases with the 100 MHz wall clock and lets every 97th wavefront print its sums.  The
instrumentation costs a few percent, so totals are a little above the real kernel's; the split is what matters.

    python -m polarquant_amd.benchmarks.phase_timing [--config 1 | --shape B,N,Nk,L] [--values4] [--pairs] [--pieces]

Phases of one 128-token group: table = build of the per-group angle table in LDS; value_issue = issue of the
next tile's value loads (16 buffer loads; the time is spent in the issue itself when the compute unit's miss
queue is full); code_wait = arrival of this tile's codes; code_issue = issue of the next tile's code loads;
score = the 64-code table walk; softmax_pv = mask, softmax update and the P.V MFMAs (including the arrival of
the value tile requested a tile earlier).
"""
from __future__ import annotations

import argparse
import json
import os
import re
import sys
import tempfile

import torch

from .. import _ffi
from ..build import TIMERS_LIB

PHASES = ("table", "value_issue", "code_wait", "code_issue", "score", "softmax_pv")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--config", type=int, default=1)
    ap.add_argument("--shape", type=str, default=None, help="B,N,Nk,L: a uniform batch of this shape (4/4 bits, float16, random keys "
                    "quantized on the GPU, one residual key) instead of a benchmark configuration")
    ap.add_argument("--values4", action="store_true")
    ap.add_argument("--even", action="store_true", help="ragged batches: even slices per sequence instead of balanced slices")
    ap.add_argument("--pairs", action="store_true", help="the default kernels instead (a scorer / accumulator pair of wavefronts per slice): "
                    "how long each role waits for the other")
    ap.add_argument("--pieces", action="store_true", help="also list every reporting piece: block, groups, us from the first entry to its entry and exit")
    args = ap.parse_args()
    if not os.path.exists(TIMERS_LIB):
        sys.exit("phase_timing: build the measuring library first: python -m polarquant_amd.build --phase-timers")
    _ffi.LIB_PATH = TIMERS_LIB
    from .. import workloads as wl
    from ..attention import polar_decode_attention, polar_decode_attention_v4
    from ..values import quantize_values
    dev = torch.device("cuda:0")
    if args.shape:
        from ..quantize import quantize_and_pack_nbit
        B, N, Nk, L = (int(x) for x in args.shape.split(","))
        g = torch.Generator(device=dev).manual_seed(5)
        quant = quantize_and_pack_nbit(torch.randn(B, Nk, L, 128, generator=g, device=dev).half(), 4, 4)
        w = dict(q=torch.randn(B, N, 1, 128, generator=g, device=dev).half(), codes=quant[0], meta=list(quant[1:]),
                 kres=torch.randn(B, Nk, 128, 128, generator=g, device=dev).half(),
                 v=torch.randn(B, Nk, L + 1, 128, generator=g, device=dev).half(), n_groups=L // 128, n_resid=1)
        kw = dict(rbits=4, tbits=4)
        args.config = args.shape
    else:
        w = wl.build_workload(args.config, dev)
        sh = w["shape"]
        kw = dict(rbits=sh.rbits, tbits=sh.tbits)
    if w.get("groups_per_seq") is not None:
        kw.update(n_groups_per_seq=w["groups_per_seq"], n_resid_per_seq=w["resid_per_seq"], total_groups=int(w["groups_per_seq"].sum()),
                  balanced=not args.even)
    if args.values4:
        L = w["n_groups"] * 128
        vq = quantize_values(w["v"][:, :, :L])
        vres = torch.zeros(w["v"].shape[0], w["v"].shape[1], 128, 128, dtype=w["v"].dtype, device=dev)
        vres[:, :, :1] = w["v"][:, :, L:L + 1]
        kw.pop("total_groups", None)
        kw.pop("balanced", None)
        call = lambda: polar_decode_attention_v4(w["q"], w["codes"], *w["meta"], w["kres"], vres, *vq, w["n_groups"], w["n_resid"], **kw)
    else:
        call = lambda: polar_decode_attention(w["q"], w["codes"], *w["meta"], w["kres"], w["v"], w["n_groups"], w["n_resid"],
                                              single_wavefront=not args.pairs, **kw)
    torch.cuda.synchronize()
    sys.stdout.flush()
    # the kernel prints from the device: collect the process's stdout of one launch in a file
    with tempfile.TemporaryFile(mode="w+b") as tmp:
        saved = os.dup(1)
        os.dup2(tmp.fileno(), 1)
        try:
            call()
            torch.cuda.synchronize()
        finally:
            os.dup2(saved, 1)
            os.close(saved)
        tmp.seek(0)
        text = tmp.read().decode(errors="replace")
    if args.pairs:
        roles = {0: [], 1: []}
        for line in text.splitlines():
            m = re.match(r"pq_pair block (\d+) wave (\d+) role (\d+) tiles (\d+) entry (\d+) first (\d+) last (\d+) exit (\d+) waited (\d+) marks (\d+) (\d+) (\d+)", line)
            if m and int(m.group(4)) > 0:
                roles[int(m.group(3))].append(tuple(int(x) for x in m.groups()[3:]))       # tiles, entry, first, last, exit, waited, marks 0..2
        if not roles[0] or not roles[1]:
            sys.exit("phase_timing: no pair reported (is this the measuring build?)")
        origin = min(v[1] for r in roles.values() for v in r)
        end = max(v[4] for r in roles.values() for v in r)
        out = {"config": args.config, "kernels": "scorer / accumulator pairs",
               "first_entry_to_last_exit_us": round((end - origin) * 0.01, 2)}
        mean = lambda xs: sum(xs) / len(xs)
        for r, name in ((0, "scorer"), (1, "accumulator")):
            v = roles[r]
            many = [x for x in v if x[0] > 1]
            out[name] = {"wavefronts_reporting": len(v), "tiles": round(mean([x[0] for x in v]), 1),
                         "life_us": round(mean([x[4] - x[1] for x in v]) * 0.01, 2),
                         "entry_after_the_first_entry_us": round(mean([x[1] - origin for x in v]) * 0.01, 2),
                         "entry_to_first_tile_handed_over_us": round(mean([x[2] - x[1] for x in v]) * 0.01, 2),
                         "us_per_tile_between_first_and_last_hand_over": round(mean([(x[3] - x[2]) / (x[0] - 1) for x in many]) * 0.01, 3) if many else None,
                         "last_hand_over_to_exit_us": round(mean([x[4] - x[3] for x in v]) * 0.01, 2),
                         "waiting_for_the_partner_us": round(mean([x[5] for x in v]) * 0.01, 2),
                         "waiting_share": round(sum(x[5] for x in v) / sum(x[4] - x[1] for x in v), 3),
                         "entry_to_role_known_us": round(mean([x[6] - x[1] for x in v]) * 0.01, 2)}
            if r == 0:
                out[name]["entry_to_first_loads_arrived_us"] = round(mean([x[7] - x[1] for x in v if x[7]]) * 0.01, 2)
                out[name]["entry_to_first_table_built_us"] = round(mean([x[8] - x[1] for x in v if x[8]]) * 0.01, 2)
        print(json.dumps(out))
        return
    rows = []
    for line in text.splitlines():
        m = re.match(r"pq_phase block (\d+) groups (\d+) total (\d+) " + " ".join(p + r" (\d+)" for p in PHASES), line)
        if m:
            rows.append([int(v) for v in m.groups()])
    pieces = []
    for line in text.splitlines():
        m = re.match(r"pq_piece block (\d+) groups (\d+) entry (\d+) exit (\d+) before_loop (\d+) first_group (\d+) loop (\d+) after_loop (\d+)", line)
        if m:
            pieces.append([int(v) for v in m.groups()])
    rows = [r for r in rows if r[1] > 0]
    if not rows:
        sys.exit("phase_timing: no wavefront reported (is this the measuring build?)")
    groups = sum(r[1] for r in rows)
    per_group = {"total": sum(r[2] for r in rows) / groups * 0.01}
    for i, p in enumerate(PHASES):
        per_group[p] = sum(r[3 + i] for r in rows) / groups * 0.01
    per_group["other"] = per_group["total"] - sum(per_group[p] for p in PHASES)
    out = {"config": args.config, "values4": bool(args.values4), "wavefronts_reporting": len(rows),
           "groups_per_wavefront": round(groups / len(rows), 2),
           "us_per_group": {k: round(v, 3) for k, v in per_group.items()}}
    with_loop = [r for r in pieces if r[1] > 0]
    if with_loop:
        # the life of a piece outside its steady state (clock ticks of 10 ns -> us)
        n = len(with_loop)
        mean = lambda i: sum(r[i] for r in with_loop) / n * 0.01
        # absolute clocks: only a block's first piece (a later piece of the same wavefront starts after the print)
        seen, firsts = set(), []
        for r in pieces:
            if r[0] not in seen:
                seen.add(r[0])
                firsts.append(r)
        first = min(r[2] for r in firsts)
        out["piece_us"] = {
            "pieces_reporting": n,
            "entry_to_loop (addresses, first loads issued, residual keys if they come first)": round(mean(4), 2),
            "first_group (waits for the query, the first metadata and codes)": round(mean(5), 2),
            "loop": round(mean(6), 2),
            "loop_to_exit (4-bit values' rescale, residual keys if they come last, partial written)": round(mean(7), 2),
            "entry_spread_over_wavefronts": round((max(r[2] for r in firsts) - first) * 0.01, 2),
            "first_entry_to_exit_of_first_pieces_min_mean_max": [round((min(r[3] for r in firsts) - first) * 0.01, 2),
                                                                 round((sum(r[3] for r in firsts) / len(firsts) - first) * 0.01, 2),
                                                                 round((max(r[3] for r in firsts) - first) * 0.01, 2)],
        }
        if args.pieces:
            out["pieces (block, groups, entry us, exit us)"] = [[r[0], r[1], round((r[2] - first) * 0.01, 2), round((r[3] - first) * 0.01, 2)]
                                                                for r in pieces]
    print(json.dumps(out))


if __name__ == "__main__":
    main()
