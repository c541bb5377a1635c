#!/usr/bin/env python3
"""Writes tests/golden/polar_vectors.npz: seeded inputs and the outputs the CPU oracle gives for
them.  The vectors are made by the oracle (oracle/polar_oracle.py, cross-checked here against the
plain-C restatement), NOT by the reference implementation: the reference ships no vectors and its
modules cannot be imported in this environment.  Their purpose is to freeze today's pinned
behaviour, so that a change of torch version, of the oracle or of a kernel shows up as a diff
against committed data rather than as two things drifting together.

    python tests/golden/make_vectors.py          # rewrites the .npz (deterministic)
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import c_oracle as co            # noqa: E402
from oracle import polar_oracle as po        # noqa: E402
from polarquant_amd import workloads as wl   # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "polar_vectors.npz")
CASES = [  # name, dtype, B, N, Nk, groups, residual keys, rbits, tbits, rope theta, angle mode
    ("llama_f16_44", torch.float16, 1, 8, 2, 2, 5, 4, 4, 5e5, "group"),
    ("qwen_bf16_33", torch.bfloat16, 2, 7, 1, 1, 128, 3, 3, 1e6, "group"),
    ("uniform_f16_44", torch.float16, 1, 4, 4, 1, 0, 4, 4, 1e4, "uniform"),
]


def words(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16) if t.dtype != torch.uint8 else t.numpy()


def main():
    torch.set_num_threads(1)
    data = {}
    for ci, (name, dtype, B, N, Nk, nb, res, rb, tb, theta, mode) in enumerate(CASES):
        g = torch.Generator().manual_seed(7000 + ci)
        L = nb * 128
        keys = wl.make_keys(B, Nk, L + max(res, 1), theta, g, dtype)
        kq, kres = keys[:, :, :L], (keys[:, :, L:L + res] if res else None)
        q = wl.make_half((B, N, 1, 128), g, dtype)
        v = wl.make_half((B, Nk, L + res, 128), g, dtype)
        quant = po.quantize_and_pack_nbit(kq, rb, tb, angle_mode=mode)
        cq = co.quantize(kq, rb, tb, angle_mode=mode)
        assert torch.equal(quant[0], cq[0]) and all(torch.equal(words_t(a), words_t(b)) for a, b in zip(quant[1:], cq[1:])), \
            "the two restatements disagree on case %s: pick another seed" % name
        scores = po.decode_scores(q, *quant, rb, tb)
        mask = None
        if B > 1:
            mask = torch.ones(B, L + res, dtype=torch.uint8)
            mask[1, :37] = 0                                     # left padding on the second sequence
        out = po.decode_attention(q, kres, *quant, v, mask, rb, tb)
        exact = po.decode_attention_exact(q, kres, *quant, v, mask, rb, tb)
        data[name + ".keys"], data[name + ".q"], data[name + ".v"] = words(keys[:, :, :L + res]), words(q), words(v)
        for n, t in zip(("codes", "rscale", "rmn", "tscale", "tmn"), quant):
            data[name + "." + n] = words(t)
        data[name + ".scores_f32"] = scores.numpy()
        data[name + ".attn_out"] = words(out)
        data[name + ".attn_out_f64"] = exact.double().numpy()
        if mask is not None:
            data[name + ".mask"] = mask.numpy()
    np.savez_compressed(OUT, **data)
    print("wrote", OUT, os.path.getsize(OUT), "bytes,", len(data), "arrays")


def words_t(t):
    return t if t.dtype == torch.uint8 else t.contiguous().view(torch.int16)


if __name__ == "__main__":
    main()
