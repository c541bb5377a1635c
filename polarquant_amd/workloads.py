"""Seeded synthetic workloads for the polar-key decode path.

All tensors are generated on the CPU with a seeded torch.Generator so that a
CPU checker and the GPU kernels see identical bits; callers move them to the
GPU.  Keys follow the benchmark recipe: N(0,1) with 4 of the 128 channels
scaled x8 (outliers), then HF rotate-half RoPE at positions 0..L-1, then cast
to the model dtype.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional

import torch

HEAD_DIM = 128
GROUP = 128


@dataclass
class Shape:
    name: str
    batch: int
    n_heads: int
    n_kv_heads: int
    context: int
    rbits: int
    tbits: int
    rope_theta: float
    seed: int
    ragged: bool = False


# index k == benchmark workload configs[k] (config 4, the end-to-end model, has its own builder)
CONFIGS = [
    Shape("cfg0-llama2-7b-scores-b1-4k", 1, 32, 32, 4096, 4, 4, 1e4, 1000),
    Shape("cfg1-llama3-8b-b16-32k", 16, 32, 8, 32768, 4, 4, 5e5, 1001),
    Shape("cfg2-qwen2.5-7b-ragged-b64", 64, 28, 4, 8192, 3, 3, 1e6, 1002, ragged=True),
    Shape("cfg3-llama3-8b-b1-128k", 1, 32, 8, 131072, 4, 4, 5e5, 1003),
]


def _rope_tables(L: int, theta: float, start: int = 0):
    inv_freq = 1.0 / (theta ** (torch.arange(0, HEAD_DIM, 2, dtype=torch.float32) / HEAD_DIM))
    pos = torch.arange(start, start + L, dtype=torch.float32)
    ang = pos[:, None] * inv_freq[None, :]
    emb = torch.cat([ang, ang], dim=-1)
    return emb.cos(), emb.sin()


def _rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    h = HEAD_DIM // 2
    rot = torch.cat([-x[..., h:], x[..., :h]], dim=-1)
    return x * cos + rot * sin


def make_keys(B: int, Nk: int, L: int, theta: float, gen: torch.Generator, dtype=torch.float16,
              chunk: int = 8192) -> torch.Tensor:
    """Post-RoPE keys [B,Nk,L,128] in `dtype`, with 4 outlier channels x8."""
    outliers = torch.randperm(HEAD_DIM, generator=gen)[:4]
    out = torch.empty(B, Nk, L, HEAD_DIM, dtype=dtype)
    for s in range(0, L, chunk):
        n = min(chunk, L - s)
        k = torch.randn(B, Nk, n, HEAD_DIM, generator=gen, dtype=torch.float32)
        k[..., outliers] *= 8.0
        cos, sin = _rope_tables(n, theta, s)
        out[:, :, s:s + n] = _rope(k, cos, sin).to(dtype)
    return out


def make_half(shape, gen: torch.Generator, dtype=torch.float16, chunk_elems: int = 1 << 26) -> torch.Tensor:
    """N(0,1) tensor in `dtype`, generated in bounded fp32 chunks."""
    out = torch.empty(shape, dtype=dtype)
    flat = out.view(-1)
    for s in range(0, flat.numel(), chunk_elems):
        n = min(chunk_elems, flat.numel() - s)
        flat[s:s + n] = torch.randn(n, generator=gen, dtype=torch.float32).to(dtype)
    return out


def ragged_lengths(B: int, gen: torch.Generator, lo: int = 512, hi: int = 8192) -> torch.Tensor:
    return torch.randint(lo, hi + 1, (B,), generator=gen)


@dataclass
class DecodeInputs:
    shape: Shape
    q: torch.Tensor                 # [B,N,1,128]
    k: torch.Tensor                 # [B,Nk,L,128] post-RoPE keys (context)
    v: torch.Tensor                 # [B,Nk,L,128]
    lengths: Optional[torch.Tensor]  # [B] for ragged shapes


def make_decode_inputs(shape: Shape, dtype=torch.float16, context: Optional[int] = None,
                       batch: Optional[int] = None) -> DecodeInputs:
    """Inputs of one decode step for `shape`; `context`/`batch` override the
    full size (tests use reduced sizes of the same recipe and seed)."""
    g = torch.Generator().manual_seed(shape.seed)
    B = batch or shape.batch
    L = context or shape.context
    k = make_keys(B, shape.n_kv_heads, L, shape.rope_theta, g, dtype)
    q = make_half((B, shape.n_heads, 1, HEAD_DIM), g, dtype)
    v = make_half((B, shape.n_kv_heads, L, HEAD_DIM), g, dtype)
    lengths = None
    if shape.ragged:
        lengths = ragged_lengths(B, g, min(512, L), L)
    return DecodeInputs(shape, q, k, v, lengths)


def algorithmic_bytes(n_kv_heads: int, n_heads: int, quant_tokens: List[int], resid_tokens: List[int],
                      rbits: int = 4, tbits: int = 4, code_bytes_per_pair: float = 1.0, value_bits: int = 16) -> int:
    """HBM bytes one fused decode-attention step must move: one byte per pair
    code (the stored layout), 4 half metadata words per (group, pair), fp16 V
    for every token, fp16 residual keys, plus q in / out.  With value_bits=4 (Mixed
    variant) the values of the quantized tokens are 64 bytes of codes plus a half
    scale and zero-point each; the residual window's values stay fp16."""
    total = 0
    for lq, res in zip(quant_tokens, resid_tokens):
        v_bytes = lq * HEAD_DIM * 2 if value_bits == 16 else lq * (HEAD_DIM * value_bits // 8 + 4)
        total += n_kv_heads * (int(lq * 64 * code_bytes_per_pair) + (lq // GROUP) * 4 * 64 * 2
                               + v_bytes + res * HEAD_DIM * 2 + res * HEAD_DIM * 2)
    total += 2 * len(quant_tokens) * n_heads * HEAD_DIM * 2
    return total


# ----------------------------------------------------------------------------- GPU-resident workloads and timing
def build_workload(idx, dev, dtype=torch.float16, keep_keys=False, packed=False, keep_keys_of=None, variant=0):
    """configs[idx] resident in HBM: polar key cache of L/128 groups per (sequence, KV head),
    fp16 V cache, one new token whose key sits in the fp16 residual buffer.  Ragged shapes
    (configs[2]) carry per-sequence group / residual counts; their caches are sized for the longest.
    keep_keys keeps the half-precision keys of every sequence in w["keys"], keep_keys_of=n those of the
    first n sequences only.  variant > 0: an independent input set of the same shape (other random
    data in other memory, the same per-sequence lengths), for timings that rotate input sets so that no
    call finds its inputs in a cache."""
    from .quantize import quantize_and_pack_nbit

    sh = CONFIGS[idx]
    B, N, Nk, L = sh.batch, sh.n_heads, sh.n_kv_heads, sh.context
    Nb = L // 128
    g = torch.Generator(device=dev).manual_seed(sh.seed + 7919 * variant)
    # packed: 6-bit codes stored 48 bytes per token (needs rbits + tbits <= 6, i.e. configs[2])
    codes = torch.empty(B, Nk, Nb, 128, 48 if packed else 64, dtype=torch.uint8, device=dev)
    meta = [torch.empty(B, Nk, Nb, 1, 64, dtype=dtype, device=dev) for _ in range(4)]
    inv_freq = 1.0 / (sh.rope_theta ** (torch.arange(0, 128, 2, dtype=torch.float32, device=dev) / 128))
    ang = torch.arange(L, dtype=torch.float32, device=dev)[:, None] * inv_freq[None, :]
    cos, sin = torch.cat([ang, ang], -1).cos(), torch.cat([ang, ang], -1).sin()
    outl = torch.randperm(128, generator=g, device=dev)[:4]
    keys = []
    for b in range(B):                      # keys of one sequence at a time
        k = torch.randn(1, Nk, L, 128, generator=g, device=dev, dtype=torch.float32)
        k[..., outl] *= 8.0
        k = (k * cos + torch.cat([-k[..., 64:], k[..., :64]], -1) * sin).to(dtype)
        quantize_and_pack_nbit(k, sh.rbits, sh.tbits, packed=packed, out=(codes[b:b + 1], *[m[b:b + 1] for m in meta]))
        if keep_keys or (keep_keys_of is not None and b < keep_keys_of):
            keys.append(k)
    v = torch.empty(B, Nk, L + 1, 128, dtype=dtype, device=dev)
    for b in range(B):
        v[b] = torch.randn(Nk, L + 1, 128, generator=g, device=dev, dtype=torch.float32).to(dtype)
    q = torch.randn(B, N, 1, 128, generator=g, device=dev, dtype=torch.float32).to(dtype)
    k_new = torch.randn(B, Nk, 1, 128, generator=g, device=dev, dtype=torch.float32).to(dtype)
    kres = torch.zeros(B, Nk, 128, 128, dtype=dtype, device=dev)
    kres[:, :, :1] = k_new
    w = dict(shape=sh, q=q, codes=codes, meta=meta, kres=kres, v=v, n_groups=Nb, n_resid=1, lengths=None,
             groups_per_seq=None, resid_per_seq=None, keys=torch.cat(keys, 0) if keys else None)
    if sh.ragged:
        # per-sequence context lengths, uniform in [512, L]: full groups are quantized, the tail
        # (L % 128 tokens) stays fp16 in the residual buffer, which is filled from the keys' tail
        lens = torch.randint(512, L + 1, (B,), generator=torch.Generator().manual_seed(sh.seed))
        w["lengths"] = lens
        w["groups_per_seq"] = (lens // 128).int().to(dev)
        w["resid_per_seq"] = (lens % 128).int().to(dev)
        w["kres"] = torch.randn(B, Nk, 128, 128, generator=g, device=dev, dtype=torch.float32).to(dtype)
        w["n_groups"], w["n_resid"] = 0, 0
    return w


RAMP_SECONDS = 0.25


def ramp_clocks(fn, seconds: Optional[float] = None) -> int:
    """Run `fn` untimed for `seconds` of wall time.  After an idle stretch (input generation on the host, a CPU
    checker) the GPU sits in a low power state and takes some 30-50 ms of continuous work to reach its
    sustained clocks: a configs[1] step measures 280 -> 240 -> 226 us over its first 150 launches.  Timed
    regions are meant to show the sustained rate of a decode loop, so each one is preceded by this.
    -> number of calls made."""
    import time
    seconds = RAMP_SECONDS if seconds is None else seconds
    n, t0 = 0, time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(10):
            fn()
        n += 10
        torch.cuda.synchronize()
    return n


def time_events(fn, steps, warmup, ramp_seconds: Optional[float] = None):
    """ms per call: clock ramp (untimed), `warmup` untimed calls, then exactly `steps` calls between one pair of
    events on the current stream, with a device synchronisation on both sides."""
    ramp_seconds = RAMP_SECONDS if ramp_seconds is None else ramp_seconds
    if ramp_seconds > 0:
        ramp_clocks(fn, ramp_seconds)
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps      # ms per call
