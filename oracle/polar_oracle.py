"""CPU oracle for the polar-key decode path.  TEST INFRASTRUCTURE ONLY.

This file restates, with torch-CPU library routines, the algorithm of the
reference's polar-key decode path.  Only tests/, __graft_entry__.smoke() and
bench.py's cpu_baseline leg may import it; the product (polarquant_amd/) never
does.  Every function cites the reference lines it follows.

Pin status (what proves each function is right, beyond retyping a formula;
the checks live in tests/test_oracle_pins.py):

  quantize_and_pack_nbit   pinned: brute-force fp64 quantizer on tiny inputs,
                           closed-form known-answer group (angles on bin
                           centres), min/max-element invariants, error bounds,
                           cross-check against the independent C restatement
                           (oracle/polar_oracle.c, bit for bit, its own restatement
                           of SLEEF's arctangent included).  The reference holds no
                           golden vectors for it.  Its wrap_fp32 switch (the one
                           line eager torch evaluates differently on GPU tensors)
                           is pinned the same way; the remaining difference of a
                           GPU evaluation, the device library's atan2f, cannot be
                           restated on the CPU and is pinned on the GPU against
                           eager torch ops on device tensors
                           (oracle/device_eager.py holds those ops, itself pinned
                           on CPU tensors against this function bit for bit;
                           tests/test_quantize_gpu.py runs them on the GPU).
  dequantize_keys          pinned: closed form on the known-answer group,
                           error bounds |phi-phi^|<=tscale/2, |r-r^|<=rscale/2.
  decode_scores            pinned: textbook q.K^T (torch.matmul) on the
                           dequantized keys, LUT identity |q|cos(phi-psi),
                           pure-python brute force on one group, C cross-check.
  decode_attention         pinned: composition of torch.matmul/softmax library
                           routines; cross-checked against a one-shot softmax
                           over the concatenated dequantized+residual keys.
  residual_score_rounding_band
                           (a tolerance aid, no reference counterpart: how far the
                           reference's own rounding of the window's scores, :79,
                           can move the output) pinned: it covers the movement
                           measured when those scores are actually rounded, and
                           that movement reaches a fair fraction of it.
  prefill_cache/decode_step pinned: shape/bookkeeping property tests (quantized
                           token count, residual length, kv_seq_len).
  quantize_values_along_last_dim / dequantize_values / decode_attention_mixed
                           (4-bit values of the reference's Mixed variant):
                           the routines the reference calls live in a kivi_quant
                           package that is NOT in its tree and carries no version
                           pin; they are restated from KIVI's published source.
                           Pinned by what the mathematics fixes: closed-form row
                           (codes and packed words known), min->0 / max->2^b-1,
                           |v - v^| <= scale/2, round-half-even, independent C
                           restatement, fp64 one-shot attention over dequantized
                           values.  PARITY UNPINNED: the nibble order inside a
                           packed int32 and the rounding mode are taken from the
                           published KIVI source, which nothing in the reference
                           tree confirms.
  snapkv_scores / snapkv_select / prefill_cache_snapkv (SnapKV prompt eviction in
                           front of the polar cache): compositions of torch library
                           routines (matmul, softmax, avg_pool1d, topk, gather), the
                           literal reference lines; pinned by a hand-built prompt whose
                           heavy keys are known, by permutation invariance of the kept
                           set, and by bookkeeping properties.
  Degenerate groups (tscale==0 or rscale==0 -> 0/0) are undefined behaviour in
  the reference (NaN -> uint8); this oracle defines the code as 0 there, which
  is what torch-CPU's cast yields.  That choice is "parity unpinned".
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch

GROUP_SIZE = 128


# --------------------------------------------------------------------------
# RoPE (HF rotate-half convention, transformers modeling_llama.apply_rotary_pos_emb)
# used only to build synthetic post-RoPE keys.
# --------------------------------------------------------------------------
def rope_cos_sin(positions: torch.Tensor, head_dim: int, theta: float, dtype=torch.float32):
    inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))
    freqs = positions.to(torch.float32)[:, None] * inv_freq[None, :]
    emb = torch.cat([freqs, freqs], dim=-1)
    return emb.cos().to(dtype), emb.sin().to(dtype)


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    h = x.shape[-1] // 2
    return torch.cat([-x[..., h:], x[..., :h]], dim=-1)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """x [..., L, D]; cos/sin [L, D]."""
    return x * cos + rotate_half(x) * sin


# --------------------------------------------------------------------------
# Q: polar quantizer  (models/modeling_llama_polar.py:135-157, identical to
# models/modeling_qwen_polar.py:134-156 and models/kernel4group.py:126-139)
# --------------------------------------------------------------------------
def _to_u8_defined(x: torch.Tensor) -> torch.Tensor:
    """floor(x).to(uint8) with NaN/Inf -> 0 made explicit (torch-CPU behaviour)."""
    x = torch.floor(x)
    x = torch.where(torch.isfinite(x), x, torch.zeros_like(x))
    return x.to(torch.float32).clamp_(0, 255).to(torch.uint8)


def quantize_and_pack_nbit(key_states: torch.Tensor, rbits: int = 4, tbits: int = 4,
                           group_size: int = GROUP_SIZE, angle_mode: str = "group", wrap_fp32: bool = False):
    """key_states [B,Nk,L,2*D] half/bf16 (post-RoPE) ->
    (indices u8 [B,Nk,Nb,G,D], rscale, rmn, tscale, tmn [B,Nk,Nb,1,D] in key dtype).

    Every op runs eagerly in the key dtype, exactly as the reference does
    (modeling_llama_polar.py:141-155): x = dims [0,D), y = dims [D,2D).

    angle_mode="uniform" (no reference counterpart; the fixed-grid special case of the same
    formula): the angle is not wrapped, tmn = -pi and tscale = 2*pi / 2^tbits as key-dtype
    constants, theta by line :148 unchanged.

    wrap_fp32: line :144 as eager torch evaluates it on GPU tensors, where a python scalar added to a
    half tensor stays fp32 (phi is widened, 2*pi added as the fp32 6.2831855, the sum rounded once);
    on CPU tensors, the default here, the scalar is first cast to the tensor dtype (6.28125).
    """
    B, N, L, D2 = key_states.shape
    assert D2 % 2 == 0 and L % group_size == 0 and rbits + tbits <= 8
    D, G = D2 // 2, group_size
    ks = key_states.reshape(B, N, L // G, G, 2, D)

    phi = torch.atan2(ks[:, :, :, :, 1, :], ks[:, :, :, :, 0, :])             # :143
    if angle_mode == "uniform":
        tmn = torch.full_like(phi[..., :1, :], -math.pi)
        tscale = torch.full_like(tmn, 2 * math.pi) / (2 ** tbits)
    else:
        wrapped = (phi.float() + 2 * math.pi).to(phi.dtype) if wrap_fp32 else phi + 2 * math.pi
        phi = torch.where(phi < 0, wrapped, phi)                              # :144
        tmx, tmn = phi.max(-2, keepdim=True)[0], phi.min(-2, keepdim=True)[0]  # :146
        tscale = (tmx - tmn) / (2 ** tbits)                                   # :147
    theta = torch.clamp(_to_u8_defined((phi - tmn) / tscale), 0, 2 ** tbits - 1)  # :148

    radii = torch.norm(ks, p=2, dim=-2)                                       # :150
    rmx, rmn = radii.max(-2, keepdim=True)[0], radii.min(-2, keepdim=True)[0]  # :151
    rscale = (rmx - rmn) / (2 ** rbits)                                       # :152
    rho = torch.clamp(_to_u8_defined((radii - rmn) / rscale), 0, 2 ** rbits - 1)  # :153

    indices = (rho << tbits) + theta                                          # :155
    return indices, rscale, rmn, tscale, tmn


def quantize_brute_fp64(key_states: torch.Tensor, rbits: int, tbits: int, group_size: int = GROUP_SIZE):
    """Same quantizer in exact-ish fp64 arithmetic with no half rounding of the
    intermediates.  Where it disagrees with quantize_and_pack_nbit the
    disagreement is by definition a rounding "edge flip"."""
    B, N, L, D2 = key_states.shape
    D, G = D2 // 2, group_size
    ks = key_states.to(torch.float64).reshape(B, N, L // G, G, 2, D)
    x, y = ks[..., 0, :], ks[..., 1, :]
    phi = torch.atan2(y, x)
    phi = torch.where(phi < 0, phi + 2 * math.pi, phi)
    tmx, tmn = phi.amax(-2, keepdim=True), phi.amin(-2, keepdim=True)
    tscale = (tmx - tmn) / (2 ** tbits)
    theta = torch.clamp(torch.nan_to_num(torch.floor((phi - tmn) / tscale), nan=0.0, posinf=0.0), 0, 2 ** tbits - 1)
    r = torch.sqrt(x * x + y * y)
    rmx, rmn = r.amax(-2, keepdim=True), r.amin(-2, keepdim=True)
    rscale = (rmx - rmn) / (2 ** rbits)
    rho = torch.clamp(torch.nan_to_num(torch.floor((r - rmn) / rscale), nan=0.0, posinf=0.0), 0, 2 ** rbits - 1)
    idx = (rho.to(torch.int64) << tbits) + theta.to(torch.int64)
    return idx.to(torch.uint8), rscale, rmn, tscale, tmn


# --------------------------------------------------------------------------
# Packed 6-bit code rows.  The reference stores one byte per pair code for every
# bit width and announces a sub-byte store as future work (models/kernel4group.py:1-3);
# the build's optional packed layout is defined here independently of the kernels:
# the 64 codes of a token (each < 64) as 384 consecutive bits, code i in bits [6i, 6i+6)
# of the 48-byte row, little-endian.
# --------------------------------------------------------------------------
def pack_codes6(indices: torch.Tensor) -> torch.Tensor:
    """u8 [..., 64] (values < 64) -> u8 [..., 48]."""
    assert indices.dtype == torch.uint8 and indices.shape[-1] == 64 and int(indices.max()) < 64
    c = indices.to(torch.int64).reshape(*indices.shape[:-1], 16, 4)
    x = c[..., 0] | (c[..., 1] << 6) | (c[..., 2] << 12) | (c[..., 3] << 18)            # 24 bits per 4 codes
    b = torch.stack([x & 0xFF, (x >> 8) & 0xFF, (x >> 16) & 0xFF], dim=-1)              # 3 bytes, little-endian
    return b.reshape(*indices.shape[:-1], 48).to(torch.uint8)


def unpack_codes6(packed: torch.Tensor) -> torch.Tensor:
    """u8 [..., 48] -> u8 [..., 64]."""
    assert packed.dtype == torch.uint8 and packed.shape[-1] == 48
    b = packed.to(torch.int64).reshape(*packed.shape[:-1], 16, 3)
    x = b[..., 0] | (b[..., 1] << 8) | (b[..., 2] << 16)
    c = torch.stack([x & 0x3F, (x >> 6) & 0x3F, (x >> 12) & 0x3F, (x >> 18) & 0x3F], dim=-1)
    return c.reshape(*packed.shape[:-1], 64).to(torch.uint8)


# --------------------------------------------------------------------------
# dequantize (models/kernel4group.py:151-153; fp32 bin centres as the Triton
# kernel evaluates them, kernel4group.py:67,73)
# --------------------------------------------------------------------------
def dequantize_keys(indices, rscale, rmn, tscale, tmn, rbits: int = 4, tbits: int = 4,
                    dtype=torch.float32) -> torch.Tensor:
    """-> K^ [B,Nk,Nb*G,2*D] in `dtype` (fp32 or fp64): (r^ cos phi^ || r^ sin phi^)."""
    B, Nk, Nb, G, D = indices.shape
    theta = (indices & (2 ** tbits - 1)).to(dtype)
    rho = (indices >> tbits).to(dtype)
    phi = tscale.to(dtype) * (theta + 0.5) + tmn.to(dtype)
    rad = rscale.to(dtype) * (rho + 0.5) + rmn.to(dtype)
    k = torch.stack([rad * torch.cos(phi), rad * torch.sin(phi)], dim=-2)  # [B,Nk,Nb,G,2,D]
    return k.reshape(B, Nk, Nb * G, 2 * D)


def repeat_kv(x: torch.Tensor, n_rep: int) -> torch.Tensor:
    """HF repeat_kv: [B,Nk,L,D] -> [B,Nk*n_rep,L,D], query head h uses kv head h//n_rep."""
    if n_rep == 1:
        return x
    B, Nk, L, D = x.shape
    return x[:, :, None, :, :].expand(B, Nk, n_rep, L, D).reshape(B, Nk * n_rep, L, D)


# --------------------------------------------------------------------------
# S: quantized-key scores (models/kernel4group.py:14-109; oracle formula :151-155)
# --------------------------------------------------------------------------
def decode_scores(query_states, indices, rscale, rmn, tscale, tmn, rbits: int = 4, tbits: int = 4,
                  dtype=torch.float32) -> torch.Tensor:
    """query [B,N,1,2D] -> fp32/fp64 scores [B,N,1,Nb*G] = q . K^^T, no 1/sqrt(d)."""
    B, N = query_states.shape[:2]
    Nk = indices.shape[1]
    khat = dequantize_keys(indices, rscale, rmn, tscale, tmn, rbits, tbits, dtype)
    return torch.matmul(query_states.to(dtype), repeat_kv(khat, N // Nk).transpose(2, 3))


def decode_scores_lut_python(query, indices, rscale, rmn, tscale, tmn, rbits, tbits, b, h, group):
    """Pure-python float64 restatement of one program of the Triton kernel
    (kernel4group.py:64-77): LUT over angle bins, gather, radius, sum over pairs.
    Returns a list of G python floats for query head h, one 128-token group."""
    B, Nk, Nb, G, D = indices.shape
    N = query.shape[1]
    kvh = h // (N // Nk)
    out = []
    q = query[b, h, 0].to(torch.float64).tolist()
    ts = tscale[b, kvh, group, 0].to(torch.float64).tolist()
    tm = tmn[b, kvh, group, 0].to(torch.float64).tolist()
    rs = rscale[b, kvh, group, 0].to(torch.float64).tolist()
    rm = rmn[b, kvh, group, 0].to(torch.float64).tolist()
    idx = indices[b, kvh, group].tolist()
    for g in range(G):
        acc = 0.0
        for d in range(D):
            code = idx[g][d]
            th, rh = code & ((1 << tbits) - 1), code >> tbits
            phi = ts[d] * (th + 0.5) + tm[d]
            rad = rs[d] * (rh + 0.5) + rm[d]
            acc += (q[d] * math.cos(phi) + q[d + D] * math.sin(phi)) * rad
        out.append(acc)
    return out


# --------------------------------------------------------------------------
# R/M/X/V: full decode attention (models/modeling_llama_polar.py:61-101)
# --------------------------------------------------------------------------
def decode_attention(query_states, key_resid, indices, rscale, rmn, tscale, tmn, value_states,
                     attention_mask: Optional[torch.Tensor] = None, rbits: int = 4, tbits: int = 4,
                     score_dtype=torch.float32) -> torch.Tensor:
    """One decode step's attention, AFTER the new key/value have been appended
    to key_resid / value_states (modeling_llama_polar.py:77,98).

    query [B,N,1,128]; key_resid [B,Nk,res,128] (res>=1) or None; quant tensors
    or None; value_states [B,Nk,Lq+res,128]; attention_mask [B,Lq+res] of {0,1}.
    Returns attn_output [B,N,1,128] in query dtype.
    """
    B, N, _, hd = query_states.shape
    Nk = value_states.shape[1]
    rep = N // Nk
    parts = []
    if indices is not None:
        parts.append(decode_scores(query_states, indices, rscale, rmn, tscale, tmn, rbits, tbits,
                                   score_dtype).to(torch.float32))                       # :66-75
    if key_resid is not None and key_resid.shape[2] > 0:
        # the reference multiplies in the model dtype then promotes (:79); the
        # product of two halves summed in fp32 then rounded to half is what a
        # half matmul yields, so do exactly that.
        w = torch.matmul(query_states.float(), repeat_kv(key_resid, rep).float().transpose(2, 3))
        parts.append(w.to(query_states.dtype).to(torch.float32))
    attn = torch.cat(parts, dim=-1) / math.sqrt(hd)                                     # :80
    if attention_mask is not None:
        attn = attn + (1.0 - attention_mask[:, None, None, :].to(torch.float32)) * torch.finfo(torch.float32).min  # :94-95
    p = torch.softmax(attn, dim=-1).to(query_states.dtype)                               # :97
    out = torch.matmul(p.float(), repeat_kv(value_states, rep).float())                  # :99
    return out.to(query_states.dtype)


def decode_attention_exact(query_states, key_resid, indices, rscale, rmn, tscale, tmn, value_states,
                           attention_mask=None, rbits=4, tbits=4) -> torch.Tensor:
    """Same attention in fp64 with no intermediate half rounding; returns fp64
    [B,N,1,128].  Used as the centre of the tolerance band for the HIP kernel."""
    B, N, _, hd = query_states.shape
    Nk = value_states.shape[1]
    rep = N // Nk
    ks = []
    if indices is not None:
        ks.append(dequantize_keys(indices, rscale, rmn, tscale, tmn, rbits, tbits, torch.float64))
    if key_resid is not None and key_resid.shape[2] > 0:
        ks.append(key_resid.to(torch.float64))
    k = torch.cat(ks, dim=2)
    attn = torch.matmul(query_states.to(torch.float64), repeat_kv(k, rep).transpose(2, 3)) / math.sqrt(hd)
    if attention_mask is not None:
        attn = attn.masked_fill(attention_mask[:, None, None, :] == 0, float("-inf"))
    p = torch.softmax(attn, dim=-1)
    return torch.matmul(p, repeat_kv(value_states.to(torch.float64), rep))


def residual_score_rounding_band(query_states, key_resid, indices, rscale, rmn, tscale, tmn, value_states,
                                 attention_mask=None, rbits=4, tbits=4) -> torch.Tensor:
    """How far the output can move, to first order, when each score of the residual window is rounded
    to the model dtype to either neighbour: fp64 [B,N,1,128].

    The reference multiplies q.K^T of the un-quantized keys in the model dtype (:79), so those scores
    carry one rounding of up to half an ulp (0.125 for a bfloat16 score between 32 and 64), and two
    correct evaluations of that line may round a score to different neighbours when their fp32 sums
    differ in the last bits.  With d(out) = sum_i p_i (v_i - out) d(logit_i), the bound is
        sum_{i in window} p_i |v_i - out| ulp(s_i) / 2 / sqrt(head_dim),
    everything evaluated in fp64 as in decode_attention_exact.  `value_states`: the values of all
    attended tokens (for the 4-bit variant: dequantized rows followed by the window's rows)."""
    B, N, _, hd = query_states.shape
    Nk = value_states.shape[1]
    rep = N // Nk
    ks, n_quant = [], 0
    if indices is not None:
        ks.append(dequantize_keys(indices, rscale, rmn, tscale, tmn, rbits, tbits, torch.float64))
        n_quant = ks[0].shape[2]
    if key_resid is None or key_resid.shape[2] == 0:
        return torch.zeros(B, N, 1, hd, dtype=torch.float64)
    ks.append(key_resid.to(torch.float64))
    k = torch.cat(ks, dim=2)
    s = torch.matmul(query_states.to(torch.float64), repeat_kv(k, rep).transpose(2, 3))      # [B,N,1,L], unscaled
    attn = s / math.sqrt(hd)
    if attention_mask is not None:
        attn = attn.masked_fill(attention_mask[:, None, None, :] == 0, float("-inf"))
    p = torch.softmax(attn, dim=-1)
    v = repeat_kv(value_states.to(torch.float64), rep)                                       # [B,N,L,hd]
    out = torch.matmul(p, v)                                                                 # [B,N,1,hd]
    mant = 10 if query_states.dtype == torch.float16 else 7
    half_ulp = torch.exp2(torch.floor(torch.log2(s[..., n_quant:].abs().clamp_min(2.0 ** -14))) - mant - 1)
    w = (p[..., n_quant:] * half_ulp / math.sqrt(hd)).transpose(2, 3)                        # [B,N,R,1]
    return (w * (v[:, :, n_quant:] - out).abs()).sum(dim=2, keepdim=True)


# --------------------------------------------------------------------------
# C/P/F: cache tuple bookkeeping (modeling_llama_polar.py:62,83-92,101,116-128)
# --------------------------------------------------------------------------
def prefill_cache(key_states, value_states, rbits=4, tbits=4, residual_length=GROUP_SIZE):
    """Prompt keys/values [B,Nk,L,128] -> the reference's 8-tuple (:116-128)."""
    L = key_states.shape[2]
    r = L % residual_length
    if r == 0:
        k_full, k_quant = None, key_states
    else:
        k_full = key_states if L < residual_length else key_states[:, :, -r:, :]
        k_quant = None if L < residual_length else key_states[:, :, :-r, :]
    ind = rs = rm = ts = tm = None
    if k_quant is not None:
        ind, rs, rm, ts, tm = quantize_and_pack_nbit(k_quant.contiguous(), rbits, tbits, residual_length)
    return (k_full, ind, rs, rm, ts, tm, value_states, L)


def decode_step(query_states, key_states, value_states, past_key_value, attention_mask=None,
                rbits=4, tbits=4, residual_length=GROUP_SIZE):
    """One decode step on post-RoPE q/k/v [B,H,1,128] (:61-101) -> (attn_output, new tuple)."""
    k_full, ind, rs, rm, ts, tm, v_full, kv_len = past_key_value
    k_full = key_states if k_full is None else torch.cat([k_full, key_states], dim=2)       # :77
    v_full = torch.cat([v_full, value_states], dim=2)                                       # :98
    out = decode_attention(query_states, k_full, ind, rs, rm, ts, tm, v_full, attention_mask, rbits, tbits)
    if k_full.shape[2] % residual_length == 0:                                              # :83
        i2, rs2, rm2, ts2, tm2 = quantize_and_pack_nbit(k_full.contiguous(), rbits, tbits, residual_length)
        cat = lambda a, b: b if a is None else torch.cat([a, b], dim=2)
        ind, rs, rm, ts, tm = cat(ind, i2), cat(rs, rs2), cat(rm, rm2), cat(ts, ts2), cat(tm, tm2)
        k_full = None
    return out, (k_full, ind, rs, rm, ts, tm, v_full, kv_len + 1)


# --------------------------------------------------------------------------
# SnapKV prompt eviction in front of the polar cache (LlamaSnapKVAttention,
# models/modeling_llama_polar.py:295-443).  Decode is the plain polar decode step
# (:343-388, no mask, batch 1); only the prompt pass differs.
# --------------------------------------------------------------------------
def snapkv_scores(query_states, key_states, window_size: int = 128, kernel_size: int = 7):
    """Pooled attention mass the last `window_size` queries put on each earlier key (:398-410)
    -> [B, Nk, L - window_size] in the query dtype.  query [B,N,L,128], key [B,Nk,L,128]."""
    B, N, L, hd = query_states.shape
    Nk = key_states.shape[1]
    rep = N // Nk
    w = torch.matmul(query_states[:, :, -window_size:, :], repeat_kv(key_states, rep).transpose(2, 3))           # :398 (no 1/sqrt(d))
    mask = torch.full((window_size, window_size), torch.finfo(w.dtype).min)
    cond = torch.arange(window_size)
    mask.masked_fill_(cond < (cond + 1).view(window_size, 1), 0)                                                # :399-401
    w[:, :, -window_size:, -window_size:] += mask[None, None].to(w.dtype)                                       # :405
    w = torch.softmax(w, dim=-1, dtype=torch.float32).to(query_states.dtype)                                    # :407
    s = w[:, :, -window_size:, :-window_size].sum(dim=-2)                                                       # :408
    pooled = torch.nn.functional.avg_pool1d(s, kernel_size=kernel_size, padding=kernel_size // 2, stride=1)     # :410
    return pooled.view(B, Nk, rep, -1).mean(dim=2)                                                              # :412


def snapkv_select(query_states, key_states, window_size: int = 128, kernel_size: int = 7,
                  max_capacity_prompt: int = 1024 + 128) -> torch.Tensor:
    """-> indices [B, Nk, max_capacity_prompt - window_size] of the kept earlier tokens (:414)."""
    return snapkv_scores(query_states, key_states, window_size, kernel_size).topk(max_capacity_prompt - window_size, dim=-1).indices


def prefill_cache_snapkv(query_states, key_states, value_states, rbits=4, tbits=4, window_size=128, kernel_size=7,
                         max_capacity_prompt=1024 + 128, residual_length=GROUP_SIZE, indices=None):
    """Prompt q/k/v -> the 8-tuple LlamaSnapKVAttention leaves (:392-441): when the prompt is longer
    than max_capacity_prompt only the selected earlier tokens and the last window are cached, and the
    tuple's last slot still holds the FULL prompt length (positions continue from there).
    `indices` overrides the selection (tests pass the product's own, to compare caches exactly)."""
    L = key_states.shape[2]
    if L > max_capacity_prompt:
        if indices is None:
            indices = snapkv_select(query_states, key_states, window_size, kernel_size, max_capacity_prompt)
        idx = indices.unsqueeze(-1).expand(-1, -1, -1, key_states.shape[-1])
        k_past = key_states[:, :, :-window_size, :].gather(dim=2, index=idx)                                    # :417
        v_past = value_states[:, :, :-window_size, :].gather(dim=2, index=idx)
        key_states = torch.cat([k_past, key_states[:, :, -window_size:, :]], dim=2)                            # :420
        value_states = torch.cat([v_past, value_states[:, :, -window_size:, :]], dim=2)
    kept = key_states.shape[2]
    r = kept % residual_length                                                                                  # :426
    if r == 0:
        k_full, k_quant = None, key_states
    else:
        k_full = key_states if L < residual_length else key_states[:, :, -r:, :]                               # :431 tests the FULL length
        k_quant = None if L < residual_length else key_states[:, :, :-r, :]
    ind = rs = rm = ts = tm = None
    if k_quant is not None:
        ind, rs, rm, ts, tm = quantize_and_pack_nbit(k_quant.contiguous(), rbits, tbits, residual_length)
    return (k_full, ind, rs, rm, ts, tm, value_states, L)


# --------------------------------------------------------------------------
# 4-bit values of the Mixed variant (models/modeling_llama_polar.py:158-292).
# The reference imports triton_quantize_and_pack_along_last_dim and
# cuda_bmm_fA_qB_outer from `.kivi_quant` (modeling_llama_polar.py:18-19), a
# directory that is absent from its tree and has no pinned version.  What
# follows restates the published KIVI routines (github.com/jy-yuan/KIVI,
# quant/new_pack.py: triton_quantize_and_pack_along_last_dim, _pack_along_last_dim;
# quant/matmul.py + csrc: cuda_bmm_fA_qB_outer), anchored on the reference's call
# sites: values [B,Nk,T,128] are quantized per token along the 128 dims with
# group size 128 (:236,:275: one group per token and head), 4 bits (:161).
# --------------------------------------------------------------------------
def quantize_values_along_last_dim(data: torch.Tensor, group_size: int = GROUP_SIZE, bits: int = 4):
    """data [B,Nk,T,D] half/bf16 -> (code int32 [B,Nk,T,D*bits/32], scale [B,Nk,T,D/group], mn [B,Nk,T,D/group]).

    Eager ops in the data dtype, as KIVI does them: scale = (mx - mn) / (2^bits - 1);
    q = round(clamp((x - mn) / scale, 0, 2^bits - 1)) (torch.round: half to even);
    32/bits consecutive codes share an int32, element i in bits [i*bits, (i+1)*bits)."""
    B, nh, T, D = data.shape
    assert D % group_size == 0 and 32 % bits == 0
    ng = D // group_size
    x = data.reshape(B * nh * T, ng, group_size)
    mn, mx = x.min(dim=-1)[0], x.max(dim=-1)[0]
    scale = (mx - mn) / (2 ** bits - 1)
    x = x - mn.unsqueeze(-1)
    x = x / scale.unsqueeze(-1)
    x = x.clamp(0, 2 ** bits - 1).round()
    x = torch.where(torch.isfinite(x), x, torch.zeros_like(x)).to(torch.int32)      # constant row: 0/0 -> code 0 (defined here)
    per = 32 // bits
    x = x.reshape(B * nh * T, D // per, per).to(torch.int64)
    shifts = torch.arange(per, dtype=torch.int64) * bits
    word = (x << shifts).sum(-1)                                                     # disjoint bit fields: sum == or
    word = torch.where(word >= 2 ** 31, word - 2 ** 32, word).to(torch.int32)        # two's complement int32
    return word.view(B, nh, T, D // per), scale.reshape(B, nh, T, ng), mn.reshape(B, nh, T, ng)


def unpack_values(code: torch.Tensor, bits: int = 4) -> torch.Tensor:
    """int32 [..., W] -> integer codes [..., W*32/bits] (int64)."""
    per = 32 // bits
    w = code.to(torch.int64) & 0xFFFFFFFF
    shifts = torch.arange(per, dtype=torch.int64) * bits
    return ((w.unsqueeze(-1) >> shifts) & (2 ** bits - 1)).reshape(*code.shape[:-1], code.shape[-1] * per)


def dequantize_values(code, scale, mn, bits: int = 4, dtype=torch.float32) -> torch.Tensor:
    """-> [B,Nk,T,128]: q * scale + zero, as cuda_bmm_fA_qB_outer forms each weight (group size 128:
    one scale / zero per token and head)."""
    return unpack_values(code, bits).to(dtype) * scale.to(dtype) + mn.to(dtype)


def decode_attention_mixed(query_states, key_resid, indices, rscale, rmn, tscale, tmn,
                           value_resid, value_codes, value_scale, value_mn,
                           attention_mask: Optional[torch.Tensor] = None, rbits: int = 4, tbits: int = 4,
                           vbits: int = 4) -> torch.Tensor:
    """One decode step of LlamaPolarMixedGroupAttention (:185-241), AFTER the new key / value were
    appended to key_resid / value_resid.  value_resid [B,Nk,res,128] (res >= 1), value_codes /
    value_scale / value_mn for the tokens before it, or None."""
    B, N, _, hd = query_states.shape
    Nk = value_resid.shape[1]
    rep = N // Nk
    parts = []
    if indices is not None:
        parts.append(decode_scores(query_states, indices, rscale, rmn, tscale, tmn, rbits, tbits).to(torch.float32))  # :189-199
    w = torch.matmul(query_states.float(), repeat_kv(key_resid, rep).float().transpose(2, 3))                           # :203
    parts.append(w.to(query_states.dtype).to(torch.float32))
    attn = torch.cat(parts, dim=-1) / math.sqrt(hd)                                                                     # :204
    if attention_mask is not None:
        attn = attn + (1.0 - attention_mask[:, None, None, :].to(torch.float32)) * torch.finfo(torch.float32).min       # :219-220
    p = torch.softmax(attn, dim=-1).to(query_states.dtype)                                                               # :222
    vfl = value_resid.shape[2]
    if value_codes is None:
        return torch.matmul(p.float(), repeat_kv(value_resid, rep).float()).to(query_states.dtype)                      # :227
    vhat = dequantize_values(value_codes, value_scale, value_mn, vbits)
    out = torch.matmul(p[..., :-vfl].float(), repeat_kv(vhat, rep)).to(value_scale.dtype)                                # :229-236
    return out + torch.matmul(p[..., -vfl:].float(), repeat_kv(value_resid, rep).float()).to(query_states.dtype)        # :238


def decode_attention_mixed_exact(query_states, key_resid, indices, rscale, rmn, tscale, tmn,
                                 value_resid, value_codes, value_scale, value_mn, attention_mask=None,
                                 rbits=4, tbits=4, vbits=4) -> torch.Tensor:
    """Same step as one fp64 softmax attention over [dequantized ; residual] keys and values."""
    v = value_resid.to(torch.float64)
    if value_codes is not None:
        v = torch.cat([dequantize_values(value_codes, value_scale, value_mn, vbits, torch.float64), v], dim=2)
    return decode_attention_exact(query_states, key_resid, indices, rscale, rmn, tscale, tmn, v, attention_mask, rbits, tbits)


def prefill_cache_mixed(key_states, value_states, rbits=4, tbits=4, vbits=4, residual_length=GROUP_SIZE):
    """Prompt keys/values -> the Mixed variant's 11-tuple (:259-281)."""
    k_full, ind, rs, rm, ts, tm, _, L = prefill_cache(key_states, value_states, rbits, tbits, residual_length)
    r = L % residual_length
    if r == 0:
        v_full, v_quant = None, value_states
    else:
        v_full = value_states if L < residual_length else value_states[:, :, -r:, :]
        v_quant = None if L < residual_length else value_states[:, :, :-r, :]
    vc = vs = vm = None
    if v_quant is not None:
        vc, vs, vm = quantize_values_along_last_dim(v_quant.contiguous(), residual_length, vbits)
    return (k_full, ind, rs, rm, ts, tm, v_full, vc, vs, vm, L)


def decode_step_mixed(query_states, key_states, value_states, past_key_value, attention_mask=None,
                      rbits=4, tbits=4, vbits=4, residual_length=GROUP_SIZE):
    """One Mixed decode step on post-RoPE q/k/v [B,H,1,128] (:185-257) -> (attn_output, new 11-tuple)."""
    k_full, ind, rs, rm, ts, tm, v_full, vc, vs, vm, kv_len = past_key_value
    cat = lambda a, b: b if a is None else torch.cat([a, b], dim=2)
    k_full, v_full = cat(k_full, key_states), cat(v_full, value_states)                     # :201, :223
    out = decode_attention_mixed(query_states, k_full, ind, rs, rm, ts, tm, v_full, vc, vs, vm, attention_mask,
                                 rbits, tbits, vbits)
    if k_full.shape[2] % residual_length == 0:                                              # :207
        q5 = quantize_and_pack_nbit(k_full.contiguous(), rbits, tbits, residual_length)
        ind, rs, rm, ts, tm = [cat(a, b) for a, b in zip((ind, rs, rm, ts, tm), q5)]
        k_full = None
    if v_full.shape[2] % residual_length == 0:                                              # :243
        c2, s2, m2 = quantize_values_along_last_dim(v_full.contiguous(), residual_length, vbits)
        vc, vs, vm = cat(vc, c2), cat(vs, s2), cat(vm, m2)
        v_full = None
    return out, (k_full, ind, rs, rm, ts, tm, v_full, vc, vs, vm, kv_len + 1)


# --------------------------------------------------------------------------
# fp16 un-quantized decode attention: the baseline the reference benchmarks
# against (benchmark/models/modeling_llama_exp.py:39-54)
# --------------------------------------------------------------------------
def fp16_decode_attention(query_states, key_states, value_states, attention_mask=None):
    B, N, _, hd = query_states.shape
    rep = N // key_states.shape[1]
    attn = torch.matmul(query_states.float(), repeat_kv(key_states, rep).float().transpose(2, 3))
    attn = attn.to(query_states.dtype).float() / math.sqrt(hd)
    if attention_mask is not None:
        attn = attn + (1.0 - attention_mask[:, None, None, :].float()) * torch.finfo(torch.float32).min
    p = torch.softmax(attn, dim=-1).to(query_states.dtype)
    return torch.matmul(p.float(), repeat_kv(value_states, rep).float()).to(query_states.dtype)
