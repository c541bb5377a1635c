"""Fused elementwise steps of one decode layer (HIP): RoPE + cache append, residual add + RMS norm,
SiLU * up.  Each replaces a chain of 8-12 eager launches on a [B, 1, hidden] activation
(reference: models/modeling_llama_polar.py:47-59,77,98 and the decoder layer :456-486)."""
from __future__ import annotations

from typing import Optional

import torch

from . import _ffi
from .kernel4group import _dtype_code, _stream_ptr


def _gpu(t: torch.Tensor):
    if not t.is_cuda:
        raise RuntimeError("polarquant_amd: the fused decode ops need tensors on the GPU (no CPU fallback)")


def rope_append(q_lin: torch.Tensor, k_lin: torch.Tensor, v_lin: torch.Tensor, cos_table: torch.Tensor,
                sin_table: torch.Tensor, pos: torch.Tensor, k_dst: torch.Tensor, k_row: torch.Tensor,
                v_dst: torch.Tensor, v_row: torch.Tensor, n_heads: int, n_kv_heads: int) -> torch.Tensor:
    """q_lin [B,1,N*128], k_lin / v_lin [B,1,Nk*128] (projection outputs of the new token; each may be a
    slice along the last dim of one fused projection output: unit element stride, any batch stride);
    cos/sin tables [rows,128]; pos, k_row, v_row: int64 tensors of one element on the device.
    Writes the rotated key into k_dst[:, :, k_row] and the value into v_dst[:, :, v_row]
    ([B,Nk,rows,128] each); returns the rotated query [B,N,1,128]."""
    _gpu(q_lin)
    B = q_lin.shape[0]
    assert q_lin.stride(-1) == 1 and k_lin.stride(-1) == 1 and v_lin.stride(-1) == 1
    assert k_lin.stride(0) == v_lin.stride(0) or B == 1
    assert k_dst.is_contiguous() and v_dst.is_contiguous() and cos_table.is_contiguous() and sin_table.is_contiguous()
    assert pos.dtype == k_row.dtype == v_row.dtype == torch.int64
    assert q_lin.shape[-1] == n_heads * 128 and k_lin.shape[-1] == n_kv_heads * 128 == v_lin.shape[-1] and q_lin.numel() == B * n_heads * 128
    assert k_dst.shape[:2] == (B, n_kv_heads) == v_dst.shape[:2] and k_dst.shape[3] == 128 == v_dst.shape[3]
    q_out = torch.empty((B, n_heads, 1, 128), dtype=q_lin.dtype, device=q_lin.device)
    with torch.cuda.device(q_lin.device):
        rc = _ffi.lib().pq_rope_append(q_lin.data_ptr(), k_lin.data_ptr(), v_lin.data_ptr(), cos_table.data_ptr(),
                                       sin_table.data_ptr(), cos_table.shape[0], pos.data_ptr(), q_out.data_ptr(),
                                       k_dst.data_ptr(), k_dst.shape[2], k_row.data_ptr(), v_dst.data_ptr(), v_dst.shape[2],
                                       v_row.data_ptr(), B, n_heads, n_kv_heads, _dtype_code(q_lin),
                                       q_lin.stride(0), k_lin.stride(0), _stream_ptr(q_lin.device))
    _ffi.check(rc, "pq_rope_append")
    return q_out


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, residual: Optional[torch.Tensor] = None,
            sum_out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """weight * rms_norm(x), or of x + residual (the sum, rounded to the dtype, goes to sum_out,
    which may be x itself)."""
    _gpu(x)
    hidden = x.shape[-1]
    assert x.is_contiguous() and weight.is_contiguous() and weight.dtype == x.dtype and weight.numel() == hidden
    if residual is not None:
        assert residual.is_contiguous() and residual.shape == x.shape and residual.dtype == x.dtype
    if sum_out is not None:
        assert sum_out.is_contiguous() and sum_out.shape == x.shape and sum_out.dtype == x.dtype
    y = torch.empty_like(x)
    with torch.cuda.device(x.device):
        rc = _ffi.lib().pq_rmsnorm(x.data_ptr(), None if residual is None else residual.data_ptr(), weight.data_ptr(),
                                   y.data_ptr(), None if sum_out is None else sum_out.data_ptr(), x.numel() // hidden, hidden,
                                   float(eps), _dtype_code(x), _stream_ptr(x.device))
    _ffi.check(rc, "pq_rmsnorm")
    return y


def silu_mul(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """silu(gate) * up; gate and up [..., cols] with unit element stride and a common row stride (they
    may be the two halves of one fused projection output)."""
    _gpu(gate)
    cols = gate.shape[-1]
    assert gate.shape == up.shape and gate.dtype == up.dtype and gate.stride(-1) == 1 and up.stride(-1) == 1
    rows = gate.numel() // cols
    stride = gate.stride(-2) if gate.dim() > 1 else cols
    assert up.dim() == gate.dim() and (up.dim() == 1 or up.stride(-2) == stride)
    assert gate.dim() <= 2 or all(gate.stride(i) == gate.stride(i + 1) * gate.shape[i + 1] for i in range(gate.dim() - 2)), \
        "rows must be evenly spaced"
    y = torch.empty(gate.shape, dtype=gate.dtype, device=gate.device)
    esz = gate.element_size()
    with torch.cuda.device(gate.device):
        for r0 in range(0, rows, 65535):          # one launch covers at most 65535 rows (a prompt has more)
            n = min(65535, rows - r0)
            rc = _ffi.lib().pq_silu_mul(gate.data_ptr() + r0 * stride * esz, up.data_ptr() + r0 * stride * esz,
                                        y.data_ptr() + r0 * cols * esz, n, cols, stride, _dtype_code(gate),
                                        _stream_ptr(gate.device))
            _ffi.check(rc, "pq_silu_mul")
    return y


def linear_small_m(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
                   up_weight: Optional[torch.Tensor] = None) -> torch.Tensor:
    """`F.linear(x, weight, bias)` for at most 16 rows (x [..., K] with up to 16 leading elements, unit
    element stride, one row stride), streamed through the weight-streaming kernel.  With `up_weight`:
    the gated MLP input `silu(x @ weight.T) * (x @ up_weight.T)` in one launch (no bias)."""
    _gpu(x)
    K = x.shape[-1]
    N = weight.shape[0]
    x2 = x.reshape(-1, K)
    M = x2.shape[0]
    assert weight.is_contiguous() and weight.shape == (N, K) and weight.dtype == x.dtype and x2.stride(1) == 1
    if up_weight is not None:
        assert up_weight.is_contiguous() and up_weight.shape == weight.shape and up_weight.dtype == x.dtype
    if bias is not None:
        assert bias.is_contiguous() and bias.numel() == N and bias.dtype == x.dtype
    y = torch.empty(x.shape[:-1] + (N,), dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        rc = _ffi.lib().pq_linear_small_m(x2.data_ptr(), x2.stride(0) if M > 1 else K, weight.data_ptr(),
                                          None if up_weight is None else up_weight.data_ptr(),
                                          None if bias is None else bias.data_ptr(), y.data_ptr(), N, M, N, K,
                                          _dtype_code(x), _stream_ptr(x.device))
    _ffi.check(rc, "pq_linear_small_m")
    return y


def qkv_rope_append(x: torch.Tensor, w_qkv: torch.Tensor, b_qkv: Optional[torch.Tensor], cos_table: torch.Tensor,
                    sin_table: torch.Tensor, pos: torch.Tensor, k_dst: torch.Tensor, k_row: torch.Tensor,
                    v_dst: torch.Tensor, v_row: torch.Tensor, n_heads: int, n_kv_heads: int) -> torch.Tensor:
    """`linear_small_m(x, w_qkv, b_qkv)` followed by `rope_append(...)` in one launch, bit-identical to the pair:
    x [B <= 8, 1, K]; w_qkv [(N + 2 Nk) * 128, K] (q, k, v heads in that order); returns the rotated query
    [B, N, 1, 128], writes the rotated key into k_dst[:, :, k_row] and the value into v_dst[:, :, v_row]."""
    _gpu(x)
    K = x.shape[-1]
    x2 = x.reshape(-1, K)
    B = x2.shape[0]
    assert w_qkv.is_contiguous() and w_qkv.shape == ((n_heads + 2 * n_kv_heads) * 128, K) and w_qkv.dtype == x.dtype
    assert x2.stride(1) == 1 and (b_qkv is None or (b_qkv.is_contiguous() and b_qkv.numel() == w_qkv.shape[0] and b_qkv.dtype == x.dtype))
    assert k_dst.is_contiguous() and v_dst.is_contiguous() and cos_table.is_contiguous() and sin_table.is_contiguous()
    assert pos.dtype == k_row.dtype == v_row.dtype == torch.int64
    assert k_dst.shape[:2] == (B, n_kv_heads) == v_dst.shape[:2] and k_dst.shape[3] == 128 == v_dst.shape[3]
    q_out = torch.empty((B, n_heads, 1, 128), dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        rc = _ffi.lib().pq_qkv_rope_append(x2.data_ptr(), x2.stride(0) if B > 1 else K, w_qkv.data_ptr(),
                                           None if b_qkv is None else b_qkv.data_ptr(), B, K, _dtype_code(x),
                                           cos_table.data_ptr(), sin_table.data_ptr(), cos_table.shape[0], pos.data_ptr(),
                                           q_out.data_ptr(), k_dst.data_ptr(), k_dst.shape[2], k_row.data_ptr(),
                                           v_dst.data_ptr(), v_dst.shape[2], v_row.data_ptr(), n_heads, n_kv_heads,
                                           _stream_ptr(x.device))
    _ffi.check(rc, "pq_qkv_rope_append")
    return q_out


def rope_qk(q_lin: torch.Tensor, k_lin: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, n_heads: int, n_kv_heads: int):
    """`apply_rotary_pos_emb` on projection outputs in one launch, bit-identical to the eager ops: q_lin [B,L,N*128],
    k_lin [B,L,Nk*128] (unit element stride, uniform token stride), cos / sin [1 or B, L, 128] in the same dtype.
    Returns (q [B,N,L,128], k [B,Nk,L,128]) as transposed views of [B,L,heads,128] tensors, the layout the eager
    `.view(B, L, heads, 128).transpose(1, 2)` followed by the rotation produces."""
    _gpu(q_lin)
    B, L = q_lin.shape[0], q_lin.shape[1]
    assert q_lin.shape[-1] == n_heads * 128 and k_lin.shape[-1] == n_kv_heads * 128 and k_lin.shape[:2] == (B, L)
    assert cos.shape == sin.shape and cos.shape[-2:] == (L, 128) and cos.shape[0] in (1, B) and cos.dtype == q_lin.dtype == k_lin.dtype

    def rows(t):                       # token b * L + l at (b * L + l) * token_stride, unit element stride
        def token_stride(u):
            return u.stride(1) if L > 1 else (u.stride(0) if B > 1 else u.shape[-1])
        if (t.stride(-1) != 1 or (B > 1 and L > 1 and t.stride(0) != L * t.stride(1)) or token_stride(t) % 8 != 0
                or token_stride(t) < t.shape[-1] or t.data_ptr() % 16):
            t = t.contiguous()
        return t, token_stride(t)
    q_lin, qs = rows(q_lin)
    k_lin, ks = rows(k_lin)
    cos, sin = cos.contiguous(), sin.contiguous()
    q_out = torch.empty((B, L, n_heads, 128), dtype=q_lin.dtype, device=q_lin.device)
    k_out = torch.empty((B, L, n_kv_heads, 128), dtype=q_lin.dtype, device=q_lin.device)
    with torch.cuda.device(q_lin.device):
        rc = _ffi.lib().pq_rope_qk(q_lin.data_ptr(), qs, k_lin.data_ptr(), ks, cos.data_ptr(), sin.data_ptr(),
                                   0 if cos.shape[0] == 1 else L * 128, q_out.data_ptr(), k_out.data_ptr(), B, L, n_heads,
                                   n_kv_heads, _dtype_code(q_lin), _stream_ptr(q_lin.device))
    _ffi.check(rc, "pq_rope_qk")
    return q_out.transpose(1, 2), k_out.transpose(1, 2)
