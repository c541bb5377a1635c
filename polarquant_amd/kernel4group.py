"""Quantized-key decode scores: drop-in for the reference's Triton launcher.

`attention_decode_forward_triton_impl` keeps the reference's name, argument
order, defaults and return value (models/kernel4group.py:83-109) so that the
reference's attention classes can import it from here unchanged; it launches
the hand-written HIP kernel through the C ABI (no Triton involved).
"""
from __future__ import annotations

import torch

from . import _ffi


def _dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.float16:
        return _ffi.PQ_F16
    if t.dtype == torch.bfloat16:
        return _ffi.PQ_BF16
    raise TypeError("polarquant_amd: expected float16 or bfloat16, got %s" % t.dtype)


def _stream_ptr(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def attention_decode_forward_hip_impl(
    query_states: torch.Tensor,   # (b, n, 1, d * 2)
    indices: torch.Tensor,        # (b, nk, nb, g, d) uint8
    rscale: torch.Tensor,         # (b, nk, nb, 1, d)
    rmn: torch.Tensor,            # (b, nk, nb, 1, d)
    tscale: torch.Tensor,         # (b, nk, nb, 1, d)
    tmn: torch.Tensor,            # (b, nk, nb, 1, d)
    rbits: int = 4,
    tbits: int = 4,
) -> torch.Tensor:
    if not query_states.is_cuda:
        raise RuntimeError("polarquant_amd: decode scores need tensors on the GPU (no CPU fallback)")
    B, Nk, Nb, G, D = indices.shape
    N = query_states.shape[1]
    # last dim 64: one byte per pair code (the reference's layout); 48: packed 6-bit codes
    if G != 128 or D not in (64, 48) or query_states.shape[2] != 1 or query_states.shape[3] != 128:
        raise ValueError("polarquant_amd: expected group 128, head_dim 128 and one query token")
    flags = _ffi.PQ_CODES_PACKED6 if D == 48 else 0
    if indices.dtype != torch.uint8:
        raise TypeError("indices must be uint8")
    dt = _dtype_code(query_states)
    meta = [rscale, rmn, tscale, tmn]
    for m in meta:
        if m.dtype != query_states.dtype:
            raise TypeError("metadata dtype must match the query dtype")
    q = query_states.contiguous()
    indices = indices.contiguous()
    meta = [m.contiguous() for m in meta]
    out = torch.empty((B, N, 1, Nb * G), device=q.device, dtype=torch.float32)
    with torch.cuda.device(q.device):
        rc = _ffi.lib().pq_decode_scores(q.data_ptr(), indices.data_ptr(), *[m.data_ptr() for m in meta],
                                         out.data_ptr(), B, N, Nk, Nb, rbits, tbits, dt, flags, _stream_ptr(q.device))
    _ffi.check(rc, "pq_decode_scores")
    return out


# the reference's public name
attention_decode_forward_triton_impl = attention_decode_forward_hip_impl
