"""4-bit value quantizer of the Mixed variant: HIP counterpart of the
`triton_quantize_and_pack_along_last_dim(value_states, 128, 4)` calls in
LlamaPolarMixedGroupAttention (reference: models/modeling_llama_polar.py:236,275)."""
from __future__ import annotations

import ctypes
from typing import Optional, Tuple

import torch

from . import _ffi
from .kernel4group import _dtype_code, _stream_ptr

HEAD_DIM = 128
WORDS = 16          # int32 words per token row: 8 four-bit codes each


def quantize_values(value_states: torch.Tensor, group_size: int = HEAD_DIM, bits: int = 4,
                    out: Optional[Tuple[torch.Tensor, torch.Tensor, torch.Tensor]] = None, token_offset: int = 0):
    """value_states [B,Nk,T,128] half/bf16 on the GPU (any batch/head/token strides, unit dim stride)
    -> (code int32 [B,Nk,T,16], scale [B,Nk,T,1], mn [B,Nk,T,1]).

    `out`, if given, is (code [B,Nk,cap,16], scale [B,Nk,cap,1], mn [B,Nk,cap,1]) pre-allocated
    cache tensors that receive the T rows at token index `token_offset`."""
    if not value_states.is_cuda:
        raise RuntimeError("polarquant_amd: the value quantizer needs tensors on the GPU (no CPU fallback)")
    B, Nk, T, D = value_states.shape
    assert D == HEAD_DIM and group_size == HEAD_DIM and bits == 4, "head_dim 128, one group per row, 4 bits only"
    dt = _dtype_code(value_states)
    if value_states.stride(3) != 1 or any(s % 8 for s in value_states.stride()[:3]) or value_states.data_ptr() % 16:
        value_states = value_states.contiguous()
    dev = value_states.device
    if out is None:
        code = torch.empty((B, Nk, T, WORDS), dtype=torch.int32, device=dev)
        scale = torch.empty((B, Nk, T, 1), dtype=value_states.dtype, device=dev)
        mn = torch.empty((B, Nk, T, 1), dtype=value_states.dtype, device=dev)
        cap, off = T, 0
    else:
        code, scale, mn = out
        cap, off = code.shape[2], token_offset
        assert code.is_contiguous() and scale.is_contiguous() and mn.is_contiguous() and code.dtype == torch.int32
    strides = (ctypes.c_int64 * 4)(*value_states.stride())
    with torch.cuda.device(dev):
        rc = _ffi.lib().pq_quantize_values(value_states.data_ptr(), ctypes.cast(strides, ctypes.c_void_p), dt, B, Nk, T,
                                           code.data_ptr(), scale.data_ptr(), mn.data_ptr(), cap, off, _stream_ptr(dev))
    _ffi.check(rc, "pq_quantize_values")
    if out is None:
        return code, scale, mn
    sl = slice(off, off + T)
    return code[:, :, sl], scale[:, :, sl], mn[:, :, sl]
