"""Polar quantizer: HIP counterpart of `quantize_and_pack_nbit`
(reference: models/modeling_llama_polar.py:135-157)."""
from __future__ import annotations

import ctypes
from typing import Optional, Tuple

import torch

from . import _ffi
from .kernel4group import _dtype_code, _stream_ptr

GROUP = 128
PAIRS = 64


def quantize_and_pack_nbit(key_states: torch.Tensor, rbits: int = 4, tbits: int = 4, group_size: int = GROUP,
                           wrap_fp32: bool = False, angle_mode: str = "group", packed: bool = False,
                           out: Optional[Tuple[torch.Tensor, ...]] = None, group_offset: int = 0,
                           device_atan2: bool = False, eager_gpu: bool = False):
    """key_states [B,Nk,L,128] half/bf16 on the GPU (any batch/head/token strides, unit dim stride)
    -> (indices u8 [B,Nk,Nb,128,64], rscale, rmn, tscale, tmn [B,Nk,Nb,1,64]).

    `out`, if given, is a 5-tuple of pre-allocated cache tensors
    ([B,Nk,cap,128,64] u8 and four [B,Nk,cap,1,64]) that receive the Nb new groups
    at group index `group_offset`; nothing is allocated then.

    `angle_mode="group"` is the reference's binning (2^tbits bins over each group's own angle
    range); `"uniform"` uses fixed bins over [-pi, pi) and writes the constants
    tmn = -pi, tscale = 2*pi/2^tbits into the metadata, so decode is unchanged.

    By default codes and metadata are those of the reference's lines evaluated by eager torch on CPU
    tensors.  `eager_gpu=True` gives those of the same lines evaluated by eager torch on GPU tensors,
    which is where the reference runs them; it differs in two places, selectable one by one:
    `wrap_fp32` (2*pi is added to negative angles in fp32 instead of as the dtype-rounded 6.28125) and
    `device_atan2` (the GPU math library's atan2f instead of SLEEF's).

    `packed=True` (rbits + tbits <= 6) stores the 64 codes of a token as 48 bytes of packed 6-bit
    codes ([B,Nk,Nb,128,48]) instead of one byte each; the decode entry points recognise the shape.
    """
    assert angle_mode in ("group", "uniform")
    assert not packed or rbits + tbits <= 6, "packed 6-bit codes need rbits + tbits <= 6"
    row = 48 if packed else PAIRS
    if not key_states.is_cuda:
        raise RuntimeError("polarquant_amd: the quantizer needs tensors on the GPU (no CPU fallback)")
    B, Nk, L, D2 = key_states.shape
    assert D2 == 2 * PAIRS and group_size == GROUP, "head_dim 128 and group size 128 only"
    assert L % GROUP == 0 and rbits + tbits <= 8
    Nb = L // GROUP
    dt = _dtype_code(key_states)
    if key_states.stride(3) != 1 or any(s % 4 for s in key_states.stride()[:3]) or key_states.data_ptr() % 8:
        key_states = key_states.contiguous()
    dev = key_states.device
    if out is None:
        codes = torch.empty((B, Nk, Nb, GROUP, row), dtype=torch.uint8, device=dev)
        meta = [torch.empty((B, Nk, Nb, 1, PAIRS), dtype=key_states.dtype, device=dev) for _ in range(4)]
        cap, off = Nb, 0
    else:
        codes, meta = out[0], list(out[1:])
        cap, off = codes.shape[2], group_offset
        assert codes.is_contiguous() and all(m.is_contiguous() for m in meta) and codes.shape[-1] == row
    strides = (ctypes.c_int64 * 4)(*key_states.stride())
    with torch.cuda.device(dev):
        rc = _ffi.lib().pq_quantize_groups(key_states.data_ptr(), ctypes.cast(strides, ctypes.c_void_p), dt, B, Nk, Nb,
                                           rbits, tbits, (_ffi.PQ_WRAP_FP32 if wrap_fp32 or eager_gpu else 0)
                                           | (_ffi.PQ_DEVICE_ATAN2 if device_atan2 or eager_gpu else 0)
                                           | (_ffi.PQ_ANGLE_UNIFORM if angle_mode == "uniform" else 0)
                                           | (_ffi.PQ_CODES_PACKED6 if packed else 0),
                                           codes.data_ptr(), *[m.data_ptr() for m in meta], cap, off,
                                           _stream_ptr(dev))
    _ffi.check(rc, "pq_quantize_groups")
    if out is None:
        return (codes, *meta)
    sl = slice(off, off + Nb)
    return (codes[:, :, sl], *[m[:, :, sl] for m in meta])


def convert_codes6(indices: torch.Tensor, pack: bool) -> torch.Tensor:
    """Byte-per-code rows [..., 64] (codes < 64) -> packed 6-bit rows [..., 48] (pack=True), or back."""
    if not indices.is_cuda:
        raise RuntimeError("polarquant_amd: the layout converter needs tensors on the GPU (no CPU fallback)")
    src_row, dst_row = (PAIRS, 48) if pack else (48, PAIRS)
    assert indices.dtype == torch.uint8 and indices.shape[-1] == src_row
    src = indices.contiguous()
    dst = torch.empty(src.shape[:-1] + (dst_row,), dtype=torch.uint8, device=src.device)
    with torch.cuda.device(src.device):
        rc = _ffi.lib().pq_convert_codes6(src.data_ptr(), dst.data_ptr(), src.numel() // src_row, int(pack), _stream_ptr(src.device))
    _ffi.check(rc, "pq_convert_codes6")
    return dst
