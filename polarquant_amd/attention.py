"""Fused polar-key decode attention (HIP) behind a torch-tensor interface.

`polar_decode_attention` computes what the decode branch of the reference's
LlamaPolarGroupAttention.forward computes between RoPE and o_proj
(models/modeling_llama_polar.py:66-99), in one pass over HBM.
"""
from __future__ import annotations

import math
from typing import Optional

import torch

from . import _ffi
from .kernel4group import _dtype_code, _stream_ptr

GROUP = 128
_WORKSPACES = {}


def _num_cus(device: torch.device) -> int:
    return torch.cuda.get_device_properties(device).multi_processor_count


def plan_splits(B: int, Nk: int, max_groups: int, device: torch.device) -> int:
    return _ffi.lib().pq_decode_attn_plan(B, Nk, max(max_groups, 1), _num_cus(device))


def workspace_bytes(B: int, N: int, n_splits: int) -> int:
    return _ffi.lib().pq_decode_attn_workspace_bytes(B, N, n_splits)


def new_workspace(B: int, N: int, n_splits: int, device: torch.device) -> torch.Tensor:
    """An fp32 workspace for the split-K partials that the caller owns (pass it as `workspace=`).
    A caller that records the attention call into a HIP graph must own its workspace: the graph keeps
    the buffer's address, not a reference to the tensor."""
    return torch.empty((workspace_bytes(B, N, n_splits) + 3) // 4, dtype=torch.float32, device=device)


def workspace_for(B: int, N: int, n_splits: int, device: torch.device) -> torch.Tensor:
    """The cached workspace of eager calls: one per (device, stream), grown on demand.  Calls on one
    stream are ordered, so they can share it; calls on different streams get different buffers.  A
    replaced buffer goes back to torch's allocator, which hands it out again only behind the work
    already queued on that stream."""
    need = workspace_bytes(B, N, n_splits)
    key = (device.type, device.index, torch.cuda.current_stream(device).cuda_stream)
    ws = _WORKSPACES.get(key)
    if ws is None or ws.numel() * 4 < need:
        ws = torch.empty((need + 3) // 4, dtype=torch.float32, device=device)
        _WORKSPACES[key] = ws
    return ws


def balanced_slots(B: int, Nk: int, group_capacity: int, total_groups: Optional[int], wave_slots: int,
                   resid_capacity: int = GROUP) -> int:
    """Partial slots per head for PQ_BALANCED_SLICES: enough for the segment length the device will pick
    when the batch holds `total_groups` groups per KV head (None: sequences half full on average)."""
    # in tiles of 64 tokens: two per group, and per sequence one for its residual keys (on average) and three that
    # stand for a plane's start-up
    units = 2 * (total_groups if total_groups is not None else (B * group_capacity + 1) // 2) + 4 * B
    seg = max(1, -(-units * Nk // max(wave_slots, 1)))
    return max(2, -(-(2 * group_capacity + -(-resid_capacity // 64) + 3) // seg) + 1)


def _pick_workspace(workspace: Optional[torch.Tensor], B: int, N: int, n_splits: int, device: torch.device) -> torch.Tensor:
    if workspace is None:
        return workspace_for(B, N, n_splits, device)
    if (workspace.dtype != torch.float32 or workspace.device != device or not workspace.is_contiguous()
            or workspace.numel() * 4 < workspace_bytes(B, N, n_splits)):
        raise ValueError("polarquant_amd: workspace must be a contiguous fp32 tensor on %s with at least %d bytes"
                         % (device, workspace_bytes(B, N, n_splits)))
    return workspace


def polar_decode_attention(
    query_states: torch.Tensor,               # [B,N,1,128] or [B,N,128]
    indices: Optional[torch.Tensor],          # [B,Nk,cap,128,64] u8 (cap >= used groups; last dim 48: packed 6-bit codes) or None
    rscale: Optional[torch.Tensor], rmn: Optional[torch.Tensor],
    tscale: Optional[torch.Tensor], tmn: Optional[torch.Tensor],   # [B,Nk,cap,1,64]
    key_resid: Optional[torch.Tensor],        # [B,Nk,res_cap,128] fp16 keys not yet quantized (new key included)
    value_states: torch.Tensor,               # [B,Nk,v_cap,128]; rows [0, n_groups*128 + n_resid) are used
    n_groups: int, n_resid: int,
    attention_mask: Optional[torch.Tensor] = None,   # [B, >= n_groups*128 + n_resid] of {0,1}
    rbits: int = 4, tbits: int = 4, sm_scale: Optional[float] = None,
    n_groups_per_seq: Optional[torch.Tensor] = None, n_resid_per_seq: Optional[torch.Tensor] = None,
    n_splits: Optional[int] = None, out: Optional[torch.Tensor] = None,
    total_groups: Optional[int] = None, min_groups_per_split: Optional[int] = None,
    workspace: Optional[torch.Tensor] = None, balanced: Optional[bool] = None, single_wavefront: bool = False,
    status: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """-> attention output [B,N,1,128] in the query dtype.

    Ragged batches (`n_groups_per_seq` given): `total_groups`, the sum of the per-sequence group
    counts if the caller knows it on the host (no device sync is made here), lets the context be
    cut into slices of equal size across sequences, so that short sequences do not leave
    wavefronts idle; without it the average sequence is assumed to be half the capacity.
    `balanced` (the default with per-sequence counts and no explicit split): the slices are cut on the
    device from the actual counts so that all wavefronts get equal work (PQ_BALANCED_SLICES);
    `n_splits` is then the number of partial slots per head.
    `workspace`: a buffer from `new_workspace` that the caller owns (needed under graph capture);
    by default the cached buffer of the current stream is used.
    `single_wavefront`: the earlier kernels, in which one wavefront does all the work of a slice
    (PQ_SINGLE_WAVEFRONT), instead of the scorer / accumulator pairs; for comparison.
    `status`: an int32 tensor of one element on the same device that the caller has zeroed.  The default
    kernels set it to PQ_STATUS_HANDOVER_TIMEOUT (1) if a hand-over between a scorer and its accumulator
    gives up (the affected output rows are NaN too); nothing here reads it back, so no synchronisation
    is added: `int(status)` after the call is the caller's."""
    if not query_states.is_cuda:
        raise RuntimeError("polarquant_amd: decode attention needs tensors on the GPU (no CPU fallback)")
    dev = query_states.device
    B, N = query_states.shape[:2]
    hd = query_states.shape[-1]
    Nk = value_states.shape[1]
    assert hd == 128
    dt = _dtype_code(query_states)
    q = query_states.reshape(B, N, hd)
    if not q.is_contiguous() or q.data_ptr() % 16:
        q = q.clone(memory_format=torch.contiguous_format)
    assert value_states.is_contiguous() and value_states.dtype == query_states.dtype
    v_cap = value_states.shape[2]
    if indices is not None:
        assert indices.is_contiguous() and all(m.is_contiguous() for m in (rscale, rmn, tscale, tmn))
        g_cap = indices.shape[2]
        cptr = [indices.data_ptr(), rscale.data_ptr(), rmn.data_ptr(), tscale.data_ptr(), tmn.data_ptr()]
        flags = _ffi.PQ_CODES_PACKED6 if indices.shape[-1] == 48 else 0      # [.., 128, 48]: packed 6-bit codes
    else:
        g_cap, cptr, flags = 0, [None] * 5, 0
    if key_resid is not None:
        assert key_resid.is_contiguous() and key_resid.dtype == query_states.dtype
        r_cap, kptr = key_resid.shape[2], key_resid.data_ptr()
    else:
        r_cap, kptr = 0, None
    mptr, mstride = None, 0
    if attention_mask is not None:
        m8 = attention_mask if attention_mask.dtype == torch.uint8 else (attention_mask != 0).to(torch.uint8)
        m8 = m8.contiguous()
        mptr, mstride = m8.data_ptr(), m8.stride(0)
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(hd)
    max_groups = g_cap if n_groups_per_seq is not None else n_groups
    min_gps = 0
    if balanced is None:
        balanced = n_groups_per_seq is not None and n_splits is None and min_groups_per_split is None
    if single_wavefront:
        flags |= _ffi.PQ_SINGLE_WAVEFRONT
    if balanced:
        flags |= _ffi.PQ_BALANCED_SLICES
        if n_splits is None:
            n_splits = balanced_slots(B, Nk, max_groups, total_groups, 4 * _num_cus(dev), r_cap)
    elif n_groups_per_seq is not None and n_splits is None and max_groups > 0:
        tot = total_groups if total_groups is not None else (B * max_groups + 1) // 2
        # one wavefront per SIMD; every (sequence, KV head) rounds its slice count up, so leave one
        # slot per plane for that and the whole batch still runs in a single round
        slots = max(4 * _num_cus(dev) - B * Nk, B * Nk)
        min_gps = max(1, -(-tot * Nk // slots))
        n_splits = max(1, -(-max_groups // min_gps))
    if min_groups_per_split is not None:
        min_gps = min_groups_per_split
    if n_splits is None:
        n_splits = plan_splits(B, Nk, max_groups, dev)
    ws = _pick_workspace(workspace, B, N, n_splits, dev)
    if out is None:
        out = torch.empty((B, N, 1, hd), dtype=query_states.dtype, device=dev)
    gps = n_groups_per_seq.data_ptr() if n_groups_per_seq is not None else None
    rps = n_resid_per_seq.data_ptr() if n_resid_per_seq is not None else None
    sptr = None
    if status is not None:
        if status.dtype != torch.int32 or status.device != dev or status.numel() != 1:
            raise ValueError("polarquant_amd: status must be one int32 on %s" % dev)
        sptr = status.data_ptr()
    with torch.cuda.device(dev):
        rc = _ffi.lib().pq_decode_attn(
            q.data_ptr(), *cptr, g_cap, n_groups, gps, kptr, r_cap, n_resid, rps,
            value_states.data_ptr(), v_cap, mptr, mstride, float(sm_scale), B, N, Nk, rbits, tbits, dt,
            n_splits, min_gps, ws.data_ptr(), ws.numel() * 4, out.data_ptr(), flags, sptr, _stream_ptr(dev))
    _ffi.check(rc, "pq_decode_attn")
    return out


def polar_decode_attention_v4(
    query_states: torch.Tensor,               # [B,N,1,128] or [B,N,128]
    indices: Optional[torch.Tensor], rscale: Optional[torch.Tensor], rmn: Optional[torch.Tensor],
    tscale: Optional[torch.Tensor], tmn: Optional[torch.Tensor],
    key_resid: torch.Tensor,                  # [B,Nk,res_cap,128] keys of the residual window (new key included)
    value_resid: torch.Tensor,                # [B,Nk,res_cap,128] values of the same window
    value_codes: Optional[torch.Tensor],      # int32 [B,Nk,cap_tokens,16]; rows [0, n_groups*128) are used
    value_scale: Optional[torch.Tensor], value_mn: Optional[torch.Tensor],   # [B,Nk,cap_tokens,1]
    n_groups: int, n_resid: int,
    attention_mask: Optional[torch.Tensor] = None,
    rbits: int = 4, tbits: int = 4, sm_scale: Optional[float] = None,
    n_groups_per_seq: Optional[torch.Tensor] = None, n_resid_per_seq: Optional[torch.Tensor] = None,
    n_splits: Optional[int] = None, out: Optional[torch.Tensor] = None, min_groups_per_split: int = 0,
    workspace: Optional[torch.Tensor] = None, balanced: bool = False, total_groups: Optional[int] = None,
    single_wavefront: bool = False, status: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Decode attention of the reference's Mixed variant (polar keys + 4-bit values,
    models/modeling_llama_polar.py:185-241) -> [B,N,1,128] in the query dtype.
    `single_wavefront`, `status`: as for polar_decode_attention."""
    if not query_states.is_cuda:
        raise RuntimeError("polarquant_amd: decode attention needs tensors on the GPU (no CPU fallback)")
    dev = query_states.device
    B, N = query_states.shape[:2]
    hd = query_states.shape[-1]
    Nk = key_resid.shape[1]
    assert hd == 128
    dt = _dtype_code(query_states)
    q = query_states.reshape(B, N, hd)
    if not q.is_contiguous() or q.data_ptr() % 16:
        q = q.clone(memory_format=torch.contiguous_format)
    assert key_resid.is_contiguous() and value_resid.is_contiguous() and key_resid.shape == value_resid.shape
    assert key_resid.dtype == query_states.dtype == value_resid.dtype
    r_cap = key_resid.shape[2]
    if indices is not None:
        assert indices.is_contiguous() and all(m.is_contiguous() for m in (rscale, rmn, tscale, tmn))
        assert value_codes is not None and value_codes.is_contiguous() and value_codes.dtype == torch.int32
        assert value_scale.is_contiguous() and value_mn.is_contiguous() and value_scale.dtype == query_states.dtype
        g_cap, v4_cap = indices.shape[2], value_codes.shape[2]
        cptr = [indices.data_ptr(), rscale.data_ptr(), rmn.data_ptr(), tscale.data_ptr(), tmn.data_ptr()]
        vptr = [value_codes.data_ptr(), value_scale.data_ptr(), value_mn.data_ptr()]
        flags = _ffi.PQ_CODES_PACKED6 if indices.shape[-1] == 48 else 0
    else:
        g_cap, v4_cap, cptr, vptr, flags = 0, 0, [None] * 5, [None] * 3, 0
    mptr, mstride = None, 0
    if attention_mask is not None:
        m8 = attention_mask if attention_mask.dtype == torch.uint8 else (attention_mask != 0).to(torch.uint8)
        m8 = m8.contiguous()
        mptr, mstride = m8.data_ptr(), m8.stride(0)
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(hd)
    max_groups = g_cap if n_groups_per_seq is not None else n_groups
    if single_wavefront:
        flags |= _ffi.PQ_SINGLE_WAVEFRONT
    if balanced:
        flags |= _ffi.PQ_BALANCED_SLICES
        if n_splits is None:
            n_splits = balanced_slots(B, Nk, max_groups, total_groups, (8 if N // Nk <= 4 else 4) * _num_cus(dev), r_cap)
    if n_splits is None:
        n_splits = _ffi.lib().pq_decode_attn_v4_plan(B, N, Nk, max(max_groups, 1), _num_cus(dev))
    sptr = None
    if status is not None:
        if status.dtype != torch.int32 or status.device != dev or status.numel() != 1:
            raise ValueError("polarquant_amd: status must be one int32 on %s" % dev)
        sptr = status.data_ptr()
    ws = _pick_workspace(workspace, B, N, n_splits, dev)
    if out is None:
        out = torch.empty((B, N, 1, hd), dtype=query_states.dtype, device=dev)
    gps = n_groups_per_seq.data_ptr() if n_groups_per_seq is not None else None
    rps = n_resid_per_seq.data_ptr() if n_resid_per_seq is not None else None
    with torch.cuda.device(dev):
        rc = _ffi.lib().pq_decode_attn_v4(
            q.data_ptr(), *cptr, g_cap, n_groups, gps, key_resid.data_ptr(), r_cap, n_resid, rps,
            value_resid.data_ptr(), *vptr, v4_cap, mptr, mstride, float(sm_scale), B, N, Nk, rbits, tbits, dt,
            n_splits, min_groups_per_split, ws.data_ptr(), ws.numel() * 4, out.data_ptr(), flags, sptr, _stream_ptr(dev))
    _ffi.check(rc, "pq_decode_attn_v4")
    return out
