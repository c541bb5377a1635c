"""ctypes wrapper around oracle/libpolar_oracle.so (plain-C oracle).  TEST INFRASTRUCTURE ONLY."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build() -> str:
    subprocess.run(["make", "-C", _HERE, "-s"], check=True)
    return os.path.join(_HERE, "libpolar_oracle.so")


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "libpolar_oracle.so")
        if not os.path.exists(path):
            build()
        _LIB = ctypes.CDLL(path)
    return _LIB


def _words(t: torch.Tensor) -> np.ndarray:
    assert t.dtype in (torch.float16, torch.bfloat16)
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def _p(a: np.ndarray):
    return a.ctypes.data_as(ctypes.c_void_p)


def sleef_atan2f(y: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    """The C restatement of Sleef_atan2f_u10 on float32 tensors, element by element."""
    fn = lib().po_sleef_atan2f_u10
    fn.restype, fn.argtypes = ctypes.c_float, [ctypes.c_float, ctypes.c_float]
    ya, xa = y.contiguous().view(-1).tolist(), x.contiguous().view(-1).tolist()
    return torch.tensor([fn(a, b) for a, b in zip(ya, xa)], dtype=torch.float32).view(y.shape)


def quantize(key_states: torch.Tensor, rbits=4, tbits=4, group_size=128, wrap_fp32=False, angle_mode="group", libm_atan2=False):
    """libm_atan2: the angle by libm's atan2f instead of the SLEEF routine eager torch evaluates."""
    B, Nk, L, D2 = key_states.shape
    D, G, Nb = D2 // 2, group_size, L // group_size
    bf = int(key_states.dtype == torch.bfloat16)
    k = _words(key_states)
    codes = np.empty((B, Nk, Nb, G, D), np.uint8)
    meta = [np.empty((B, Nk, Nb, 1, D), np.uint16) for _ in range(4)]
    rc = lib().po_quantize(_p(k), bf, int(wrap_fp32) | (2 if angle_mode == "uniform" else 0) | (4 if libm_atan2 else 0), B, Nk, L, D, G, rbits, tbits, _p(codes), *[_p(m) for m in meta])
    assert rc == 0
    back = lambda m: torch.from_numpy(m.view(np.int16)).view(key_states.dtype)
    return (torch.from_numpy(codes),) + tuple(back(m) for m in meta)


def quantize_values(v: torch.Tensor, bits=4):
    """[B,Nk,T,128] -> (int32 [B,Nk,T,16], scale [B,Nk,T,1], mn [B,Nk,T,1])"""
    B, Nk, T, D = v.shape
    bf = int(v.dtype == torch.bfloat16)
    per = 32 // bits
    codes = np.empty((B, Nk, T, D // per), np.int32)
    scale, mn = np.empty((B, Nk, T, 1), np.uint16), np.empty((B, Nk, T, 1), np.uint16)
    rc = lib().po_quantize_values(_p(_words(v)), bf, ctypes.c_long(B * Nk * T), D, bits, _p(codes), _p(scale), _p(mn))
    assert rc == 0
    back = lambda m: torch.from_numpy(m.view(np.int16)).view(v.dtype)
    return torch.from_numpy(codes), back(scale), back(mn)


def scores(q, codes, rscale, rmn, tscale, tmn, rbits=4, tbits=4):
    B, N = q.shape[:2]
    _, Nk, Nb, G, D = codes.shape
    bf = int(q.dtype == torch.bfloat16)
    out = np.empty((B, N, 1, Nb * G), np.float32)
    rc = lib().po_scores(_p(_words(q)), bf, _p(codes.contiguous().numpy()), _p(_words(rscale)), _p(_words(rmn)),
                         _p(_words(tscale)), _p(_words(tmn)), _p(out), B, N, Nk, Nb, G, D, rbits, tbits)
    assert rc == 0
    return torch.from_numpy(out)


def decode_attn(q, codes, rscale, rmn, tscale, tmn, kres, v, mask=None, rbits=4, tbits=4):
    B, N, _, hd = q.shape
    Nk = v.shape[1]
    D, G = hd // 2, 128
    Nb = 0 if codes is None else codes.shape[2]
    res = 0 if kres is None else kres.shape[2]
    bf = int(q.dtype == torch.bfloat16)
    out = np.empty((B, N, 1, hd), np.uint16)
    nul = ctypes.c_void_p(0)
    args = [_p(_words(q)), bf]
    if Nb:
        args += [_p(codes.contiguous().numpy()), _p(_words(rscale)), _p(_words(rmn)), _p(_words(tscale)), _p(_words(tmn))]
    else:
        args += [nul] * 5
    args += [_p(_words(kres)) if res else nul, res, _p(_words(v))]
    args += [_p(mask.to(torch.uint8).contiguous().numpy()) if mask is not None else nul, _p(out)]
    rc = lib().po_decode_attn(*args, B, N, Nk, Nb, G, D, rbits, tbits)
    assert rc == 0
    return torch.from_numpy(out.view(np.int16)).view(q.dtype)
