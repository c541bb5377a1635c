"""The reference's quantizer lines as eager torch ops on DEVICE tensors.  TEST INFRASTRUCTURE ONLY.

Only tests/ and bench.py's checker legs may import this; the product (polarquant_amd/) never does.

oracle/polar_oracle.py evaluates the reference's lines on CPU tensors.  The reference itself runs them
on GPU tensors, where eager torch evaluates two of them differently (`phi + 2*pi` keeps the scalar in
fp32 instead of casting it to the tensor dtype, and `torch.atan2` is the device math library's atan2f
instead of SLEEF's).  The second difference cannot be restated on a CPU, so the GPU-eager mode of the HIP
quantizer (PQ_EAGER_GPU) is pinned against this function run ON THE GPU BOX: torch-ROCm's own kernels
(a library, not the reference) then evaluate each line the way the reference's lines are evaluated
when the model runs on a GPU.

Pin status: the function is the reference's twelve lines (models/modeling_llama_polar.py:141-155) with
library routines only; on CPU tensors it must agree bit for bit with polar_oracle.quantize_and_pack_nbit
(tests/test_oracle_pins.py), whose pins then carry over; what the device evaluation adds (the device
atan2f, the fp32 wrap) is torch's own behaviour and is not restated anywhere.  PARITY UNPINNED against
CUDA's atan2f: the reference publishes no vectors, and ROCm's device library is what can be run here.
"""
from __future__ import annotations

import math

import torch


def quantize_and_pack_nbit_eager(key_states: torch.Tensor, rbits: int = 4, tbits: int = 4, group_size: int = 128):
    """key_states [B,Nk,L,2*D] half/bf16 on ANY device -> (indices u8 [B,Nk,Nb,G,D], rscale, rmn, tscale, tmn
    [B,Nk,Nb,1,D]) by the literal lines of models/modeling_llama_polar.py:141-155.  Degenerate groups
    (0/0 -> uint8, undefined in the reference) must be avoided by the caller."""
    B, N, L, D2 = key_states.shape
    D, G = D2 // 2, group_size
    ks = key_states.view(B, N, L // G, G, 2, D)                                  # :141
    phi = torch.atan2(ks[:, :, :, :, 1, :], ks[:, :, :, :, 0, :])               # :143
    phi = torch.where(phi < 0, phi + 2 * math.pi, phi)                          # :144
    tmx, tmn = phi.max(-2, keepdim=True)[0], phi.min(-2, keepdim=True)[0]       # :146
    tscale = (tmx - tmn) / (2 ** tbits)                                         # :147
    theta = torch.clamp(torch.floor((phi - tmn) / tscale).to(torch.uint8), 0, 2 ** tbits - 1)   # :148
    radii = torch.norm(ks, p=2, dim=-2)                                         # :150
    rmx, rmn = radii.max(-2, keepdim=True)[0], radii.min(-2, keepdim=True)[0]   # :151
    rscale = (rmx - rmn) / (2 ** rbits)                                         # :152
    rho = torch.clamp(torch.floor((radii - rmn) / rscale).to(torch.uint8), 0, 2 ** rbits - 1)   # :153
    return (rho << tbits) + theta, rscale, rmn, tscale, tmn                     # :155
