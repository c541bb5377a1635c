"""The quantizer's scalar math (polarquant_amd/csrc/pq_math.h), built for the host,
against eager torch-CPU.  atan2f_sleef_u10 must equal torch.atan2 on float32 bit
for bit: that is what makes the GPU angle codes identical to eager torch's.

torch.atan2 itself is not one function: its AVX2 kernel (SLEEF with FMA), its
AVX-512 kernel and its scalar tail (libm) differ from each other by one fp32 ulp
on a few extreme-ratio inputs per million.  The restatement is that of the AVX2
kernel: the bit-for-bit tests run torch in a child process pinned to AVX2
(ATEN_CPU_CAPABILITY=avx2), and one test bounds the distance to whatever kernel
this machine dispatches by default."""
import ctypes
import os
import subprocess

import numpy as np
import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def shim():
    out_dir = os.path.join(HERE, "_build")
    os.makedirs(out_dir, exist_ok=True)
    so = os.path.join(out_dir, "libpq_host_math.so")
    src = os.path.join(HERE, "host_math_shim.cpp")
    subprocess.run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-mfma", "-ffp-contract=off", "-fno-fast-math",
                    "-o", so, src], check=True)
    return ctypes.CDLL(so)


def _atan2(shim, y, x):
    y = np.ascontiguousarray(y, np.float32); x = np.ascontiguousarray(x, np.float32)
    out = np.empty_like(y)
    shim.pqh_atan2f(ctypes.c_void_p(y.ctypes.data), ctypes.c_void_p(x.ctypes.data), ctypes.c_void_p(out.ctypes.data),
                    ctypes.c_long(y.size))
    return out


def _torch_atan2_avx2(y, x):
    """torch.atan2(y, x) on float32, evaluated by a child process pinned to torch's AVX2 kernels."""
    import sys
    import tempfile
    with tempfile.TemporaryDirectory() as d:
        np.save(os.path.join(d, "y.npy"), np.ascontiguousarray(y, np.float32))
        np.save(os.path.join(d, "x.npy"), np.ascontiguousarray(x, np.float32))
        code = ("import numpy as np, torch, sys; d=sys.argv[1]; "
                "assert torch.backends.cpu.get_cpu_capability()=='AVX2', torch.backends.cpu.get_cpu_capability(); "
                "r=torch.atan2(torch.from_numpy(np.load(d+'/y.npy')), torch.from_numpy(np.load(d+'/x.npy'))); "
                "np.save(d+'/r.npy', r.numpy())")
        env = dict(os.environ, ATEN_CPU_CAPABILITY="avx2")
        r = subprocess.run([sys.executable, "-c", code, d], env=env, capture_output=True, text=True)
        if r.returncode != 0:
            pytest.skip("torch cannot be pinned to AVX2 here: " + r.stderr[-200:])
        return np.load(os.path.join(d, "r.npy"))


def _same_bits(a, b):
    a, b = a.view(np.int32), b.view(np.int32)
    nan = (np.isnan(a.view(np.float32)) & np.isnan(b.view(np.float32)))
    return int(((a != b) & ~nan).sum())


def test_atan2_bit_exact_on_half_valued_inputs(shim):
    g = torch.Generator().manual_seed(0)
    n = 1 << 23
    y = (torch.randn(n, generator=g) * 3).half().float()
    x = (torch.randn(n, generator=g) * 3).half().float()
    # pad to a multiple of the vector width so that no element takes torch's scalar (libm) tail
    assert _same_bits(_atan2(shim, y.numpy(), x.numpy()), _torch_atan2_avx2(y.numpy(), x.numpy())) == 0


def test_atan2_bit_exact_on_bf16_and_wide_range_inputs(shim):
    g = torch.Generator().manual_seed(1)
    n = 1 << 22
    e = torch.randint(-14, 15, (n,), generator=g).float()
    y = (torch.randn(n, generator=g) * torch.exp2(e)).bfloat16().float()
    e2 = torch.randint(-14, 15, (n,), generator=g).float()
    x = (torch.randn(n, generator=g) * torch.exp2(e2)).half().float()
    assert _same_bits(_atan2(shim, y.numpy(), x.numpy()), _torch_atan2_avx2(y.numpy(), x.numpy())) == 0


def test_atan2_all_pairs_of_a_half_grid_and_specials(shim):
    """Every (y, x) pair from a grid of 1500 half values (all exponents, subnormals, zeros,
    infinities, both signs): 2.25M pairs, including every special case of atan2."""
    bits = np.concatenate([np.arange(0, 0x7c01, 43, dtype=np.uint16), np.array([0, 1, 2, 0x3ff, 0x400, 0x7bff, 0x7c00, 0x3c00], np.uint16)])
    bits = np.concatenate([bits, bits | 0x8000]).astype(np.uint16)
    vals = torch.from_numpy(bits.view(np.int16)).view(torch.float16).float()
    y = vals[:, None].expand(-1, vals.numel()).reshape(-1).contiguous()
    x = vals[None, :].expand(vals.numel(), -1).reshape(-1).contiguous()
    pad = (-y.numel()) % 64
    y = torch.cat([y, torch.ones(pad)]); x = torch.cat([x, torch.ones(pad)])
    ours = _atan2(shim, y.numpy(), x.numpy())
    assert _same_bits(ours, _torch_atan2_avx2(y.numpy(), x.numpy())) == 0
    # against this machine's default torch kernel: at most one ulp apart, on a handful of extreme ratios
    ref = torch.atan2(y, x).numpy()
    diff = np.abs(ours.view(np.int32).astype(np.int64) - ref.view(np.int32).astype(np.int64))
    diff[np.isnan(ours) & np.isnan(ref)] = 0
    print("vs default torch kernel (%s): %d of %d differ" % (torch.backends.cpu.get_cpu_capability(), int((diff > 0).sum()), diff.size))
    assert int(diff.max()) <= 1 and int((diff > 0).sum()) <= 1e-5 * diff.size
    nan = torch.tensor([float("nan"), 1.0, float("nan")]); one = torch.tensor([1.0, float("nan"), float("nan")])
    assert np.isnan(_atan2(shim, nan.numpy(), one.numpy())).all()


def test_half_and_bf16_conversions_match_torch(shim):
    allh = np.arange(0, 65536, dtype=np.uint16)
    f = np.empty(65536, np.float32)
    shim.pqh_half_to_float(ctypes.c_void_p(allh.ctypes.data), ctypes.c_void_p(f.ctypes.data), ctypes.c_long(65536))
    ref = torch.from_numpy(allh.view(np.int16)).view(torch.float16).float().numpy()
    assert _same_bits(f, ref) == 0
    g = torch.Generator().manual_seed(2)
    x = torch.cat([torch.randn(1 << 20, generator=g) * 100, torch.randn(1 << 20, generator=g) * 1e-5,
                   torch.tensor([0.0, -0.0, 65504.0, 65520.0, 1e9, -1e9, 6.1e-5, 5.96e-8, 2.98e-8, 3e-8, float("inf")])])
    # ties: midpoints between adjacent halves
    mid = (ref[1024:30000:7].astype(np.float64) + ref[1025:30001:7].astype(np.float64)) / 2
    x = torch.cat([x, torch.from_numpy(mid.astype(np.float32))]).contiguous()
    h = np.empty(x.numel(), np.uint16); b = np.empty(x.numel(), np.uint16)
    shim.pqh_float_to_half(ctypes.c_void_p(x.numpy().ctypes.data), ctypes.c_void_p(h.ctypes.data), ctypes.c_long(x.numel()))
    shim.pqh_float_to_bf16(ctypes.c_void_p(x.numpy().ctypes.data), ctypes.c_void_p(b.ctypes.data), ctypes.c_long(x.numel()))
    assert np.array_equal(h.view(np.int16), x.half().view(torch.int16).numpy())
    assert np.array_equal(b.view(np.int16), x.bfloat16().view(torch.int16).numpy())
