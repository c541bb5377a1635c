"""GPU parity of pq_quantize_groups (through the C ABI) against the CPU oracle.

Bar: packed codes and the four metadata tensors bit-exact.  Any disagreement
is an "edge flip"; flips are counted and the target (asserted) is 0.
"""
import math

import pytest
import torch

from oracle import polar_oracle as po
from oracle.device_eager import quantize_and_pack_nbit_eager
from polarquant_amd import workloads as wl
from polarquant_amd.quantize import quantize_and_pack_nbit

pytestmark = pytest.mark.gpu

NAMES = ["codes", "rscale", "rmn", "tscale", "tmn"]


def _bits(t):
    return t if t.dtype == torch.uint8 else t.view(torch.int16)


def count_flips(got, ref):
    """-> dict name -> number of differing elements (metadata compared by value so that -0.0 == +0.0)."""
    out = {}
    for n, g, r in zip(NAMES, got, ref):
        g = g.cpu()
        if g.dtype == torch.uint8:
            out[n] = int((g != r).sum())
        else:
            out[n] = int(((g.float() != r.float()) & ~(g.float().isnan() & r.float().isnan())).sum())
    return out


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("rbits,tbits", [(4, 4), (3, 3), (2, 4), (5, 3), (4, 2), (2, 6), (1, 7)])
def test_quantize_bit_exact(gpu, dtype, rbits, tbits):
    print("case", dtype, rbits, tbits, flush=True)
    g = torch.Generator().manual_seed(21)
    k = wl.make_keys(2, 4, 1024, 5e5, g, dtype)
    ref = po.quantize_and_pack_nbit(k, rbits, tbits)
    got = quantize_and_pack_nbit(k.to(gpu), rbits, tbits)
    torch.cuda.synchronize()
    assert [tuple(t.shape) for t in got] == [tuple(t.shape) for t in ref]
    flips = count_flips(got, ref)
    print("flips", flips, flush=True)
    assert all(v == 0 for v in flips.values()), flips


def test_quantize_cfg0_full_flip_count(gpu):
    """Workload configs[0] keys: [1,32,4096,128] fp16, RoPE theta 1e4, 4/4 bits."""
    sh = wl.CONFIGS[0]
    inp = wl.make_decode_inputs(sh)
    ref = po.quantize_and_pack_nbit(inp.k, 4, 4)
    got = quantize_and_pack_nbit(inp.k.to(gpu), 4, 4)
    flips = count_flips(got, ref)
    print("cfg0 flips", flips, "of", ref[0].numel(), "codes", flush=True)
    assert all(v == 0 for v in flips.values()), flips


def test_quantize_strided_transposed_view(gpu):
    """Keys arrive as a transposed view of the [B,L,Nk,128] projection output
    (modeling_llama_polar.py:54); the kernel reads them in place."""
    g = torch.Generator().manual_seed(5)
    B, Nk, L = 2, 4, 256
    k_blhd = wl.make_half((B, L, Nk, 128), g)
    k = k_blhd.transpose(1, 2)
    ref = po.quantize_and_pack_nbit(k.contiguous(), 4, 4)
    kd = k_blhd.to(gpu).transpose(1, 2)
    assert not kd.is_contiguous()
    got = quantize_and_pack_nbit(kd, 4, 4)
    assert all(v == 0 for v in count_flips(got, ref).values())


def test_quantize_into_cache_slot(gpu):
    """Quantize-on-append writes one group into a pre-allocated cache at a group offset."""
    g = torch.Generator().manual_seed(6)
    B, Nk, cap = 2, 2, 5
    k = wl.make_keys(B, Nk, 256, 1e4, g)
    ref = po.quantize_and_pack_nbit(k, 4, 4)
    codes = torch.zeros(B, Nk, cap, 128, 64, dtype=torch.uint8, device=gpu)
    meta = [torch.zeros(B, Nk, cap, 1, 64, dtype=torch.float16, device=gpu) for _ in range(4)]
    got = quantize_and_pack_nbit(k.to(gpu), 4, 4, out=(codes, *meta), group_offset=2)
    assert all(v == 0 for v in count_flips(got, ref).values())
    assert int(codes[:, :, :2].sum()) == 0 and int(codes[:, :, 4:].sum()) == 0
    assert torch.equal(codes[:, :, 2:4].cpu(), ref[0])


def test_quantize_special_values(gpu):
    """Zeros, axis-aligned keys, constant groups (scale == 0 -> code 0), negative zero, tiny and huge values."""
    g = torch.Generator().manual_seed(9)
    k = wl.make_half((1, 2, 256, 128), g)
    k[0, 0, :128, :8] = 0.0                      # x == 0 for pairs 0..7 in group 0
    k[0, 0, :128, 64 + 8:64 + 16] = 0.0          # y == 0 for pairs 8..15
    k[0, 0, :128, 16] = 1.5; k[0, 0, :128, 64 + 16] = -2.0   # constant pair -> both scales 0
    k[0, 0, :128, 17] = 0.0; k[0, 0, :128, 64 + 17] = 0.0    # origin
    k[0, 1, :128, 18] = -0.0
    k[0, 1, 5, 19] = 6.0e-8; k[0, 1, 6, 64 + 19] = -6.0e-8    # subnormal halves
    k[0, 1, 7, 20] = 60000.0; k[0, 1, 8, 64 + 20] = -60000.0
    ref = po.quantize_and_pack_nbit(k, 4, 4)
    got = quantize_and_pack_nbit(k.to(gpu), 4, 4)
    flips = count_flips(got, ref)
    assert all(v == 0 for v in flips.values()), flips


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("rbits,tbits", [(4, 4), (3, 3)])
def test_quantize_uniform_angle_mode(gpu, dtype, rbits, tbits):
    """Fixed angle bins over [-pi, pi): bit-exact against the oracle's same mode, and the cache
    it writes is decoded by the unchanged score kernel."""
    from polarquant_amd.kernel4group import attention_decode_forward_triton_impl
    print("case uniform", dtype, rbits, tbits, flush=True)
    g = torch.Generator().manual_seed(23)
    k = wl.make_keys(2, 4, 1024, 5e5, g, dtype)
    ref = po.quantize_and_pack_nbit(k, rbits, tbits, angle_mode="uniform")
    got = quantize_and_pack_nbit(k.to(gpu), rbits, tbits, angle_mode="uniform")
    flips = count_flips(got, ref)
    print("flips", flips, flush=True)
    assert all(v == 0 for v in flips.values()), flips
    q = wl.make_half((2, 8, 1, 128), g, dtype)
    want = po.decode_scores(q, *ref, rbits, tbits)
    have = attention_decode_forward_triton_impl(q.to(gpu), *got, rbits=rbits, tbits=tbits).cpu()
    assert (have - want).abs().max().item() <= 1e-3 * want.abs().max().item()
    # and they approximate the scores of the unquantized keys
    exact = torch.matmul(q.float(), po.repeat_kv(k, 2).float().transpose(2, 3))
    rel = (have - exact).norm() / exact.norm()
    assert rel < (0.15 if tbits == 4 else 0.3), rel    # quantization noise of a fixed 2*pi/2^t grid


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape,rbits,tbits,theta", [((1, 2, 512), 4, 4, 1e4), ((2, 4, 1024), 3, 3, 1e6), ((1, 8, 2048), 4, 4, 5e5)])
def test_quantize_wrap_fp32_flag(gpu, dtype, shape, rbits, tbits, theta):
    """PQ_WRAP_FP32 adds 2*pi in fp32 (what an eager GPU add of a half tensor and a python float does): bit for bit
    the codes and metadata of both CPU restatements with the same switch (torch ops; plain C with its own SLEEF
    arctangent)."""
    from oracle import c_oracle as co
    print("case wrap_fp32", dtype, shape, rbits, tbits, flush=True)
    g = torch.Generator().manual_seed(2)
    k = wl.make_keys(*shape, theta, g, dtype)
    got = quantize_and_pack_nbit(k.to(gpu), rbits, tbits, wrap_fp32=True)
    for name, ref in (("torch", po.quantize_and_pack_nbit(k, rbits, tbits, wrap_fp32=True)), ("C", co.quantize(k, rbits, tbits, wrap_fp32=True))):
        flips = count_flips(got, ref)
        print("wrap_fp32 flips vs", name, "oracle", flips, flush=True)
        assert all(v == 0 for v in flips.values()), (name, flips)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("cfg,rbits,tbits", [(0, 4, 4), (2, 3, 3)])
def test_quantize_eager_gpu_mode_against_eager_torch_on_the_device(gpu, dtype, cfg, rbits, tbits):
    """eager_gpu=True (PQ_WRAP_FP32 | PQ_DEVICE_ATAN2) against the reference's lines evaluated by eager torch ops on
    device tensors, on the keys of configs[0] (all 8.4 M codes) and a configs[2]-like shape.  The radius side and
    its metadata must be identical; the angle side can only differ where the device library's atan2f linked into
    this library and the one inside torch differ, which is counted, printed and required to be nil.  The default
    (CPU-eager) mode is measured against the same device evaluation and reported: that distance is why the
    switch exists."""
    print("case eager gpu", dtype, cfg, flush=True)
    sh = wl.CONFIGS[cfg]
    g = torch.Generator().manual_seed(sh.seed)
    k = wl.make_keys(1, sh.n_kv_heads, 4096, sh.rope_theta, g, dtype).to(gpu)
    ref = quantize_and_pack_nbit_eager(k, rbits, tbits)
    got = quantize_and_pack_nbit(k, rbits, tbits, eager_gpu=True)
    torch.cuda.synchronize()
    flips = count_flips([t.cpu() for t in got], [t.cpu() for t in ref])
    base = count_flips([t.cpu() for t in quantize_and_pack_nbit(k, rbits, tbits)], [t.cpu() for t in ref])
    rho_flips = int(((got[0] >> tbits) != (ref[0] >> tbits)).sum())
    print("eager_gpu mode vs eager torch on the device:", flips, "radius-code flips", rho_flips, "| default (CPU-eager) mode vs the same:", base, flush=True)
    assert rho_flips == 0 and flips["rscale"] == 0 and flips["rmn"] == 0
    assert all(v == 0 for v in flips.values()), flips


def test_quantize_device_atan2_flag_alone(gpu):
    """PQ_DEVICE_ATAN2 without the fp32 wrap differs from the default only through the arctangent: a few angle codes
    and angle metadata words per million, never the radius side."""
    g = torch.Generator().manual_seed(41)
    k = wl.make_keys(1, 8, 4096, 5e5, g).to(gpu)
    a = quantize_and_pack_nbit(k, 4, 4)
    b = quantize_and_pack_nbit(k, 4, 4, device_atan2=True)
    flips = count_flips([t.cpu() for t in b], [t.cpu() for t in a])
    print("device atan2f vs SLEEF atan2f:", flips, flush=True)
    assert flips["rscale"] == 0 and flips["rmn"] == 0 and int(((a[0] >> 4) != (b[0] >> 4)).sum()) == 0
    assert flips["codes"] <= 1e-4 * a[0].numel()


@pytest.mark.parametrize("dtype_code,name", [(0, "float16"), (1, "bfloat16")])
def test_quantizer_math_selftest_exhaustive(gpu, dtype_code, name):
    """The cheap-estimate-with-guard path against the exact path on all 2^32 operand pairs of the dtype."""
    from polarquant_amd import _ffi
    counters = torch.zeros(5, dtype=torch.int64, device=gpu)
    rc = _ffi.lib().pq_selftest_quantizer_math(dtype_code, counters.data_ptr(), torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    bad, slow, bad_div, bad_dev, slow_dev = counters.tolist()
    print("%s: %d mismatching pairs, %.3f%% of pairs take the exact path, %d mismatching quotients; with the device "
          "library's atan2f as the exact routine: %d mismatching pairs, %.3f%% take the exact path"
          % (name, bad, 100.0 * slow / 2 ** 32, bad_div, bad_dev, 100.0 * slow_dev / 2 ** 32), flush=True)
    assert bad == 0
    assert bad_dev == 0
    assert bad_div == 0     # reciprocal + two fused multiply-adds against the fp32 division, every (dividend, scale) pair


def test_radius_on_a_double_rounding_tie(gpu):
    """x = 0xa2cd, y = 0x15b1 (half words): the correctly rounded fp32 square root of x^2 + y^2 lies one ulp above
    a midpoint between two half values, a 1-ulp-low square root lies exactly on it and rounds (to even) the other
    way.  Eager torch gives the upper neighbour; the kernel's exact path must use a correctly rounded root."""
    bits = torch.tensor([0xa2cd - 65536, 0x15b1], dtype=torch.int16).view(torch.float16)
    g = torch.Generator().manual_seed(77)
    k = (torch.randn(1, 1, 128, 128, generator=g) * 0.5 + 2.0).half()       # every other radius is far larger
    k[0, 0, 5, 0], k[0, 0, 5, 64] = bits[0], bits[1]
    ref = po.quantize_and_pack_nbit(k, 4, 4)
    assert ref[2][0, 0, 0, 0, 0].item() == 0.01335906982421875              # the minimum radius of pair 0
    got = quantize_and_pack_nbit(k.to(gpu), 4, 4)
    flips = count_flips(got, ref)
    assert all(v == 0 for v in flips.values()), flips
