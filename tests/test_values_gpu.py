"""4-bit values of the Mixed variant on the GPU against the CPU oracle: the value quantizer is
bit-exact (codes, scale, zero-point), the fused decode attention over polar keys + 4-bit values
meets the output bar against the literal restatement and the fp64 evaluation."""
import math

import pytest
import torch

from oracle import polar_oracle as po
from polarquant_amd import workloads as wl
from polarquant_amd.attention import polar_decode_attention_v4 as _polar_decode_attention_v4
from polarquant_amd.values import quantize_values

pytestmark = pytest.mark.gpu
RTOL, ATOL = 1e-2, 1e-3

# Every test of this file runs twice: with the default flags and with PQ_SINGLE_WAVEFRONT, which for this entry point
# changes the kernels only while nothing has been quantized yet (the residual window alone goes through the
# half-precision-value kernels: scorer / accumulator pairs, or one wavefront per slice).
_FORM = {"single": False}


@pytest.fixture(autouse=True, params=[False, True], ids=["pairs", "single"])
def _kernel_form(request):
    _FORM["single"] = request.param
    yield
    _FORM["single"] = False


def polar_decode_attention_v4(*args, **kwargs):
    return _polar_decode_attention_v4(*args, single_wavefront=_FORM["single"], **kwargs)


def _same_bits(a, b):
    a, b = a.cpu(), b.cpu()
    if a.dtype != torch.int32:
        a, b = a.view(torch.int16), b.view(torch.int16)
    return int((a != b).sum())


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("T", [1, 17, 128, 1000])
def test_value_quantizer_bit_exact(gpu, dtype, T):
    print("case values", dtype, T, flush=True)
    g = torch.Generator().manual_seed(31 + T)
    v = wl.make_half((2, 3, T, 128), g, dtype)
    v[0, 0, 0] = 0.75                               # constant row: 0/0 -> code 0
    if T > 2:
        v[1, 2, 2] *= 1e-3                          # tiny range
        v[1, 1, 1, ::2] = 100.0                     # two-valued row
    ref = po.quantize_values_along_last_dim(v)
    got = quantize_values(v.to(gpu))
    torch.cuda.synchronize()
    assert [tuple(t.shape) for t in got] == [tuple(t.shape) for t in ref]
    flips = [_same_bits(a, b) for a, b in zip(got, ref)]
    print("value flips (codes words, scale, mn)", flips, flush=True)
    assert flips == [0, 0, 0]


def test_value_quantizer_strided_input_and_cache_slot(gpu):
    g = torch.Generator().manual_seed(5)
    v = wl.make_half((2, 256, 4, 128), g)            # [B, T, Nk, 128] as the projection leaves it
    vt = v.to(gpu).transpose(1, 2)                   # [B, Nk, T, 128] view, token stride Nk*128
    ref = po.quantize_values_along_last_dim(v.transpose(1, 2).contiguous())
    cap = 512
    out = (torch.full((2, 4, cap, 16), -1, dtype=torch.int32, device=gpu),
           torch.zeros(2, 4, cap, 1, dtype=torch.float16, device=gpu), torch.zeros(2, 4, cap, 1, dtype=torch.float16, device=gpu))
    got = quantize_values(vt, out=out, token_offset=128)
    assert all(_same_bits(a, b) == 0 for a, b in zip(got, ref))
    assert bool((out[0][:, :, :128] == -1).all()) and bool((out[0][:, :, 384:] == -1).all())


def _close(got, ref, rtol=RTOL, atol=ATOL):
    got, ref = got.double(), ref.double()
    err = (got - ref).abs()
    return int((err > atol + rtol * ref.abs()).sum()), float(err.max())


def _case(gpu, B, N, Nk, n_groups, n_resid, rbits, tbits, dtype, mask_pad=0, seed=0, n_splits=None, caps=(0, 0), ragged=None):
    g = torch.Generator().manual_seed(seed)
    Lq = n_groups * 128
    L = Lq + n_resid
    k = wl.make_keys(B, Nk, L, 5e5, g, dtype)
    q = wl.make_half((B, N, 1, 128), g, dtype)
    v = wl.make_half((B, Nk, L, 128), g, dtype)
    v[..., 5] += 2.0                                 # a channel with an offset: exercises the zero-point term
    quant, vq = (None,) * 5, (None,) * 3
    if n_groups:
        quant = po.quantize_and_pack_nbit(k[:, :, :Lq].contiguous(), rbits, tbits)
        vq = po.quantize_values_along_last_dim(v[:, :, :Lq].contiguous())
    kres, vres = k[:, :, Lq:].contiguous(), v[:, :, Lq:].contiguous()
    mask = None
    if mask_pad:
        mask = torch.ones(B, L, dtype=torch.int64)
        for b in range(B):
            mask[b, :(mask_pad * (b + 1)) % L] = 0
    ref = po.decode_attention_mixed(q, kres, *quant, vres, *vq, mask, rbits, tbits)
    ref64 = po.decode_attention_mixed_exact(q, kres, *quant, vres, *vq, mask, rbits, tbits)
    gc, rc = caps
    dq, dvq = [None] * 5, [None] * 3
    if n_groups:
        cap = n_groups + gc
        dq = [torch.zeros((B, Nk, cap) + tuple(t.shape[3:]), dtype=t.dtype, device=gpu) for t in quant]
        for d, t in zip(dq, quant):
            d[:, :, :n_groups] = t.to(gpu)
        dvq = [torch.full((B, Nk, cap * 128, t.shape[3]), -1 if t.dtype == torch.int32 else float("nan"), dtype=t.dtype, device=gpu)
               for t in vq]
        for d, t in zip(dvq, vq):
            d[:, :, :Lq] = t.to(gpu)
    dk = torch.zeros(B, Nk, 128 + rc, 128, dtype=dtype, device=gpu)
    dv = torch.full((B, Nk, 128 + rc, 128), float("nan"), dtype=dtype, device=gpu)   # rows past the fill must not contribute
    dk[:, :, :n_resid], dv[:, :, :n_resid] = kres.to(gpu), vres.to(gpu)
    out = polar_decode_attention_v4(q.to(gpu), *dq, dk, dv, *dvq, n_groups, n_resid,
                                    attention_mask=None if mask is None else mask.to(gpu),
                                    rbits=rbits, tbits=tbits, n_splits=n_splits)
    torch.cuda.synchronize()
    out = out.cpu()
    assert out.shape == (B, N, 1, 128) and out.dtype == dtype and torch.isfinite(out.float()).all()
    return out, ref, ref64


@pytest.mark.parametrize("N,Nk", [(8, 2), (4, 4), (7, 1), (2, 1)])
@pytest.mark.parametrize("n_groups,n_resid", [(3, 1), (1, 128), (8, 77), (0, 5)])
def test_attention_v4_matches_oracle(gpu, N, Nk, n_groups, n_resid):
    print("case v4", N, Nk, n_groups, n_resid, flush=True)
    out, ref, ref64 = _case(gpu, 2, N, Nk, n_groups, n_resid, 4, 4, torch.float16, seed=n_groups * 131 + n_resid)
    for r in (ref, ref64):
        nbad, emax = _close(out, r)
        assert nbad == 0, (nbad, emax)


@pytest.mark.parametrize("rbits,tbits", [(3, 3), (4, 2)])
def test_attention_v4_other_bit_widths_mask_and_capacity(gpu, rbits, tbits):
    out, ref, ref64 = _case(gpu, 3, 8, 2, 5, 33, rbits, tbits, torch.float16, mask_pad=150, seed=9, caps=(3, 7))
    for r in (ref, ref64):
        nbad, emax = _close(out, r)
        assert nbad == 0, (nbad, emax)


@pytest.mark.parametrize("n_splits", [1, 2, 5, 16])
def test_attention_v4_split_counts_agree(gpu, n_splits):
    out, ref, ref64 = _case(gpu, 1, 8, 2, 9, 2, 4, 4, torch.float16, seed=3, n_splits=n_splits)
    nbad, emax = _close(out, ref64)
    assert nbad == 0, (nbad, emax)


@pytest.mark.parametrize("n_groups,n_splits", [(1, 2), (3, 2), (8, 8), (5, 7)])
@pytest.mark.parametrize("n_resid", [64, 65, 128])
def test_attention_v4_long_residual_windows_and_split_counts(gpu, n_groups, n_splits, n_resid):
    """A full or nearly full residual window on the slice that ends the plane, at several split counts."""
    out, ref, ref64 = _case(gpu, 2, 8, 2, n_groups, n_resid, 4, 4, torch.float16, seed=17 * n_groups + n_resid, n_splits=n_splits)
    # a short context: each element against the fp64 value or the reference path's own evaluation
    o, r, r64 = out.double(), ref.double(), ref64.double()
    bad = ((o - r64).abs() > ATOL + RTOL * r64.abs()) & ((o - r).abs() > ATOL + RTOL * r.abs())
    assert int(bad.sum()) == 0, float((o - r64).abs().max())


def test_attention_v4_bf16(gpu):
    out, ref, ref64 = _case(gpu, 2, 8, 2, 16, 3, 4, 4, torch.bfloat16, seed=4)
    nbad, emax = _close(out, ref64, 2e-2, 4e-3)      # bf16 has 8 mantissa bits
    assert nbad == 0, (nbad, emax)


def test_attention_v4_peaked_softmax_keeps_code_and_zero_point_terms_consistent(gpu):
    """When one token takes nearly all the probability, code*scale (~3) and the zero-point (~-3) of
    that token must be weighted by the same rounded probability, or their cancellation leaves an
    error of a probability's rounding error times 3.  Checked tightly against fp64, for 1 and many splits."""
    g = torch.Generator().manual_seed(77)
    B, N, Nk, nb = 1, 4, 1, 24
    L = nb * 128
    k = wl.make_keys(B, Nk, L + 1, 5e5, g)
    q = wl.make_half((B, N, 1, 128), g)
    for j in range(N):
        q[0, j, 0] = (k[0, 0, 100 + 500 * j].float() * 0.9).half()      # each head locks onto one cached token
    v = wl.make_half((B, Nk, L + 1, 128), g)
    quant = po.quantize_and_pack_nbit(k[:, :, :L].contiguous())
    vq = po.quantize_values_along_last_dim(v[:, :, :L].contiguous())
    kres, vres = k[:, :, L:].contiguous(), v[:, :, L:].contiguous()
    ref64 = po.decode_attention_mixed_exact(q, kres, *quant, vres, *vq)
    dk = torch.zeros(B, Nk, 128, 128, dtype=torch.float16, device=gpu)
    dv = torch.zeros_like(dk)
    dk[:, :, :1], dv[:, :, :1] = kres.to(gpu), vres.to(gpu)
    for ns in (1, 4, 24):
        out = polar_decode_attention_v4(q.to(gpu), *[t.to(gpu) for t in quant], dk, dv, *[t.to(gpu) for t in vq], nb, 1,
                                        n_splits=ns).cpu()
        err = (out.double() - ref64).abs().max().item()
        print("peaked, n_splits", ns, "max abs err %.2e (|out| up to %.2f)" % (err, ref64.abs().max().item()), flush=True)
        assert err < 1.5e-3 * max(1.0, ref64.abs().max().item()), (ns, err)


def test_attention_v4_ragged_batch_matches_per_sequence_oracle(gpu):
    """Per-sequence group / residual counts (device arrays) with 4-bit values: every sequence must
    equal the oracle run on that sequence alone, including one with no quantized group and one
    with a full residual window; rows past a sequence's fill hold NaN and must not contribute."""
    g = torch.Generator().manual_seed(41)
    B, N, Nk, cap = 5, 8, 2, 6
    groups = [0, 1, 6, 3, 2]
    resid = [7, 128, 1, 64, 33]
    q = wl.make_half((B, N, 1, 128), g)
    codes = torch.zeros(B, Nk, cap, 128, 64, dtype=torch.uint8)
    meta = [torch.full((B, Nk, cap, 1, 64), float("nan"), dtype=torch.float16) for _ in range(4)]
    vcodes = torch.full((B, Nk, cap * 128, 16), -1, dtype=torch.int32)
    vmeta = [torch.full((B, Nk, cap * 128, 1), float("nan"), dtype=torch.float16) for _ in range(2)]
    kres = torch.full((B, Nk, 128, 128), float("nan"), dtype=torch.float16)
    vres = torch.full((B, Nk, 128, 128), float("nan"), dtype=torch.float16)
    mask = torch.ones(B, cap * 128 + 128, dtype=torch.uint8)
    refs = []
    for b in range(B):
        nb, nr = groups[b], resid[b]
        L = nb * 128 + nr
        k = wl.make_keys(1, Nk, L, 1e6, g)
        v = wl.make_half((1, Nk, L, 128), g)
        quant, vq = (None,) * 5, (None,) * 3
        if nb:
            quant = po.quantize_and_pack_nbit(k[:, :, :nb * 128].contiguous())
            vq = po.quantize_values_along_last_dim(v[:, :, :nb * 128].contiguous())
            codes[b, :, :nb] = quant[0][0]
            for m, t in zip(meta, quant[1:]):
                m[b, :, :nb] = t[0]
            vcodes[b, :, :nb * 128] = vq[0][0]
            for m, t in zip(vmeta, vq[1:]):
                m[b, :, :nb * 128] = t[0]
        kres[b, :, :nr], vres[b, :, :nr] = k[0, :, nb * 128:], v[0, :, nb * 128:]
        mb = torch.ones(1, L, dtype=torch.int64)
        mb[0, :min(5 * b, L - 1)] = 0
        mask[b, :L] = mb[0]
        refs.append(po.decode_attention_mixed_exact(q[b:b + 1], k[:, :, nb * 128:], *quant, v[:, :, nb * 128:], *vq, mb))
    dev = lambda t: t.to(gpu)
    for kw in (dict(), dict(n_splits=3), dict(n_splits=6, min_groups_per_split=2)):
        out = polar_decode_attention_v4(dev(q), dev(codes), *[dev(m) for m in meta], dev(kres), dev(vres), dev(vcodes),
                                        *[dev(m) for m in vmeta], 0, 0, attention_mask=dev(mask),
                                        n_groups_per_seq=torch.tensor(groups, dtype=torch.int32, device=gpu),
                                        n_resid_per_seq=torch.tensor(resid, dtype=torch.int32, device=gpu), **kw).cpu()
        assert torch.isfinite(out.float()).all()
        for b in range(B):
            nbad, emax = _close(out[b:b + 1], refs[b])
            assert nbad == 0, (kw, b, nbad, emax)


@pytest.mark.parametrize("values4", [True, False])
def test_attention_long_flat_tail_under_a_peak_is_not_dropped(gpu, values4):
    """One key scores 12.5 nats above 32767 others.  Each of those carries 3.7e-6 of the peak's
    weight, together 12 % of the mass: half-precision weights must keep them (the reference's
    half-precision probabilities do), which shows in a value channel with a non-zero mean."""
    g = torch.Generator().manual_seed(91)
    B, N, Nk, nb = 1, 4, 1, 256
    L = nb * 128
    u = torch.randn(128, generator=g)
    u = u / u.norm()
    k = (0.01 * torch.randn(B, Nk, L + 1, 128, generator=g)).half()
    k[0, 0, 20000] = (12.5 * math.sqrt(128) / 10.0 * u).half()
    q = (10.0 * u).half().expand(B, N, 1, 128).contiguous()
    v = wl.make_half((B, Nk, L + 1, 128), g)
    v[..., 5] += 2.0
    v[0, 0, 20000, 5] = -3.0                          # the peak's own value is far from the tail's mean
    quant = po.quantize_and_pack_nbit(k[:, :, :L].contiguous())
    kres, vres = k[:, :, L:].contiguous(), v[:, :, L:].contiguous()
    dq = [t.to(gpu) for t in quant]
    if values4:
        vq = po.quantize_values_along_last_dim(v[:, :, :L].contiguous())
        ref64 = po.decode_attention_mixed_exact(q, kres, *quant, vres, *vq)
        dk = torch.zeros(B, Nk, 128, 128, dtype=torch.float16, device=gpu)
        dv = torch.zeros_like(dk)
        dk[:, :, :1], dv[:, :, :1] = kres.to(gpu), vres.to(gpu)
        run = lambda ns: polar_decode_attention_v4(q.to(gpu), *dq, dk, dv, *[t.to(gpu) for t in vq], nb, 1, n_splits=ns)
    else:
        from polarquant_amd.attention import polar_decode_attention
        ref64 = po.decode_attention_exact(q, kres, *quant, v)
        run = lambda ns: polar_decode_attention(q.to(gpu), *dq, kres.to(gpu), v.to(gpu), nb, 1, n_splits=ns)
    # the tail really is a tenth of the mass: without it channel 5 would be off by ~0.5
    assert abs(ref64[0, 0, 0, 5].item() - (-3.0)) > 0.3
    for ns in (1, 16, 128):
        out = run(ns).cpu()
        nbad, emax = _close(out, ref64)
        print("flat tail, values4", values4, "n_splits", ns, "max abs err %.2e" % emax, flush=True)
        assert nbad == 0, (ns, nbad, emax)
