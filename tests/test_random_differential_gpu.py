"""Seeded random differential test: random batch / head / bit-width / length / mask / split
combinations of the fused decode attention, with half-precision or 4-bit values, uniform or
per-sequence lengths, against the fp64 oracle evaluated sequence by sequence."""
import os
import random

import pytest
import torch

from oracle import polar_oracle as po
from polarquant_amd import workloads as wl
from polarquant_amd.attention import polar_decode_attention, polar_decode_attention_v4

pytestmark = pytest.mark.gpu
# more seeds: PQ_RANDOM_CASES=300; another stretch of them: PQ_RANDOM_FIRST=1000
SEEDS = range(int(os.environ.get("PQ_RANDOM_FIRST", "0")),
              int(os.environ.get("PQ_RANDOM_FIRST", "0")) + int(os.environ.get("PQ_RANDOM_CASES", "24")))
HEADS = [(1, 1), (2, 1), (4, 4), (8, 2), (3, 1), (6, 1), (7, 1), (8, 1), (16, 2), (12, 4), (5, 1), (10, 2), (14, 2)]
BITS = [(4, 4), (3, 3), (4, 2), (5, 3), (2, 4), (3, 4), (3, 5), (2, 6), (1, 6)]
# dtype -> [attention cases run, cases that needed the widened band, output elements that needed it,
#           worst excess over the STATED bar (rtol 1e-2 / atol 1e-3) against the reference path's literal evaluation alone]
WIDENED = {n + v: [0, 0, 0, -1.0] for n in ("float16", "bfloat16") for v in ("", ", 4-bit values")}


@pytest.mark.parametrize("seed", SEEDS)
def test_random_decode_attention_case(gpu, seed):
    rnd = random.Random(1000 + seed)
    N, Nk = rnd.choice(HEADS)
    rb, tb = rnd.choice(BITS)
    B = rnd.randint(1, 4)
    dtype = torch.bfloat16 if seed % 6 == 5 else torch.float16
    values4 = rnd.random() < 0.5
    ragged = rnd.random() < 0.5
    cap = rnd.randint(1, 7)
    groups = [rnd.randint(0, cap) for _ in range(B)] if ragged else [rnd.randint(0, cap)] * B
    resid = [rnd.randint(1, 128) for _ in range(B)] if ragged else [rnd.randint(1, 128)] * B
    use_mask = rnd.random() < 0.4
    n_splits = rnd.choice([None, 1, 2, 3, 5])
    # further draws from a generator of their own, so that the cases above stay what they were for every seed:
    # 3/3-bit codes stored as packed 6-bit rows; slices cut on the device also where a split count is given
    rnd2 = random.Random(77000 + seed)
    if rnd2.random() < 0.06:
        rb, tb = 1, 7                       # 128 angle bins (more than four heads per KV head: two launches)
    packed = (rb, tb) == (3, 3) and rnd2.random() < 0.5
    balanced = True if (ragged and n_splits is not None and n_splits >= 2 and rnd2.random() < 0.5) else None
    print("case", dict(seed=seed, N=N, Nk=Nk, bits=(rb, tb), B=B, dtype=str(dtype), values4=values4, groups=groups,
                       resid=resid, mask=use_mask, n_splits=n_splits, packed=packed, balanced=balanced), flush=True)
    g = torch.Generator().manual_seed(seed)
    q = wl.make_half((B, N, 1, 128), g, dtype)
    codes = torch.zeros(B, Nk, cap, 128, 64, dtype=torch.uint8)
    meta = [torch.zeros(B, Nk, cap, 1, 64, dtype=dtype) for _ in range(4)]
    vcodes = torch.zeros(B, Nk, cap * 128, 16, dtype=torch.int32)
    vmeta = [torch.zeros(B, Nk, cap * 128, 1, dtype=dtype) for _ in range(2)]
    kres = torch.zeros(B, Nk, 128, 128, dtype=dtype)
    vres = torch.zeros(B, Nk, 128, 128, dtype=dtype)
    vfull = torch.zeros(B, Nk, cap * 128 + 128, 128, dtype=dtype)
    mask = torch.ones(B, cap * 128 + 128, dtype=torch.uint8)
    refs = []
    for b in range(B):
        nb, nr = groups[b], resid[b]
        L = nb * 128 + nr
        k = wl.make_keys(1, Nk, L, 5e5, g, dtype)
        v = wl.make_half((1, Nk, L, 128), g, dtype)
        v[..., 3] += 1.5
        quant, vq = (None,) * 5, (None,) * 3
        if nb:
            quant = po.quantize_and_pack_nbit(k[:, :, :nb * 128].contiguous(), rb, tb)
            codes[b, :, :nb] = quant[0][0]
            for m, t in zip(meta, quant[1:]):
                m[b, :, :nb] = t[0]
            if values4:
                vq = po.quantize_values_along_last_dim(v[:, :, :nb * 128].contiguous())
                vcodes[b, :, :nb * 128] = vq[0][0]
                for m, t in zip(vmeta, vq[1:]):
                    m[b, :, :nb * 128] = t[0]
        kres[b, :, :nr], vres[b, :, :nr] = k[0, :, nb * 128:], v[0, :, nb * 128:]
        vfull[b, :, :L] = v[0]
        mb = None
        if use_mask:
            mb = torch.ones(1, L, dtype=torch.int64)
            mb[0, :rnd.randint(0, L - 1)] = 0
            mask[b, :L] = mb[0]
        kr, vr = k[:, :, nb * 128:], v[:, :, nb * 128:]
        if values4:
            exact = po.decode_attention_mixed_exact(q[b:b + 1], kr, *quant, vr, *vq, mb, rb, tb)
            literal = po.decode_attention_mixed(q[b:b + 1], kr, *quant, vr, *vq, mb, rb, tb)
        else:
            exact = po.decode_attention_exact(q[b:b + 1], kr, *quant, v, mb, rb, tb)
            literal = po.decode_attention(q[b:b + 1], kr, *quant, v, mb, rb, tb)
        # what the reference path's own roundings can move: the distance of its half-precision evaluation
        # from the exact one, and the first-order bound for its rounding of the window's scores (:79)
        v_all = v if not values4 else (vr if not nb else torch.cat([po.dequantize_values(*vq, 4, torch.float64), vr.double()], dim=2))
        band = po.residual_score_rounding_band(q[b:b + 1], kr, *quant, v_all, mb, rb, tb)
        refs.append((exact, torch.maximum((literal.double() - exact).abs(), band), literal.double()))
    dev = lambda t: t.to(gpu)
    kw = dict(rbits=rb, tbits=tb, n_splits=n_splits, attention_mask=dev(mask) if use_mask else None)
    if ragged:
        kw.update(n_groups_per_seq=torch.tensor(groups, dtype=torch.int32, device=gpu),
                  n_resid_per_seq=torch.tensor(resid, dtype=torch.int32, device=gpu))
        ng, nr = 0, 0
    else:
        ng, nr = groups[0], resid[0]
    have_groups = any(groups) or ragged
    cq = [dev(po.pack_codes6(codes) if packed else codes)] + [dev(m) for m in meta] if have_groups else [None] * 5
    # every call gets a status word: no hand-over between a scorer and its accumulator may ever give up
    status = torch.zeros(1, dtype=torch.int32, device=gpu)
    kw.update(status=status)
    if balanced:
        kw.update(balanced=True)
    if values4:
        vq_d = [dev(vcodes)] + [dev(m) for m in vmeta] if have_groups else [None] * 3
        out = polar_decode_attention_v4(dev(q), *cq, dev(kres), dev(vres), *vq_d, ng, nr, single_wavefront=seed % 4 == 3, **kw)
    else:
        # one case in four takes the one-wavefront-per-slice kernels instead of the scorer / accumulator pairs
        out = polar_decode_attention(dev(q), *cq, dev(kres), dev(vfull), ng, nr, single_wavefront=seed % 4 == 3, **kw)
    out = out.cpu()
    assert int(status) == 0
    assert torch.isfinite(out.float()).all()
    # the band is centred on the fp64 value and widened, element by element, by the distance of the
    # reference path's own half-precision evaluation from it (scores of the residual window and
    # probabilities rounded to the dtype matter when only a few dozen tokens are attended to)
    rtol, atol = (1e-2, 1e-3) if dtype == torch.float16 else (2e-2, 4e-3)
    name = ("float16" if dtype == torch.float16 else "bfloat16") + (", 4-bit values" if values4 else "")
    needed = 0
    for b in range(B):
        exact, ref_noise, literal = refs[b]
        err = (out[b:b + 1].double() - exact).abs()
        over = err - (atol + rtol * exact.abs() + ref_noise)
        bad = int((over > 0).sum())
        worst = int(over.argmax())
        assert bad == 0, (b, bad, float(err.max()), "worst element: got %r exact %r reference-path noise %r" % (
            float(out[b:b + 1].double().flatten()[worst]), float(exact.flatten()[worst]), float(ref_noise.flatten()[worst])))
        # elements that meet the plain tolerance neither against the exact value nor against the reference path's own
        # (literal, half-precision) evaluation, which is what parity is stated against
        err_lit = (out[b:b + 1].double() - literal).abs()
        both = (err > atol + rtol * exact.abs()) & (err_lit > atol + rtol * literal.abs())
        needed += int(both.sum())
        if bool(both.any()):
            i = int(torch.where(both.flatten(), torch.minimum(err - (atol + rtol * exact.abs()),
                                                             err_lit - (atol + rtol * literal.abs())).flatten(),
                                torch.full_like(err.flatten(), -1.0)).argmax())
            print("element outside the plain tolerance against both evaluations: sequence %d index %d got %.6f fp64 %.6f "
                  "literal %.6f band %.3e" % (b, i, float(out[b:b + 1].double().flatten()[i]), float(exact.flatten()[i]),
                                              float(literal.flatten()[i]), float(ref_noise.flatten()[i])), flush=True)
        # how far the output sits from the literal reference evaluation alone, in the stated (float16) bar: > 0 means
        # outside it.  For bfloat16 this is the measured size of the band that dtype needs, instead of a choice.
        WIDENED[name][3] = max(WIDENED[name][3], float((err_lit - (1e-3 + 1e-2 * literal.abs())).max()))
    WIDENED[name][0] += 1
    WIDENED[name][1] += int(needed > 0)
    WIDENED[name][2] += needed
    # How often the widening is needed is counted, printed (test_random_widened_band_report) and bounded there as a
    # rate, not asserted case by case: the reference rounds the window's scores to the dtype (:79), so does the kernel,
    # and where the two fp32 sums behind such a score differ in their last bits the rounding can go the other way.  On an
    # output that is the remainder of a few large cancelling terms (a mask that leaves a handful of tokens) that moves one
    # element in about 10^7 a few 1e-4 outside both plain bands: 1 float16 element in 15 600 cases with half-precision values,
    # 1 in 15 200 with 4-bit values, 8 bfloat16 elements in 6 200 cases (seeds 220400-257337).


def test_random_widened_band_report(gpu):
    """How many of the attention cases above were inside the stated tolerance only thanks to the allowance for the
    reference path's own half-precision roundings: printed per dtype and value kind.  A kernel whose results leaned on
    the allowance as a matter of course would show here: at most one case in a hundred may need it."""
    for name, (cases, cases_needing, elements, excess) in WIDENED.items():
        print("%s: %d cases, %d needed the widened band (%d output elements); worst excess over rtol 1e-2 / atol 1e-3 against "
              "the literal reference evaluation alone: %.3e" % (name, cases, cases_needing, elements, excess), flush=True)
        assert cases_needing * 100 <= max(cases, 100), name


@pytest.mark.parametrize("seed", SEEDS)
def test_random_quantizer_case(gpu, seed):
    """Key and value quantizers, bit for bit against the oracle, on keys / values of random scale
    (1e-6 .. 1e4), distribution (normal, heavy-tailed, sparse, nearly constant) and bit widths."""
    from polarquant_amd.quantize import quantize_and_pack_nbit
    from polarquant_amd.values import quantize_values
    rnd = random.Random(5000 + seed)
    dtype = torch.bfloat16 if seed % 3 == 2 else torch.float16
    rb, tb = rnd.choice(BITS)
    if random.Random(78000 + seed).random() < 0.06:
        rb, tb = 1, 7
    mode = rnd.choice(["group", "group", "uniform"])
    scale = 10.0 ** rnd.uniform(-6, 4 if dtype == torch.bfloat16 else 3.5)
    kind = rnd.choice(["normal", "cauchy", "sparse", "flat"])
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(2, 2, 256, 128, generator=g)
    if kind == "cauchy":
        x = x / torch.randn(2, 2, 256, 128, generator=g).abs().clamp_min(1e-3)
    elif kind == "sparse":
        x = x * (torch.rand(2, 2, 256, 128, generator=g) < 0.1)
    elif kind == "flat":
        x = 1.0 + 1e-3 * x
    x = (x * scale).clamp(-6e4, 6e4).to(dtype)
    print("case", dict(seed=seed, dtype=str(dtype), bits=(rb, tb), mode=mode, scale=scale, kind=kind), flush=True)
    ref = po.quantize_and_pack_nbit(x, rb, tb, angle_mode=mode)
    got = quantize_and_pack_nbit(x.to(gpu), rb, tb, angle_mode=mode)
    flips = int((got[0].cpu() != ref[0]).sum())
    assert flips == 0, "code flips: %d of %d" % (flips, ref[0].numel())
    for name, a, b in zip(["rscale", "rmn", "tscale", "tmn"], got[1:], ref[1:]):
        a, b = a.cpu().float(), b.float()
        assert bool(((a == b) | (a.isnan() & b.isnan())).all()), name
    if mode == "group":
        # the same keys in the mode that follows eager torch on GPU tensors, against eager torch ops on the device
        # (0/0 groups, undefined in the reference, are left out: their metadata must agree, their codes need not)
        from oracle.device_eager import quantize_and_pack_nbit_eager
        xd = x.to(gpu)
        dref = [t.cpu() for t in quantize_and_pack_nbit_eager(xd, rb, tb)]
        dgot = [t.cpu() for t in quantize_and_pack_nbit(xd, rb, tb, eager_gpu=True)]
        for name, a, b in zip(["rscale", "rmn", "tscale", "tmn"], dgot[1:], dref[1:]):
            a, b = a.float(), b.float()
            assert bool(((a == b) | (a.isnan() & b.isnan())).all()), "eager-GPU mode: " + name
        defined = (dref[1].float() > 0) & (dref[3].float() > 0) & dref[1].float().isfinite() & dref[3].float().isfinite()
        dflips = int(((dgot[0] != dref[0]) & defined).sum())
        assert dflips == 0, "eager-GPU mode: %d code flips against eager torch on the device" % dflips
    vref = po.quantize_values_along_last_dim(x)
    vgot = quantize_values(x.to(gpu))
    assert torch.equal(vgot[0].cpu(), vref[0]), "value code words differ: %d" % int((vgot[0].cpu() != vref[0]).sum())
    for name, a, b in zip(["scale", "mn"], vgot[1:], vref[1:]):
        a, b = a.cpu().float(), b.float()
        assert bool(((a == b) | (a.isnan() & b.isnan())).all()), name


@pytest.mark.parametrize("seed", SEEDS)
def test_random_scores_case(gpu, seed):
    """The score op on random heads / bit widths / group counts, with quantized keys or (as the reference's
    micro-benchmark does) arbitrary codes and randn metadata, byte-per-code or packed 6-bit rows."""
    from polarquant_amd.kernel4group import attention_decode_forward_triton_impl
    rnd = random.Random(9000 + seed)
    N, Nk = rnd.choice(HEADS)
    rb, tb = rnd.choice(BITS)
    if random.Random(79000 + seed).random() < 0.06:
        rb, tb = 1, 7
    B, Nb = rnd.randint(1, 3), rnd.randint(1, 6)
    dtype = torch.bfloat16 if seed % 4 == 3 else torch.float16
    synthetic = rnd.random() < 0.4
    packed = (rb, tb) == (3, 3) and rnd.random() < 0.6
    print("case", dict(seed=seed, N=N, Nk=Nk, bits=(rb, tb), B=B, Nb=Nb, dtype=str(dtype), synthetic=synthetic, packed=packed), flush=True)
    g = torch.Generator().manual_seed(seed)
    q = wl.make_half((B, N, 1, 128), g, dtype)
    if synthetic:
        codes = torch.randint(0, 1 << (rb + tb), (B, Nk, Nb, 128, 64), generator=g, dtype=torch.uint8)
        meta = [torch.randn(B, Nk, Nb, 1, 64, generator=g).to(dtype) for _ in range(4)]
        if rnd.random() < 0.5:
            meta[0][0, 0, 0, 0, :5] = 0
            meta[2][0, 0, 0, 0, 5:9] = 0
    else:
        quant = po.quantize_and_pack_nbit(wl.make_keys(B, Nk, Nb * 128, 5e5, g, dtype), rb, tb)
        codes, meta = quant[0], list(quant[1:])
    ref = po.decode_scores(q, codes, *meta, rbits=rb, tbits=tb, dtype=torch.float64)
    dev_codes = po.pack_codes6(codes) if packed else codes
    got = attention_decode_forward_triton_impl(q.to(gpu), dev_codes.to(gpu), *[m.to(gpu) for m in meta], rbits=rb, tbits=tb)
    assert got.shape == (B, N, 1, Nb * 128) and got.dtype == torch.float32
    got = got.double().cpu()
    # the per-pair table is built in fp32: error relative to the largest magnitude a row can reach
    bound = ref.abs().amax(-1, keepdim=True).clamp_min(1e-30)
    assert float(((got - ref).abs() / bound).max()) < 2e-5
