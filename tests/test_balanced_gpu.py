"""PQ_BALANCED_SLICES: context slices cut on the device from the per-sequence counts.  The result may differ
from the even split only by fp32 summation order, so every case is held to the stated bar against the fp64 oracle
(rtol 1e-2 / atol 1e-3) and to a tight band against the even split of the same inputs."""
import random

import pytest
import torch

from oracle import polar_oracle as po
from polarquant_amd import attention
from polarquant_amd import workloads as wl
from polarquant_amd.attention import polar_decode_attention as _polar_decode_attention
from polarquant_amd.attention import polar_decode_attention_v4

pytestmark = pytest.mark.gpu


# Every test of this file runs twice: with the default kernels (a scorer / accumulator pair of wavefronts per slice)
# and with one wavefront per slice (PQ_SINGLE_WAVEFRONT).
_FORM = {"single": False}


@pytest.fixture(autouse=True, params=[False, True], ids=["pairs", "single"])
def _kernel_form(request):
    _FORM["single"] = request.param
    yield
    _FORM["single"] = False


def polar_decode_attention(*args, **kwargs):
    return _polar_decode_attention(*args, single_wavefront=_FORM["single"], **kwargs)


def _ragged(gpu, B, N, Nk, lens, rb, tb, dtype, seed, gcap_extra=0, mask=False):
    """-> device inputs of a ragged batch and the fp64 oracle's output, sequence by sequence."""
    g = torch.Generator().manual_seed(seed)
    Lmax = max(max(lens), 1)
    gcap = max(Lmax // 128, 1) + gcap_extra
    k = wl.make_keys(B, Nk, Lmax, 1e6, g, dtype)
    q = wl.make_half((B, N, 1, 128), g, dtype)
    v = wl.make_half((B, Nk, Lmax, 128), g, dtype)
    codes = torch.zeros(B, Nk, gcap, 128, 64, dtype=torch.uint8)
    meta = [torch.zeros(B, Nk, gcap, 1, 64, dtype=dtype) for _ in range(4)]
    kres = torch.zeros(B, Nk, 128, 128, dtype=dtype)
    m = torch.ones(B, Lmax, dtype=torch.uint8) if mask else None
    refs, lits = [], []
    for b, L in enumerate(lens):
        ng, nr = L // 128, L % 128
        quant = (None,) * 5
        if ng:
            quant = po.quantize_and_pack_nbit(k[b:b + 1, :, :ng * 128].contiguous(), rb, tb)
            codes[b, :, :ng] = quant[0][0]
            for d, t in zip(meta, quant[1:]):
                d[b, :, :ng] = t[0]
        kr = k[b:b + 1, :, ng * 128:L].contiguous() if nr else None
        if nr:
            kres[b, :, :nr] = kr[0]
        mb = None
        if mask and L > 1:
            m[b, :(37 * (b + 1)) % L] = 0
            mb = m[b:b + 1, :L].long()
        if L == 0:
            refs.append(torch.zeros(1, N, 1, 128, dtype=torch.float64))
            lits.append(torch.zeros(1, N, 1, 128, dtype=torch.float64))
        else:
            refs.append(po.decode_attention_exact(q[b:b + 1], kr, *quant, v[b:b + 1, :, :L], mb, rb, tb))
            lits.append(po.residual_score_rounding_band(q[b:b + 1], kr, *quant, v[b:b + 1, :, :L], mb, rb, tb))
    dev = dict(q=q.to(gpu), codes=codes.to(gpu), meta=[t.to(gpu) for t in meta], kres=kres.to(gpu), v=v.to(gpu),
               groups=torch.tensor([L // 128 for L in lens], dtype=torch.int32, device=gpu),
               resid=torch.tensor([L % 128 for L in lens], dtype=torch.int32, device=gpu),
               mask=None if m is None else m.to(gpu))
    # element by element, how far the reference's own rounding of the residual window's scores to the model dtype (:79) can
    # move the output (to first order): nothing for a sequence without residual keys, most for one that is only a window long
    dev["literal"] = torch.cat(lits, 0)
    return dev, torch.cat(refs, 0)


def _run(d, rb, tb, **kw):
    out = polar_decode_attention(d["q"], d["codes"], *d["meta"], d["kres"], d["v"], 0, 0, rbits=rb, tbits=tb,
                                 attention_mask=d["mask"], n_groups_per_seq=d["groups"], n_resid_per_seq=d["resid"], **kw)
    torch.cuda.synchronize()
    return out.cpu()


def _within(got, ref, rtol=1e-2, atol=1e-3, literal=None):
    """Every element within the tolerance of the fp64 value.  `literal`: the band of
    po.residual_score_rounding_band, which widens the tolerance element by element by exactly what the reference's own
    rounding of the residual window's scores to the model dtype (:79) can move: parity is stated against the reference
    path, whose scores of un-quantized keys carry that rounding.  One band, centred on the fp64 value, for every plane."""
    ref = ref.double().reshape(got.shape)
    err = (got.double() - ref).abs()
    tol = atol + rtol * ref.abs()
    if literal is not None:
        tol = tol + literal.double().reshape(got.shape)
    return bool((err <= tol).all()), float(err.max())


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("N,Nk,rb,tb", [(28, 4, 3, 3), (32, 8, 4, 4), (8, 8, 4, 4), (6, 1, 4, 2)])
def test_balanced_slices_match_the_oracle_and_the_even_split(gpu, dtype, N, Nk, rb, tb):
    lens = [129, 512, 700, 1023, 128, 77, 0, 1, 2048, 64, 127, 900]       # whole groups only, window only, empty, one token
    print("case", dtype, N, Nk, rb, tb, flush=True)
    d, ref = _ragged(gpu, len(lens), N, Nk, lens, rb, tb, dtype, seed=31, gcap_extra=2, mask=True)
    rtol, atol = (1e-2, 1e-3) if dtype == torch.float16 else (2e-2, 4e-3)
    even = _run(d, rb, tb, n_splits=4, balanced=False)
    for kw in (dict(), dict(n_splits=2), dict(n_splits=3), dict(n_splits=7), dict(n_splits=40), dict(n_splits=5, min_groups_per_split=3)):
        got = _run(d, rb, tb, balanced=True, **kw)
        assert torch.isfinite(got.float()).all(), kw
        ok, err = _within(got, ref, rtol, atol, literal=d["literal"])
        assert ok, (kw, err)
        ok, err = _within(got, even, 2e-3 if dtype == torch.float16 else 1.6e-2, 1e-3 if dtype == torch.float16 else 8e-3)   # one output ulp at |x| < 2
        assert ok, ("against the even split", kw, err)
    assert bool((even[6] == 0).all()) and bool((got[6] == 0).all())        # the empty sequence


def test_balanced_slices_ignore_what_the_workspace_held(gpu):
    """Slots behind a plane's last piece, and all slots of planes shorter than a segment, are marked empty by the
    kernel itself; the buffer's earlier contents (NaN here) must not reach the output."""
    lens = [300, 4000, 130, 5, 2600]
    d, ref = _ragged(gpu, len(lens), 8, 2, lens, 4, 4, torch.float16, seed=32)
    for ns in (3, 9, 33):
        ws = attention.new_workspace(len(lens), 8, ns, gpu)
        ws.fill_(float("nan"))
        got = _run(d, 4, 4, balanced=True, n_splits=ns, workspace=ws)
        assert torch.isfinite(got.float()).all(), ns
        ok, err = _within(got, ref, literal=d["literal"])
        assert ok, (ns, err)


def test_balanced_slices_with_uniform_counts_and_4bit_values(gpu):
    """The flag also takes uniform counts (no per-sequence arrays), and the 4-bit-value entry point."""
    from polarquant_amd.values import quantize_values
    g = torch.Generator().manual_seed(33)
    B, N, Nk, ng, nr = 3, 16, 4, 9, 50
    L = ng * 128 + nr
    k = wl.make_keys(B, Nk, L, 5e5, g)
    q = wl.make_half((B, N, 1, 128), g)
    v = wl.make_half((B, Nk, L, 128), g)
    quant = po.quantize_and_pack_nbit(k[:, :, :ng * 128].contiguous())
    kres = k[:, :, ng * 128:].contiguous()
    ref = po.decode_attention_exact(q, kres, *quant, v)
    dq = [t.to(gpu) for t in quant]
    for ns in (None, 2, 6):
        got = polar_decode_attention(q.to(gpu), *dq, kres.to(gpu), v.to(gpu), ng, nr, balanced=True, n_splits=ns).cpu()
        ok, err = _within(got, ref)
        assert ok, (ns, err)
    vq_ref = po.quantize_values_along_last_dim(v[:, :, :ng * 128].contiguous())
    ref4 = po.decode_attention_mixed_exact(q, kres, *quant, v[:, :, ng * 128:], *vq_ref)
    vq = quantize_values(v[:, :, :ng * 128].to(gpu))
    kr_d = torch.zeros(B, Nk, 128, 128, dtype=torch.float16, device=gpu)
    vr_d = torch.zeros_like(kr_d)
    kr_d[:, :, :nr], vr_d[:, :, :nr] = kres.to(gpu), v[:, :, ng * 128:].to(gpu)
    for ns in (None, 3):
        got = polar_decode_attention_v4(q.to(gpu), *dq, kr_d, vr_d, *vq, ng, nr, balanced=True, n_splits=ns).cpu()
        ok, err = _within(got, ref4)
        assert ok, ("4-bit values", ns, err)


@pytest.mark.parametrize("seed", range(12))
def test_balanced_slices_random_batches(gpu, seed):
    rnd = random.Random(700 + seed)
    B = rnd.randint(1, 70)
    N, Nk = rnd.choice([(28, 4), (32, 8), (4, 4), (7, 1), (16, 2)])
    rb, tb = rnd.choice([(4, 4), (3, 3), (4, 2)])
    lens = [rnd.choice([0, 1, rnd.randint(1, 127), rnd.randint(128, 3000), rnd.randint(128, 3000)]) for _ in range(B)]
    ns = rnd.choice([None, 2, 3, 8, 25])
    print("case", dict(seed=seed, B=B, N=N, Nk=Nk, bits=(rb, tb), n_splits=ns, lens=lens[:8]), flush=True)
    d, ref = _ragged(gpu, B, N, Nk, lens, rb, tb, torch.float16, seed=seed, mask=rnd.random() < 0.3)
    got = _run(d, rb, tb, balanced=True, n_splits=ns)
    assert torch.isfinite(got.float()).all()
    ok, err = _within(got, ref, literal=d["literal"])
    assert ok, err


def test_balanced_slices_with_a_long_residual_window(gpu):
    """The interface takes any residual capacity, not only the reference's 128: a window of 300 keys is five tiles of
    a plane's line, and the slot bound has to count them (2 slots: every plane is cut at most once)."""
    g = torch.Generator().manual_seed(35)
    B, N, Nk, ng = 3, 8, 2, 2
    lens_res = [300, 17, 129]
    k = wl.make_keys(B, Nk, ng * 128 + 300, 5e5, g)
    q = wl.make_half((B, N, 1, 128), g)
    v = wl.make_half((B, Nk, ng * 128 + 300, 128), g)
    quant = po.quantize_and_pack_nbit(k[:, :, :ng * 128].contiguous())
    kres = torch.zeros(B, Nk, 300, 128, dtype=torch.float16)
    refs = []
    for b, nr in enumerate(lens_res):
        kres[b, :, :nr] = k[b, :, ng * 128:ng * 128 + nr]
        refs.append(po.decode_attention(q[b:b + 1], k[b:b + 1, :, ng * 128:ng * 128 + nr].contiguous(), *[t[b:b + 1] for t in quant],
                                        v[b:b + 1, :, :ng * 128 + nr]).double())
    ref = torch.cat(refs, 0)
    for ns in (2, 3, 7):
        got = polar_decode_attention(q.to(gpu), *[t.to(gpu) for t in quant], kres.to(gpu), v.to(gpu), 0, 0, balanced=True, n_splits=ns,
                                     n_groups_per_seq=torch.full((B,), ng, dtype=torch.int32, device=gpu),
                                     n_resid_per_seq=torch.tensor(lens_res, dtype=torch.int32, device=gpu)).cpu()
        ok, err = _within(got, ref)
        assert ok, (ns, err)
