"""GPU parity of pq_decode_attn (through the C ABI) against the CPU oracle.

Bar: attention output within rtol 1e-2 / atol 1e-3 of the reference path
(fp16).  Two references are used: the literal restatement (half-rounded
softmax, as the reference computes) and an fp64 evaluation with no
intermediate rounding; the kernel must meet the bar against both.
"""
import math

import pytest
import torch

from oracle import polar_oracle as po
from polarquant_amd import workloads as wl
from polarquant_amd.attention import polar_decode_attention as _polar_decode_attention

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
RTOL, ATOL = 1e-2, 1e-3
# bfloat16 (the stated bar is for float16): rtol 2e-2 / atol 4e-3.  bfloat16 carries 8 significant bits against
# float16's 11: one rounding of a probability or of an output element is 2^-9 = 2e-3 relative, eight times float16's, and
# the reference path's own bfloat16 evaluation sits up to 5e-3 from the fp64 value at these shapes.  The band is the
# stated one widened by less than that factor (atol x4, rtol x2), plus, element by element, what the reference's
# rounding of the residual window's scores (:79) can move (po.residual_score_rounding_band).
BF16_RTOL, BF16_ATOL = 2e-2, 4e-3
_LAST = {}


def _close(got, ref, rtol=RTOL, atol=ATOL):
    got, ref = got.double(), ref.double()
    err = (got - ref).abs()
    bad = err > atol + rtol * ref.abs()
    return int(bad.sum()), float(err.max())


def _bf16_ok(out, ref, ref64):
    """bfloat16 outputs: every element within BF16_RTOL / BF16_ATOL of the fp64 value, widened by the reference's own
    rounding of the window's scores.  Also prints how far the output sits from the reference path's literal bfloat16
    evaluation ALONE, measured in the stated float16 bar (rtol 1e-2 / atol 1e-3): the worst excess over it."""
    o, r, r64 = out.double(), ref.double(), ref64.double()
    excess = ((o - r).abs() - (ATOL + RTOL * r.abs())).max()
    print("bf16: worst excess over rtol 1e-2 / atol 1e-3 against the literal reference evaluation alone: %.2e" % float(excess), flush=True)
    err = (o - r64).abs()
    return bool((err <= BF16_ATOL + BF16_RTOL * r64.abs() + _LAST["band"]).all()), float(err.max())


def _case(gpu, B, N, Nk, n_groups, n_resid, rbits, tbits, dtype, theta=5e5, mask_pad=0, seed=0, n_splits=None,
          caps=(0, 0, 0), workspace=None):
    g = torch.Generator().manual_seed(seed)
    L = n_groups * 128 + n_resid
    k = wl.make_keys(B, Nk, max(L, 1), theta, g, dtype)
    q = wl.make_half((B, N, 1, 128), g, dtype)
    v = wl.make_half((B, Nk, L, 128), g, dtype)
    quant = (None,) * 5
    if n_groups:
        quant = po.quantize_and_pack_nbit(k[:, :, :n_groups * 128].contiguous(), rbits, tbits)
    kres = k[:, :, n_groups * 128:L].contiguous() if n_resid else None
    mask = None
    if mask_pad:
        mask = torch.ones(B, L, dtype=torch.int64)
        for b in range(B):
            mask[b, :(mask_pad * (b + 1)) % L] = 0      # left padding, different per sequence
    ref = po.decode_attention(q, kres, *quant, v, mask, rbits, tbits)
    ref64 = po.decode_attention_exact(q, kres, *quant, v, mask, rbits, tbits)
    _LAST["band"] = po.residual_score_rounding_band(q, kres, *quant, v, mask, rbits, tbits)
    # device tensors, optionally with spare capacity behind the used part
    gc, rc, vc = caps
    dq = [None] * 5
    if n_groups:
        cap = n_groups + gc
        dq = [torch.zeros((B, Nk, cap) + tuple(t.shape[3:]), dtype=t.dtype, device=gpu) for t in quant]
        for d, t in zip(dq, quant):
            d[:, :, :n_groups] = t.to(gpu)
    dk = None
    if n_resid:
        dk = torch.zeros(B, Nk, n_resid + rc, 128, dtype=dtype, device=gpu)
        dk[:, :, :n_resid] = kres.to(gpu)
    dv = torch.zeros(B, Nk, L + vc, 128, dtype=dtype, device=gpu)
    dv[:, :, :L] = v.to(gpu)
    if vc:
        dv[:, :, L:] = float("nan")     # rows past the end must never contribute
    out = polar_decode_attention(q.to(gpu), *dq, dk, dv, n_groups, n_resid,
                                 attention_mask=None if mask is None else mask.to(gpu),
                                 rbits=rbits, tbits=tbits, n_splits=n_splits, workspace=workspace)
    torch.cuda.synchronize()
    out = out.cpu()
    assert out.shape == (B, N, 1, 128) and out.dtype == dtype
    assert torch.isfinite(out.float()).all()
    return out, ref, ref64


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("N,Nk,rbits,tbits", [(32, 8, 4, 4), (32, 32, 4, 4), (28, 4, 3, 3), (16, 8, 4, 4), (12, 2, 3, 3),
                                              # every head ratio has its own kernel: 3, 5, 6, 7 (and 7 with 16 bins)
                                              (12, 4, 4, 4), (10, 2, 4, 4), (12, 2, 4, 4), (7, 1, 4, 4), (14, 2, 2, 2),
                                              # more than 16 angle bins (the one-wavefront kernels in either form)
                                              (32, 8, 3, 5), (8, 1, 2, 6), (16, 4, 2, 6), (6, 2, 1, 6), (4, 4, 3, 5),
                                              # 128 angle bins: a table holds four heads, more heads per KV head go in two launches
                                              (8, 2, 1, 7), (3, 1, 1, 7), (8, 1, 1, 7), (14, 2, 1, 7), (10, 2, 1, 7)])
def test_attn_matches_oracle(gpu, dtype, N, Nk, rbits, tbits):
    print("case", dtype, N, Nk, rbits, tbits, flush=True)
    out, ref, ref64 = _case(gpu, 2, N, Nk, 6, 37, rbits, tbits, dtype, seed=1)
    if dtype == torch.bfloat16:
        ok, emax = _bf16_ok(out, ref, ref64)
        assert ok, emax
        return
    nbad, emax = _close(out, ref64)
    print("max err vs fp64", emax, flush=True)
    assert nbad == 0
    nbad, emax = _close(out, ref)
    assert nbad == 0


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_attn_largest_table(gpu, dtype):
    """8 heads per KV head with 16 angle bins: the largest table (32 KB per slice; 148 KB of LDS for a workgroup of four
    scorer / accumulator pairs).  (At this shape the reference path's own bfloat16 evaluation is up to 4.7e-3 away
    from the fp64 value.)"""
    out, ref, ref64 = _case(gpu, 2, 16, 2, 6, 37, 4, 4, dtype, seed=1)
    if dtype == torch.float16:
        assert _close(out, ref64)[0] == 0 and _close(out, ref)[0] == 0
    else:
        ok, emax = _bf16_ok(out, ref, ref64)
        assert ok, emax


@pytest.mark.parametrize("n_groups,n_resid", [(0, 1), (0, 64), (0, 128), (1, 0), (1, 1), (3, 127), (5, 128), (2, 65)])
def test_attn_residual_edges(gpu, n_groups, n_resid):
    """Empty quantized part, empty residual, full 128-token residual (the step before a flush)."""
    print("case", n_groups, n_resid, flush=True)
    out, ref, ref64 = _case(gpu, 2, 32, 8, n_groups, n_resid, 4, 4, torch.float16, seed=2)
    assert _close(out, ref64)[0] == 0 and _close(out, ref)[0] == 0


@pytest.mark.parametrize("n_splits", [1, 2, 3, 7, 16])
def test_attn_split_invariance(gpu, n_splits):
    out, ref, ref64 = _case(gpu, 1, 32, 8, 16, 5, 4, 4, torch.float16, seed=3, n_splits=n_splits)
    assert _close(out, ref64)[0] == 0


@pytest.mark.parametrize("N,Nk,rbits,tbits", [(7, 1, 1, 6), (8, 2, 3, 5), (4, 4, 2, 6)])
def test_attn_one_slice_per_plane_with_wide_angle_tables(gpu, N, Nk, rbits, tbits):
    """n_splits == 1 lets the paired kernels write the output themselves; angle widths above 4 bits run the
    one-wavefront kernels, which write a partial, so the merge has to follow (a call that skipped it returned
    whatever the output buffer held)."""
    print("case", N, Nk, rbits, tbits, flush=True)
    out, ref, ref64 = _case(gpu, 1, N, Nk, 3, 1, rbits, tbits, torch.float16, seed=81, n_splits=1)
    nbad, emax = _close(out, ref64)
    assert nbad == 0, emax


@pytest.mark.parametrize("n_splits,dtype", [(33, torch.float16), (70, torch.bfloat16), (130, torch.float16), (1030, torch.float16)])
def test_attn_many_splits(gpu, n_splits, dtype):
    """32 or more / 128 or more partials per head take the merge kernel's 4- and 8-group forms; more
    slices than groups leave empty partials, more than 1024 a second pass over the weight buffer."""
    print("case", n_splits, dtype, flush=True)
    out, ref, ref64 = _case(gpu, 1, 8, 2, 130, 3, 4, 4, dtype, seed=11, n_splits=n_splits)
    rtol, atol = (RTOL, ATOL) if dtype == torch.float16 else (2e-2, 4e-3)   # bf16 has 8 mantissa bits
    assert _close(out, ref64, rtol, atol)[0] == 0


@pytest.mark.parametrize("n_groups,n_splits", [(1, 2), (2, 3), (3, 2), (8, 4), (8, 8), (16, 16), (5, 7)])
def test_attn_slices_that_count_the_residual_keys(gpu, n_groups, n_splits):
    """A long residual window makes the plane's last slice the longest, so the even cut then weighs the residual
    keys and slices begin and end inside groups.  Every residual length around the weights' steps, against the
    oracle, with a workspace full of NaN so that a slot nobody wrote would show."""
    from polarquant_amd import attention
    for n_resid in (1, 42, 43, 64, 65, 85, 86, 127, 128):
        print("case", n_groups, n_splits, n_resid, flush=True)
        ws = attention.new_workspace(2, 8, n_splits, gpu)
        ws.fill_(float("nan"))
        out, ref, ref64 = _case(gpu, 2, 8, 2, n_groups, n_resid, 4, 4, torch.float16, seed=100 * n_groups + n_resid,
                                n_splits=n_splits, workspace=ws)
        # a short context whose window holds a good part of the softmax mass: the stated tolerance against the fp64
        # value or the reference path's own evaluation, else widened by what the reference's rounding of the window's
        # scores can move (as in the random differential test)
        o, r, r64 = out.double(), ref.double(), ref64.double()
        e64, el = (o - r64).abs(), (o - r).abs()
        bad = (e64 > ATOL + RTOL * r64.abs()) & (el > ATOL + RTOL * r.abs()) & (e64 > ATOL + RTOL * r64.abs() + _LAST["band"])
        assert int(bad.sum()) == 0, (n_resid, float(e64.max()))


@pytest.mark.parametrize("poison", [float("nan"), float("inf"), -1.0])
def test_attn_ignores_what_the_workspace_held(gpu, poison):
    """The workspace is never cleared, and slices past a sequence's last group write only an empty
    header: whatever bits the buffer held before (NaN, Inf, integer -1 patterns from other tensors
    that owned the memory) must not reach the output.  More slices than groups, and a ragged batch
    whose short sequences leave most slices empty, both through a caller-owned and the cached buffer."""
    from polarquant_amd import attention
    print("case poison", poison, flush=True)
    ws = attention.new_workspace(1, 8, 9, gpu)
    if poison < 0:
        ws.view(torch.int32).fill_(-1)
    else:
        ws.fill_(poison)
    out, ref, ref64 = _case(gpu, 1, 8, 2, 4, 3, 4, 4, torch.float16, seed=21, n_splits=9, workspace=ws)
    assert _close(out, ref64)[0] == 0
    # ragged: sequences of 1 and 5 groups cut into 5 slices; the cached buffer of the current stream is poisoned
    g = torch.Generator().manual_seed(22)
    B, N, Nk = 2, 8, 2
    lens = [1 * 128 + 7, 5 * 128]
    k = wl.make_keys(B, Nk, max(lens), 5e5, g)
    q = wl.make_half((B, N, 1, 128), g)
    v = wl.make_half((B, Nk, max(lens), 128), g)
    codes = torch.zeros(B, Nk, 5, 128, 64, dtype=torch.uint8)
    meta = [torch.zeros(B, Nk, 5, 1, 64, dtype=torch.float16) for _ in range(4)]
    kres = torch.zeros(B, Nk, 128, 128, dtype=torch.float16)
    refs = []
    for b, L in enumerate(lens):
        ng, nr = L // 128, L % 128
        quant = po.quantize_and_pack_nbit(k[b:b + 1, :, :ng * 128].contiguous())
        codes[b, :, :ng] = quant[0][0]
        for m, t in zip(meta, quant[1:]):
            m[b, :, :ng] = t[0]
        kr = k[b:b + 1, :, ng * 128:L].contiguous() if nr else None
        if nr:
            kres[b, :, :nr] = kr[0]
        refs.append(po.decode_attention_exact(q[b:b + 1], kr, *quant, v[b:b + 1, :, :L]))
    cached = attention.workspace_for(B, N, 5, gpu)
    if poison < 0:
        cached.view(torch.int32).fill_(-1)
    else:
        cached.fill_(poison)
    out = polar_decode_attention(q.to(gpu), codes.to(gpu), *[m.to(gpu) for m in meta], kres.to(gpu), v.to(gpu), 0, 0,
                                 n_groups_per_seq=torch.tensor([1, 5], dtype=torch.int32, device=gpu),
                                 n_resid_per_seq=torch.tensor([7, 0], dtype=torch.int32, device=gpu), n_splits=5)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()
    assert _close(out.cpu(), torch.cat(refs, 0))[0] == 0


def test_attn_left_padding_mask(gpu):
    out, ref, ref64 = _case(gpu, 3, 32, 8, 4, 19, 4, 4, torch.float16, seed=4, mask_pad=150)
    assert _close(out, ref64)[0] == 0 and _close(out, ref)[0] == 0


def test_attn_spare_capacity(gpu):
    """Cache tensors larger than the used part (pre-allocated arena); unused V rows hold NaN."""
    out, ref, ref64 = _case(gpu, 2, 32, 8, 3, 40, 4, 4, torch.float16, seed=5, caps=(5, 88, 300))
    assert _close(out, ref64)[0] == 0


def test_attn_ragged_lengths(gpu):
    """Per-sequence context lengths (continuous batching): groups and residual counts per sequence."""
    g = torch.Generator().manual_seed(8)
    B, N, Nk, rb, tb = 6, 28, 4, 3, 3
    lens = torch.tensor([129, 512, 700, 1023, 128, 77])
    Lmax = int(lens.max())
    k = wl.make_keys(B, Nk, Lmax, 1e6, g)
    q = wl.make_half((B, N, 1, 128), g)
    v = wl.make_half((B, Nk, Lmax, 128), g)
    gcap = Lmax // 128
    codes = torch.zeros(B, Nk, gcap, 128, 64, dtype=torch.uint8)
    meta = [torch.zeros(B, Nk, gcap, 1, 64, dtype=torch.float16) for _ in range(4)]
    kres = torch.zeros(B, Nk, 128, 128, dtype=torch.float16)
    refs = []
    for b in range(B):
        L = int(lens[b]); ng, nr = L // 128, L % 128
        quant = (None,) * 5
        if ng:
            quant = po.quantize_and_pack_nbit(k[b:b + 1, :, :ng * 128].contiguous(), rb, tb)
            codes[b, :, :ng] = quant[0][0]
            for m, t in zip(meta, quant[1:]):
                m[b, :, :ng] = t[0]
        kr = k[b:b + 1, :, ng * 128:L].contiguous() if nr else None
        if nr:
            kres[b, :, :nr] = kr[0]
        refs.append(po.decode_attention_exact(q[b:b + 1], kr, *quant, v[b:b + 1, :, :L], None, rb, tb))
    ref64 = torch.cat(refs, 0)
    out = polar_decode_attention(q.to(gpu), codes.to(gpu), *[m.to(gpu) for m in meta], kres.to(gpu), v.to(gpu),
                                 0, 0, rbits=rb, tbits=tb,
                                 n_groups_per_seq=(lens // 128).int().to(gpu), n_resid_per_seq=(lens % 128).int().to(gpu),
                                 n_splits=3)
    torch.cuda.synchronize()
    assert _close(out.cpu(), ref64)[0] == 0


def test_attn_sharp_softmax(gpu):
    """A query aligned with one key: the softmax is dominated by a single token
    whose score is far above the rest, in a late tile (exercises the lazy rescale)."""
    g = torch.Generator().manual_seed(12)
    B, N, Nk, ng = 1, 32, 8, 8
    L = ng * 128 + 3
    k = wl.make_keys(B, Nk, L, 5e5, g)
    v = wl.make_half((B, Nk, L, 128), g)
    q = wl.make_half((B, N, 1, 128), g)
    for h in range(N):
        q[0, h, 0] = (k[0, h // 4, 700 + h] * 1.5).half()
    quant = po.quantize_and_pack_nbit(k[:, :, :ng * 128].contiguous())
    kres = k[:, :, ng * 128:].contiguous()
    ref64 = po.decode_attention_exact(q, kres, *quant, v)
    out = polar_decode_attention(q.to(gpu), *[t.to(gpu) for t in quant], kres.to(gpu), v.to(gpu), ng, 3, n_splits=2)
    assert _close(out.cpu(), ref64)[0] == 0


def test_attn_empty_and_fully_masked_sequences(gpu):
    """A ragged batch may hold a sequence with no cached token at all, and a mask may hide every
    token of a sequence: both have nothing to attend to and must yield zeros (no NaN from 0/0),
    without disturbing their neighbours."""
    g = torch.Generator().manual_seed(14)
    B, N, Nk = 3, 8, 2
    L = 2 * 128 + 9
    k = wl.make_keys(B, Nk, L, 5e5, g)
    q = wl.make_half((B, N, 1, 128), g)
    v = wl.make_half((B, Nk, L, 128), g)
    quant = po.quantize_and_pack_nbit(k[:, :, :256].contiguous())
    kres = torch.zeros(B, Nk, 128, 128, dtype=torch.float16)
    kres[:, :, :9] = k[:, :, 256:]
    groups = torch.tensor([2, 0, 2], dtype=torch.int32)
    resid = torch.tensor([9, 0, 9], dtype=torch.int32)           # sequence 1 is empty
    mask = torch.ones(B, L, dtype=torch.uint8)
    mask[2] = 0                                                  # sequence 2 is masked out entirely
    out = polar_decode_attention(q.to(gpu), *[t.to(gpu) for t in quant], kres.to(gpu), v.to(gpu), 0, 0,
                                 attention_mask=mask.to(gpu), n_groups_per_seq=groups.to(gpu),
                                 n_resid_per_seq=resid.to(gpu), n_splits=2).cpu()
    assert torch.isfinite(out.float()).all()
    assert bool((out[1] == 0).all()) and bool((out[2] == 0).all())
    ref = po.decode_attention_exact(q[:1], k[:1, :, 256:], *[t[:1] for t in quant], v[:1])
    assert _close(out[:1], ref)[0] == 0
