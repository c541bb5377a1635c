"""Pins for the CPU oracle (oracle/polar_oracle.py, oracle/polar_oracle.c).

The reference ships no tests, fixtures or golden vectors for this path, so every
pin here is built from what the mathematics fixes: closed-form known answers,
invariants of min/max quantization, error bounds, brute force in fp64 / pure
python, library routines (torch.matmul, torch.softmax, HF rotate_half), and the
agreement of two independent restatements (torch vs plain C).  None of the checks
retypes the oracle's own formula.
"""
import math

import pytest
import torch

from oracle import c_oracle as co
from oracle import polar_oracle as po
from polarquant_amd import workloads as wl


def _keys(B, Nk, L, seed, dtype=torch.float16, theta=1e4):
    g = torch.Generator().manual_seed(seed)
    return wl.make_keys(B, Nk, L, theta, g, dtype), g


# ------------------------------------------------------------------ quantizer
def test_quantizer_known_answer_group():
    """Keys placed on exact bin centres: the codes are known in closed form.
    Pair d of token i is r_i (cos a_i, sin a_i) with a_i = a0 + (k_i + 0.5) * w, r_i = r0 + (m_i + 0.5) * u,
    plus two tokens pinning the range ends; fp16 rounding of x, y moves the angle by ~1e-3 rad,
    far less than half a bin."""
    tb, rb = 4, 4
    G, D = 128, 64
    a0, a1, r0, r1 = 0.5, 2.5, 1.0, 3.0
    w, u = (a1 - a0) / 2 ** tb, (r1 - r0) / 2 ** rb
    g = torch.Generator().manual_seed(0)
    kk = torch.randint(0, 2 ** tb, (G, D), generator=g)
    mm = torch.randint(0, 2 ** rb, (G, D), generator=g)
    ang = a0 + (kk.double() + 0.5) * w
    rad = r0 + (mm.double() + 0.5) * u
    # token 0 / 1 carry the extreme angle and radius of every pair
    ang[0], rad[0], kk[0], mm[0] = a0, r0, 0, 0
    ang[1], rad[1], kk[1], mm[1] = a1, r1, 2 ** tb - 1, 2 ** rb - 1
    x, y = rad * torch.cos(ang), rad * torch.sin(ang)
    keys = torch.cat([x, y], dim=-1).to(torch.float16).reshape(1, 1, G, 2 * D)
    want = ((mm << tb) + kk).to(torch.uint8)
    for quant in (po.quantize_and_pack_nbit, co.quantize):
        codes, rscale, rmn, tscale, tmn = quant(keys, rb, tb)
        assert torch.equal(codes[0, 0, 0], want)
        assert torch.allclose(tmn.float(), torch.full_like(tmn.float(), a0), atol=2e-3)
        assert torch.allclose(rmn.float(), torch.full_like(rmn.float(), r0), atol=2e-3)
        assert torch.allclose(tscale.float(), torch.full_like(tscale.float(), w), atol=2e-4)
        assert torch.allclose(rscale.float(), torch.full_like(rscale.float(), u), atol=2e-4)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("rbits,tbits", [(4, 4), (3, 3), (2, 5)])
def test_quantizer_invariants(dtype, rbits, tbits):
    k, _ = _keys(2, 3, 256, 1, dtype)
    codes, rscale, rmn, tscale, tmn = po.quantize_and_pack_nbit(k, rbits, tbits)
    theta, rho = codes & (2 ** tbits - 1), codes >> tbits
    assert int(codes.max()) < 2 ** (rbits + tbits)
    ks = k.reshape(2, 3, 2, 128, 2, 64).float()
    x, y = ks[..., 0, :], ks[..., 1, :]
    rad = torch.sqrt(x * x + y * y)
    # the token with the smallest radius gets rho == 0, the largest gets the top code (clamp of exactly 2^b)
    assert bool((rho.gather(3, rad.argmin(3, keepdim=True)) == 0).all())
    assert bool((rho.gather(3, rad.argmax(3, keepdim=True)) == 2 ** rbits - 1).all())
    phi = torch.atan2(y.double(), x.double())
    phi = torch.where(phi < 0, phi + 2 * math.pi, phi)
    assert bool((theta.gather(3, phi.argmin(3, keepdim=True)) == 0).all())
    assert bool((theta.gather(3, phi.argmax(3, keepdim=True)) == 2 ** tbits - 1).all())
    # scale * 2^b reproduces the range up to the dtype's rounding
    eps = 2.0 ** -10 if dtype == torch.float16 else 2.0 ** -7
    rng = (phi.amax(3, keepdim=True) - phi.amin(3, keepdim=True)).float()
    assert bool(((tscale.float() * 2 ** tbits - rng).abs() <= 8 * eps * rng.clamp_min(1.0)).all())


@pytest.mark.parametrize("dtype,tol", [(torch.float16, 2e-3), (torch.bfloat16, 3e-2)])
def test_dequantize_error_bounds(dtype, tol):
    """|phi - phi^| <= tscale/2 and |r - r^| <= rscale/2, up to the dtype's rounding of the intermediates."""
    k, _ = _keys(1, 2, 256, 2, dtype)
    q = po.quantize_and_pack_nbit(k, 4, 4)
    codes, rscale, rmn, tscale, tmn = q
    khat = po.dequantize_keys(*q, dtype=torch.float64).reshape(1, 2, 2, 128, 2, 64)
    ks = k.reshape(1, 2, 2, 128, 2, 64).double()
    r, rh = ks.pow(2).sum(-2).sqrt(), khat.pow(2).sum(-2).sqrt()
    assert bool(((r - rh).abs() <= rscale.double() / 2 + tol * (1 + r)).all())
    phi = torch.atan2(ks[..., 1, :], ks[..., 0, :]); phi = torch.where(phi < 0, phi + 2 * math.pi, phi)
    ph = torch.atan2(khat[..., 1, :], khat[..., 0, :]); ph = torch.where(ph < 0, ph + 2 * math.pi, ph)
    d = (phi - ph).abs(); d = torch.minimum(d, 2 * math.pi - d)
    assert bool((d <= tscale.double() / 2 + tol * 4).all())


def test_quantizer_vs_fp64_brute_force_counts_edge_flips():
    """The half-precision eager quantizer against exact-ish fp64 arithmetic: they may
    only disagree by one bin, on elements that sit on a bin edge ("edge flips")."""
    k, _ = _keys(1, 4, 512, 3)
    codes = po.quantize_and_pack_nbit(k, 4, 4)[0]
    brute = po.quantize_brute_fp64(k, 4, 4)[0]
    dt = (codes & 15).int() - (brute & 15).int()
    dr = (codes >> 4).int() - (brute >> 4).int()
    assert int(dt.abs().max()) <= 1 and int(dr.abs().max()) <= 1
    flips = int((codes != brute).sum())
    print("edge flips half-vs-fp64: %d of %d" % (flips, codes.numel()))
    assert flips < 0.03 * codes.numel()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("tb", [4, 3])
def test_uniform_angle_mode_known_answers(dtype, tb):
    """Fixed angle bins over [-pi, pi): keys placed on the bin centres -pi + (j + 0.5) * 2*pi/2^t
    must get theta == j, the metadata must hold the constants -pi and 2*pi/2^t (rounded to the
    dtype), the radius side must be untouched by the mode, and the two restatements must agree."""
    G, D, rb = 128, 64, 4
    w = 2 * math.pi / 2 ** tb
    g = torch.Generator().manual_seed(5)
    jj = torch.randint(0, 2 ** tb, (G, D), generator=g)
    ang = -math.pi + (jj.double() + 0.5) * w
    rad = 0.5 + 3 * torch.rand(G, D, generator=g, dtype=torch.float64)
    keys = torch.cat([rad * torch.cos(ang), rad * torch.sin(ang)], dim=-1).to(dtype).reshape(1, 1, G, 2 * D)
    ref_group = po.quantize_and_pack_nbit(keys, rb, tb)
    for quant in (po.quantize_and_pack_nbit, co.quantize):
        codes, rscale, rmn, tscale, tmn = quant(keys, rb, tb, angle_mode="uniform")
        assert torch.equal(codes[0, 0, 0] & (2 ** tb - 1), jj.to(torch.uint8))
        assert torch.equal(codes >> tb, ref_group[0] >> tb)                     # radius codes: same as reference mode
        assert torch.equal(rscale, ref_group[1]) and torch.equal(rmn, ref_group[2])
        assert torch.equal(tmn, torch.full_like(tmn, -math.pi))
        assert torch.equal(tscale, torch.full_like(tscale, 2 * math.pi) / 2 ** tb)
        assert abs(float(tmn.flatten()[0]) + math.pi) < 2e-2 and abs(float(tscale.flatten()[0]) - w) < 2e-3
    # random keys: both restatements, every angle within half a bin of its bin centre
    k, _ = _keys(1, 2, 512, 6, dtype)
    a = po.quantize_and_pack_nbit(k, rb, tb, angle_mode="uniform")
    b = co.quantize(k, rb, tb, angle_mode="uniform")
    assert int((a[0] != b[0]).sum()) <= 1e-4 * a[0].numel()
    assert all(torch.equal(x, y) for x, y in zip(a[1:], b[1:]))
    ks = k.double().reshape(1, 2, 4, 128, 2, 64)
    phi = torch.atan2(ks[..., 1, :], ks[..., 0, :])
    centre = a[4].double() + ((a[0] & (2 ** tb - 1)).double() + 0.5) * a[3].double()
    tol = 1e-2 if dtype == torch.float16 else 5e-2
    assert float((phi - centre).abs().max()) <= w / 2 + tol


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("rbits,tbits", [(4, 4), (3, 3), (5, 3)])
def test_c_and_torch_restatements_agree(dtype, rbits, tbits):
    """Two independent restatements: torch eager ops (whose atan2 is SLEEF's) and scalar C with its own
    restatement of that SLEEF routine agree bit for bit; with libm's atan2f in the C one, a last-ulp
    difference of the arctangents moves a few values across a rounding tie (counted, bounded)."""
    k, _ = _keys(2, 4, 1024, 4, dtype)
    a = po.quantize_and_pack_nbit(k, rbits, tbits)
    b = co.quantize(k, rbits, tbits)
    assert all(x.shape == y.shape for x, y in zip(a, b))
    assert torch.equal(a[0], b[0])
    for x, y in zip(a[1:], b[1:]):
        assert torch.equal(x.view(torch.int16), y.view(torch.int16))
    c = co.quantize(k, rbits, tbits, libm_atan2=True)
    # radius side shares no transcendental: bit-exact
    assert torch.equal(a[1].view(torch.int16), c[1].view(torch.int16))
    assert torch.equal(a[2].view(torch.int16), c[2].view(torch.int16))
    flips = int((a[0] != c[0]).sum())
    meta = int((a[3].view(torch.int16) != c[3].view(torch.int16)).sum()) + int((a[4].view(torch.int16) != c[4].view(torch.int16)).sum())
    print("torch-vs-C(libm atan2f) flips: codes %d / %d, angle metadata %d" % (flips, a[0].numel(), meta))
    assert flips <= 1e-4 * a[0].numel() and meta <= 8


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_c_restatement_of_the_sleef_arctangent_rounds_like_torch(dtype):
    """round_dtype(po_sleef_atan2f_u10(y, x)) == torch.atan2 on half / bfloat16 tensors (a library routine, not the
    oracle's formula), on random operands over many exponents plus the special operands."""
    g = torch.Generator().manual_seed(31)
    n = 40000
    e = torch.randint(-10, 6, (2, n), generator=g).float()
    yx = (torch.randn(2, n, generator=g) * torch.exp2(e)).to(dtype)
    special = torch.tensor([0.0, -0.0, 1.0, -1.0, float("inf"), -float("inf"), 6e-8, -6e-8, 65504.0], dtype=dtype)
    y = torch.cat([yx[0], special.repeat_interleave(special.numel())])
    x = torch.cat([yx[1], special.repeat(special.numel())])
    want = torch.atan2(y, x)
    got = co.sleef_atan2f(y.float(), x.float()).to(dtype)
    assert torch.equal(want.view(torch.int16), got.view(torch.int16))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_fp32_wrap_switch_of_both_restatements(dtype):
    """The switch that adds 2*pi in fp32 (what an eager add on the GPU does) in the torch restatement and in the C one:
    bit for bit the same codes and metadata, and different from the default wrap on a good share of the groups."""
    k, _ = _keys(1, 2, 512, 9, dtype)
    a = po.quantize_and_pack_nbit(k, 4, 4, wrap_fp32=True)
    b = co.quantize(k, 4, 4, wrap_fp32=True)
    assert torch.equal(a[0], b[0])
    for x, y in zip(a[1:], b[1:]):
        assert torch.equal(x.view(torch.int16), y.view(torch.int16))
    d = po.quantize_and_pack_nbit(k, 4, 4)
    assert int((a[3].view(torch.int16) != d[3].view(torch.int16)).sum()) > 0


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_the_device_eager_lines_agree_with_the_oracle_on_cpu_tensors(dtype):
    """oracle/device_eager.py holds the reference's lines for evaluation on GPU tensors; on CPU tensors it must be the
    torch oracle bit for bit (the C restatement then pins both), so that only torch's own device behaviour separates
    what it computes on a GPU from the pinned CPU evaluation."""
    from oracle.device_eager import quantize_and_pack_nbit_eager
    k, _ = _keys(2, 4, 1024, 5, dtype)
    for rbits, tbits in ((4, 4), (3, 3), (2, 6)):
        a = po.quantize_and_pack_nbit(k, rbits, tbits)
        b = quantize_and_pack_nbit_eager(k, rbits, tbits)
        assert torch.equal(a[0], b[0])
        for x, y in zip(a[1:], b[1:]):
            assert torch.equal(x.view(torch.int16), y.view(torch.int16))


def test_rope_pair_convention_matches_hf_rotate_half():
    """x = dims [0,64), y = dims [64,128) is the HF rotate-half pairing: rotating a
    key by RoPE turns pair (d, d+64) by the angle pos * inv_freq[d] and keeps its radius."""
    hf = pytest.importorskip("transformers.models.llama.modeling_llama")
    g = torch.Generator().manual_seed(5)
    x = torch.randn(1, 2, 16, 128, generator=g)
    cos, sin = po.rope_cos_sin(torch.arange(16), 128, 1e4)
    ours = po.apply_rope(x, cos, sin)
    theirs = x * cos + hf.rotate_half(x) * sin
    assert torch.equal(ours, theirs)
    assert torch.equal(wl._rope(x, cos, sin), theirs)
    inv = 1.0 / (1e4 ** (torch.arange(0, 128, 2).float() / 128))
    a0 = torch.atan2(x[..., 64:], x[..., :64]).double()
    a1 = torch.atan2(ours[..., 64:], ours[..., :64]).double()
    turn = (torch.arange(16).double()[:, None] * inv.double()[None, :])
    d = torch.remainder(a1 - a0 - turn + math.pi, 2 * math.pi) - math.pi
    assert float(d.abs().max()) < 1e-5
    assert torch.allclose(x[..., :64] ** 2 + x[..., 64:] ** 2, ours[..., :64] ** 2 + ours[..., 64:] ** 2, atol=1e-4)


# --------------------------------------------------------------------- scores
def test_scores_vs_pure_python_lut_loop():
    k, g = _keys(1, 2, 256, 6)
    q = wl.make_half((1, 4, 1, 128), g)
    quant = po.quantize_and_pack_nbit(k, 4, 4)
    s = po.decode_scores(q, *quant, dtype=torch.float64)
    for h, grp in [(0, 0), (3, 1)]:
        brute = torch.tensor(po.decode_scores_lut_python(q, *quant, 4, 4, 0, h, grp), dtype=torch.float64)
        assert torch.allclose(s[0, h, 0, grp * 128:(grp + 1) * 128], brute, rtol=0, atol=1e-9)


def test_scores_polar_identity():
    """q . K^ = sum_d |q_d| r^ cos(phi^ - psi_d): the angle table in polar form."""
    k, g = _keys(1, 1, 128, 7)
    q = wl.make_half((1, 1, 1, 128), g)
    quant = po.quantize_and_pack_nbit(k, 4, 4)
    codes, rscale, rmn, tscale, tmn = quant
    s = po.decode_scores(q, *quant, dtype=torch.float64)[0, 0, 0]
    qx, qy = q[0, 0, 0, :64].double(), q[0, 0, 0, 64:].double()
    qn, psi = torch.sqrt(qx * qx + qy * qy), torch.atan2(qy, qx)
    phi = tscale[0, 0, 0].double() * ((codes[0, 0, 0] & 15).double() + 0.5) + tmn[0, 0, 0].double()
    rad = rscale[0, 0, 0].double() * ((codes[0, 0, 0] >> 4).double() + 0.5) + rmn[0, 0, 0].double()
    alt = (qn * rad * torch.cos(phi - psi)).sum(-1)
    assert torch.allclose(s, alt, rtol=0, atol=1e-9)


@pytest.mark.parametrize("N,Nk", [(8, 8), (8, 2), (7, 1)])
def test_scores_c_vs_torch_and_gqa_mapping(N, Nk):
    k, g = _keys(2, Nk, 256, 8)
    q = wl.make_half((2, N, 1, 128), g)
    quant = po.quantize_and_pack_nbit(k, 3, 3)
    s_t = po.decode_scores(q, *quant, rbits=3, tbits=3, dtype=torch.float64)
    s_c = co.scores(q, *quant, rbits=3, tbits=3)
    assert float((s_t - s_c.double()).abs().max()) < 1e-4
    # query head h must read KV head h // rep (repeat-interleave): score it alone against that head
    rep = N // Nk
    for h in (0, N - 1):
        one = po.decode_scores(q[:, h:h + 1], *[t[:, h // rep:h // rep + 1] for t in quant], rbits=3, tbits=3,
                               dtype=torch.float64)
        # BLAS may block the two matmuls differently: equal to rounding, not bit-for-bit
        assert torch.allclose(one[:, 0], s_t[:, h], rtol=0, atol=1e-10)


def test_scores_approximate_the_unquantized_keys():
    """Sanity of the whole quantize -> score chain: 4/4-bit polar keys reproduce q.K^T to a few percent."""
    k, g = _keys(1, 4, 512, 9)
    q = wl.make_half((1, 4, 1, 128), g)
    quant = po.quantize_and_pack_nbit(k, 4, 4)
    s = po.decode_scores(q, *quant, dtype=torch.float64)
    exact = torch.matmul(q.double(), k.double().transpose(2, 3))
    rel = (s - exact).norm() / exact.norm()
    assert float(rel) < 0.12


# ------------------------------------------------------------------ attention
@pytest.mark.parametrize("with_mask", [False, True])
def test_attention_three_ways(with_mask):
    """Literal restatement vs one-shot fp64 softmax over concatenated keys vs the C loop."""
    B, N, Nk, ng, nr = 2, 8, 2, 2, 37
    k, g = _keys(B, Nk, ng * 128 + nr, 10)
    q = wl.make_half((B, N, 1, 128), g)
    v = wl.make_half((B, Nk, ng * 128 + nr, 128), g)
    quant = po.quantize_and_pack_nbit(k[:, :, :ng * 128].contiguous(), 4, 4)
    kres = k[:, :, ng * 128:].contiguous()
    mask = None
    if with_mask:
        mask = torch.ones(B, ng * 128 + nr, dtype=torch.int64)
        mask[0, :70] = 0
        mask[1, :5] = 0
    a = po.decode_attention(q, kres, *quant, v, mask)
    b = po.decode_attention_exact(q, kres, *quant, v, mask)
    c = co.decode_attn(q, *quant, kres, v, mask)
    assert float((a.double() - b).abs().max()) < 2e-3
    assert float((c.double() - b).abs().max()) < 2e-3
    assert float((a.double() - c.double()).abs().max()) < 2e-3


def test_fp16_baseline_is_plain_softmax_attention():
    k, g = _keys(1, 2, 200, 11)
    q = wl.make_half((1, 4, 1, 128), g)
    v = wl.make_half((1, 2, 200, 128), g)
    out = po.fp16_decode_attention(q, k, v)
    ref = torch.nn.functional.scaled_dot_product_attention(q.float(), po.repeat_kv(k, 2).float(), po.repeat_kv(v, 2).float())
    assert float((out.float() - ref).abs().max()) < 5e-3


# ---------------------------------------------------------- cache bookkeeping
@pytest.mark.parametrize("L", [1, 127, 128, 129, 300, 384])
def test_prefill_cache_split(L):
    k, g = _keys(1, 2, L, 12)
    v = wl.make_half((1, 2, L, 128), g)
    kf, ind, rs, rm, ts, tm, vv, n = po.prefill_cache(k, v)
    nq = 0 if L < 128 else L - L % 128
    assert n == L and vv.shape[2] == L
    assert (ind is None) == (nq == 0)
    if nq:
        assert ind.shape == (1, 2, nq // 128, 128, 64) and rs.shape == (1, 2, nq // 128, 1, 64)
    assert (kf is None) == (L % 128 == 0)
    if kf is not None:
        assert kf.shape[2] == L - nq and torch.equal(kf, k[:, :, nq:])


def test_decode_steps_bookkeeping_and_equivalence():
    """n decode steps from a prompt: quantized tokens = L - L%128 + 128*flushes, residual in [0,127]
    after every step, kv_seq_len = L + n; and every step's output equals one-shot attention over
    the dequantized cache + residual keys (softmax over all L + n tokens)."""
    L, steps = 250, 140
    k, g = _keys(1, 2, L + steps, 13)
    v = wl.make_half((1, 2, L + steps, 128), g)
    qs = wl.make_half((1, 4, steps, 128), g)
    cache = po.prefill_cache(k[:, :, :L], v[:, :, :L])
    for i in range(steps):
        t = L + i
        out, cache = po.decode_step(qs[:, :, i:i + 1], k[:, :, t:t + 1], v[:, :, t:t + 1], cache)
        kf, ind = cache[0], cache[1]
        nres = 0 if kf is None else kf.shape[2]
        nq = 0 if ind is None else ind.shape[2] * 128
        assert cache[-1] == t + 1 and cache[6].shape[2] == t + 1
        assert 0 <= nres <= 127 and nq + nres == t + 1 and nq % 128 == 0
        if i in (0, 5, 6, steps - 1):
            # tokens that were quantized at the time of THIS step's scoring: the flush happens after scoring
            nq_before = ((t + 1) // 128) * 128 if (t + 1) % 128 else t + 1 - 128
            nq_before = max(nq_before, 0) if L >= 128 or t + 1 > 128 else 0
            quant = po.quantize_and_pack_nbit(k[:, :, :nq_before].contiguous()) if nq_before else (None,) * 5
            ref = po.decode_attention_exact(qs[:, :, i:i + 1], k[:, :, nq_before:t + 1], *quant, v[:, :, :t + 1])
            assert float((out.double() - ref).abs().max()) < 2e-3


# ------------------------------------------------------------------ 4-bit values (Mixed variant)
def test_value_quantizer_known_answer_row_and_packing():
    """A row mn + k*s with k = dim % 16 has scale exactly s and codes exactly k; with 8 codes per
    int32, element i in bits [4i, 4i+4), the words alternate 0x76543210 / 0xFEDCBA98."""
    row = (-1 + 0.25 * (torch.arange(128) % 16)).to(torch.float16).reshape(1, 1, 1, 128)
    for quant in (po.quantize_values_along_last_dim, co.quantize_values):
        code, scale, mn = quant(row)
        assert code.dtype == torch.int32 and code.shape == (1, 1, 1, 16) and scale.shape == (1, 1, 1, 1)
        words = [int(w) & 0xFFFFFFFF for w in code.flatten()]
        assert words == [0x76543210, 0xFEDCBA98] * 8
        assert float(scale) == 0.25 and float(mn) == -1.0
    assert torch.equal(po.unpack_values(code).flatten(), torch.arange(128) % 16)
    assert torch.equal(po.dequantize_values(code, scale, mn).flatten(), row.float().flatten())


def test_value_quantizer_rounds_half_to_even_after_clamp():
    """(x - mn)/scale landing exactly on k + 0.5 goes to the even neighbour (torch.round), and the
    clamp comes first, so nothing above 15 survives."""
    k = torch.tensor([0.0, 0.5, 1.5, 2.5, 3.5, 13.5, 14.5, 15.0])
    row = torch.zeros(128)
    row[:8] = k * 0.25                      # scale = 15*0.25/15 = 0.25 exactly, mn = 0
    row[8:] = 3.75
    for quant in (po.quantize_values_along_last_dim, co.quantize_values):
        code, scale, mn = quant(row.to(torch.float16).reshape(1, 1, 1, 128))
        assert float(scale) == 0.25 and float(mn) == 0.0
        assert po.unpack_values(code).flatten()[:8].tolist() == [0, 0, 2, 2, 4, 14, 14, 15]


@pytest.mark.parametrize("dtype,eps", [(torch.float16, 2e-3), (torch.bfloat16, 2e-2)])
def test_value_quantizer_invariants_and_restatements(dtype, eps):
    g = torch.Generator().manual_seed(12)
    v = wl.make_half((2, 3, 200, 128), g, dtype)
    v[0, 0, 0] = 0.5                        # constant row: 0/0, defined as code 0
    a = po.quantize_values_along_last_dim(v)
    b = co.quantize_values(v)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1].view(torch.int16), b[1].view(torch.int16))
    assert torch.equal(a[2].view(torch.int16), b[2].view(torch.int16))
    codes = po.unpack_values(a[0])
    assert int(codes.min()) == 0 and int(codes.max()) == 15 and bool((codes[0, 0, 0] == 0).all())
    vf = v.float()
    # the row minimum gets code 0, the row maximum 15 (constant row aside)
    lo, hi = vf.argmin(-1, keepdim=True), vf.argmax(-1, keepdim=True)
    assert bool((codes.gather(-1, lo)[1:] == 0).all()) and bool((codes.gather(-1, hi)[1:] == 15).all())
    assert torch.equal(a[2].float(), vf.min(-1, keepdim=True)[0])
    # reconstruction within half a step (plus the dtype's own rounding of the intermediates)
    err = (po.dequantize_values(*a) - vf).abs()
    assert bool((err <= a[1].float() / 2 + eps * vf.abs().amax(-1, keepdim=True)).all())


def test_mixed_attention_literal_vs_one_shot_fp64():
    """The literal Mixed decode step (two matmuls, half-rounded probabilities) against one fp64
    softmax attention over [dequantized ; residual] keys and values; and with no quantized part it
    reduces to the plain fp16 attention."""
    g = torch.Generator().manual_seed(13)
    B, N, Nk, nb, res = 2, 8, 2, 3, 40
    L = nb * 128 + res
    k = wl.make_keys(B, Nk, L, 5e5, g)
    q, v = wl.make_half((B, N, 1, 128), g), wl.make_half((B, Nk, L, 128), g)
    quant = po.quantize_and_pack_nbit(k[:, :, :nb * 128].contiguous())
    vq = po.quantize_values_along_last_dim(v[:, :, :nb * 128].contiguous())
    kres, vres = k[:, :, nb * 128:], v[:, :, nb * 128:]
    mask = torch.ones(B, L, dtype=torch.int64)
    mask[1, :200] = 0
    for m in (None, mask):
        a = po.decode_attention_mixed(q, kres, *quant, vres, *vq, m)
        e = po.decode_attention_mixed_exact(q, kres, *quant, vres, *vq, m)
        assert (a.double() - e).abs().max().item() < 2e-3
        # 4-bit values are a perturbation of the fp16-value attention, of the size the step predicts
        plain = po.decode_attention_exact(q, kres, *quant, v, m)
        assert (e - plain).abs().max().item() < 0.5 * float(vq[1].float().max())
    a = po.decode_attention_mixed(q, kres, None, None, None, None, None, vres, None, None, None)
    f = po.fp16_decode_attention(q, kres, vres)
    assert (a.float() - f.float()).abs().max().item() < 2e-3


@pytest.mark.parametrize("L", [1, 127, 128, 129, 300, 384])
def test_mixed_cache_bookkeeping(L):
    """Keys and values share the residual window: after any prompt length and any number of decode
    steps, quantized tokens = 128 * floor(kv_len / 128) on both sides (0 when the prompt was
    shorter than 128 and no flush happened yet), and the tuple has the reference's 11 slots."""
    g = torch.Generator().manual_seed(L)
    k, v = wl.make_keys(1, 2, L + 140, 1e4, g), wl.make_half((1, 2, L + 140, 128), g)
    cache = po.prefill_cache_mixed(k[:, :, :L], v[:, :, :L])
    assert len(cache) == 11 and cache[-1] == L
    for i in range(140):
        q = wl.make_half((1, 4, 1, 128), g)
        out, cache = po.decode_step_mixed(q, k[:, :, L + i:L + i + 1], v[:, :, L + i:L + i + 1], cache)
        n = L + i + 1
        kf, ind, vf, vc, vs, vm = cache[0], cache[1], cache[6], cache[7], cache[8], cache[9]
        nres = 0 if kf is None else kf.shape[2]
        assert (vf is None) == (kf is None) and (vf is None or vf.shape[2] == nres)
        nq = 0 if ind is None else ind.shape[2] * 128
        assert nq + nres == n == cache[-1] and 0 <= nres < 128
        assert (vc is None) == (ind is None)
        if vc is not None:
            assert vc.shape == (1, 2, nq, 16) and vs.shape == vm.shape == (1, 2, nq, 1)
        assert out.shape == (1, 4, 1, 128)


# ------------------------------------------------------------------ SnapKV prompt eviction
def test_snapkv_selection_keeps_the_keys_the_window_attends_to():
    """Hand-built prompt: a few earlier keys are aligned with every query of the last window, the rest
    are noise.  With a pooling kernel of 7 each heavy key lifts its 6 neighbours; the kept set must
    contain all of those neighbourhoods, for every KV head."""
    torch.manual_seed(0)
    B, N, Nk, L, ws, cap = 1, 4, 2, 600, 64, 64 + 80
    u = torch.randn(128)
    u = u / u.norm()
    q = (0.05 * torch.randn(B, N, L, 128) + 3.0 * u).half()
    k = (0.05 * torch.randn(B, Nk, L, 128)).half()
    heavy = [20, 75, 130, 222, 301, 377, 444, 500]
    k[:, :, heavy] = (4.0 * u).half()
    idx = po.snapkv_select(q, k, window_size=ws, kernel_size=7, max_capacity_prompt=cap)
    assert idx.shape == (B, Nk, cap - ws) and int(idx.max()) < L - ws
    want = {p + d for p in heavy for d in range(-3, 4)}
    for h in range(Nk):
        got = set(idx[0, h].tolist())
        assert len(got) == cap - ws and want <= got
    # with no pooling the choice depends on each key alone: permuting the earlier keys permutes the kept set
    perm = torch.randperm(L - ws)
    k2 = k.clone()
    k2[:, :, :L - ws] = k[:, :, perm]
    a = po.snapkv_select(q, k, ws, 1, cap)
    b = po.snapkv_select(q, k2, ws, 1, cap)
    s = po.snapkv_scores(q, k, ws, 1)
    kth = s.topk(cap - ws, dim=-1).values[..., -1:]
    for h in range(Nk):
        strictly_in = set(torch.nonzero(s[0, h] > kth[0, h]).flatten().tolist())      # ties at the threshold may go either way
        assert strictly_in <= set(a[0, h].tolist()) and strictly_in <= {int(perm[j]) for j in b[0, h].tolist()}


@pytest.mark.parametrize("L", [100, 128, 700, 1152, 1153, 1400])
def test_snapkv_cache_bookkeeping(L):
    """Prompts up to max_capacity_prompt are cached whole (the plain polar prefill); longer ones keep
    1024 selected tokens + the last 128, all quantized (1152 = 9 groups), their values gathered with
    the same indices, and the tuple still reports the full prompt length."""
    g = torch.Generator().manual_seed(L)
    q, k, v = wl.make_half((1, 4, L, 128), g), wl.make_keys(1, 2, L, 1e4, g), wl.make_half((1, 2, L, 128), g)
    cache = po.prefill_cache_snapkv(q, k, v)
    assert len(cache) == 8 and cache[-1] == L
    kept = min(L, 1152)
    assert cache[6].shape[2] == kept
    nq = 0 if cache[1] is None else cache[1].shape[2] * 128
    nr = 0 if cache[0] is None else cache[0].shape[2]
    assert nq + nr == kept and (nq == (kept // 128) * 128 if L >= 128 else nq == 0)
    if L <= 1152:
        plain = po.prefill_cache(k, v)
        for a, b in zip(cache[:-1], plain[:-1]):
            assert (a is None) == (b is None) and (a is None or torch.equal(a, b))
    else:
        idx = po.snapkv_select(q, k)
        assert torch.equal(cache[6][:, :, :1024], v[:, :, :-128].gather(2, idx.unsqueeze(-1).expand(-1, -1, -1, 128)))
        assert torch.equal(cache[6][:, :, 1024:], v[:, :, -128:])
        kk = torch.cat([k[:, :, :-128].gather(2, idx.unsqueeze(-1).expand(-1, -1, -1, 128)), k[:, :, -128:]], 2)
        assert torch.equal(cache[1], po.quantize_and_pack_nbit(kk)[0])
        # decode continues at position L and appends to the 1152 cached tokens
        out, c2 = po.decode_step(wl.make_half((1, 4, 1, 128), g), k[:, :, :1], v[:, :, :1], cache)
        assert c2[-1] == L + 1 and c2[6].shape[2] == 1153 and c2[0].shape[2] == 1


# ------------------------------------------------------------------ packed 6-bit code rows
def test_packed6_layout_known_answer_and_round_trip():
    """Code i of a row sits in bits [6i, 6i+6) of the 48-byte row (little-endian): checked on rows
    with a single non-zero code against the bit position computed by hand, then as a round trip."""
    for i, val in [(0, 63), (1, 1), (4, 33), (5, 63), (21, 42), (63, 63)]:
        row = torch.zeros(64, dtype=torch.uint8)
        row[i] = val
        packed = po.pack_codes6(row)
        assert packed.shape == (48,)
        bits = sum(int(b) << (8 * j) for j, b in enumerate(packed.tolist()))
        assert bits == val << (6 * i)
    g = torch.Generator().manual_seed(3)
    codes = torch.randint(0, 64, (2, 3, 5, 128, 64), generator=g, dtype=torch.uint8)
    packed = po.pack_codes6(codes)
    assert packed.shape == (2, 3, 5, 128, 48) and torch.equal(po.unpack_codes6(packed), codes)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_residual_score_rounding_band_covers_the_actual_rounding(dtype):
    """The band is a first-order bound: rounding the window's scores to the model dtype (what the
    reference's half-precision matmul does, :79) must move the fp64 output by no more than it,
    and a band with a dropped factor (half of it) must be exceeded somewhere (so the bound is not slack by construction)."""
    g = torch.Generator().manual_seed(41)
    B, N, Nk, nb, nr = 2, 8, 2, 1, 37
    L = nb * 128 + nr
    k = wl.make_keys(B, Nk, L, 5e5, g, dtype)
    v = wl.make_half((B, Nk, L, 128), g, dtype)
    q = wl.make_half((B, N, 1, 128), g, dtype)
    quant = po.quantize_and_pack_nbit(k[:, :, :nb * 128].contiguous(), 4, 4)
    kr = k[:, :, nb * 128:]
    mask = torch.ones(B, L, dtype=torch.int64)
    mask[1, :140] = 0                                   # sequence 1 attends to 25 window tokens only
    exact = po.decode_attention_exact(q, kr, *quant, v, mask, 4, 4)
    band = po.residual_score_rounding_band(q, kr, *quant, v, mask, 4, 4)
    assert band.shape == exact.shape and bool((band >= 0).all())
    # the same attention with the window's scores rounded to the dtype
    kd = torch.cat([po.dequantize_keys(*quant, 4, 4, torch.float64), kr.double()], dim=2)
    s = torch.matmul(q.double(), po.repeat_kv(kd, N // Nk).transpose(2, 3))
    s[..., nb * 128:] = s[..., nb * 128:].to(dtype).double()
    a = (s / math.sqrt(128)).masked_fill(mask[:, None, None, :] == 0, float("-inf"))
    rounded = torch.matmul(torch.softmax(a, -1), po.repeat_kv(v.double(), N // Nk))
    moved = (rounded - exact).abs()
    assert bool((moved <= band * 1.02 + 1e-12).all()), float((moved - band).max())
    assert bool((moved > band * 0.15).any())           # typical movement is a fair fraction of the worst case
    # no window, no band
    z = po.residual_score_rounding_band(q, None, *quant, v[:, :, :nb * 128], None, 4, 4)
    assert float(z.abs().max()) == 0.0
