"""Packed 6-bit code rows (48 bytes per token instead of 64) on the GPU: the quantizer writes exactly
the oracle's packing of the oracle's codes, and every decode kernel gives bit-identical results from
packed and from byte-per-code rows (the arithmetic after unpacking is the same)."""
import pytest
import torch

from oracle import polar_oracle as po
from polarquant_amd import workloads as wl
from polarquant_amd.attention import polar_decode_attention, polar_decode_attention_v4
from polarquant_amd.kernel4group import attention_decode_forward_triton_impl
from polarquant_amd.quantize import quantize_and_pack_nbit
from polarquant_amd.values import quantize_values

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("rbits,tbits", [(3, 3), (2, 4), (4, 2), (2, 3), (1, 1)])
def test_quantizer_writes_the_oracle_packing(gpu, dtype, rbits, tbits):
    g = torch.Generator().manual_seed(61)
    k = wl.make_keys(2, 3, 512, 1e6, g, dtype)
    ref = po.quantize_and_pack_nbit(k, rbits, tbits)
    got = quantize_and_pack_nbit(k.to(gpu), rbits, tbits, packed=True)
    assert got[0].shape == (2, 3, 4, 128, 48) and got[0].dtype == torch.uint8
    assert torch.equal(got[0].cpu(), po.pack_codes6(ref[0]))
    for a, b in zip(got[1:], ref[1:]):
        assert bool((a.cpu().float() == b.float()).all())
    # into a slot of a larger pre-allocated packed store, from a strided view
    kt = k.to(gpu).transpose(1, 2).contiguous().transpose(1, 2)
    out = (torch.full((2, 3, 9, 128, 48), 0xEE, dtype=torch.uint8, device=gpu),
           *[torch.zeros(2, 3, 9, 1, 64, dtype=dtype, device=gpu) for _ in range(4)])
    quantize_and_pack_nbit(kt, rbits, tbits, packed=True, out=out, group_offset=3)
    assert torch.equal(out[0][:, :, 3:7].cpu(), po.pack_codes6(ref[0]))
    assert bool((out[0][:, :, :3] == 0xEE).all()) and bool((out[0][:, :, 7:] == 0xEE).all())


def test_packing_needs_six_bits(gpu):
    k = torch.zeros(1, 1, 128, 128, dtype=torch.float16, device=gpu)
    with pytest.raises(AssertionError):
        quantize_and_pack_nbit(k, 4, 4, packed=True)


@pytest.mark.parametrize("N,Nk", [(4, 4), (8, 2), (7, 1), (2, 1)])
@pytest.mark.parametrize("rbits", [3, 2])
def test_decode_kernels_agree_on_packed_and_unpacked_rows(gpu, N, Nk, rbits):
    tbits = 3
    g = torch.Generator().manual_seed(62 + N)
    B, nb, nr = 2, 5, 37
    L = nb * 128 + nr
    k = wl.make_keys(B, Nk, L, 1e6, g)
    q = wl.make_half((B, N, 1, 128), g).to(gpu)
    v = wl.make_half((B, Nk, L, 128), g).to(gpu)
    plain = quantize_and_pack_nbit(k[:, :, :nb * 128].to(gpu), rbits, tbits)
    packed = quantize_and_pack_nbit(k[:, :, :nb * 128].to(gpu), rbits, tbits, packed=True)
    assert torch.equal(po.unpack_codes6(packed[0].cpu()), plain[0].cpu())
    # scores: same fp32 bits
    s0 = attention_decode_forward_triton_impl(q, *plain, rbits=rbits, tbits=tbits)
    s1 = attention_decode_forward_triton_impl(q, *packed, rbits=rbits, tbits=tbits)
    assert torch.equal(s0, s1)
    ref = po.decode_scores(q.cpu(), *[t.cpu() for t in plain], rbits, tbits)
    assert (s1.cpu() - ref).abs().max().item() <= 1e-3 * ref.abs().max().item()
    # fused attention, half-precision values, with a mask and spare capacity
    kres = torch.zeros(B, Nk, 128, 128, dtype=torch.float16, device=gpu)
    kres[:, :, :nr] = k[:, :, nb * 128:].to(gpu)
    mask = torch.ones(B, L, dtype=torch.uint8, device=gpu)
    mask[1, :100] = 0
    grow = lambda t: torch.cat([t, torch.zeros_like(t[:, :, :2])], dim=2).contiguous()
    for ns in (None, 1, 3):
        o0 = polar_decode_attention(q, *[grow(t) for t in plain], kres, v, nb, nr, attention_mask=mask, rbits=rbits, tbits=tbits, n_splits=ns)
        o1 = polar_decode_attention(q, *[grow(t) for t in packed], kres, v, nb, nr, attention_mask=mask, rbits=rbits, tbits=tbits, n_splits=ns)
        assert torch.equal(o0, o1)
    # fused attention, 4-bit values
    vq = quantize_values(v[:, :, :nb * 128])
    vres = torch.zeros_like(kres)
    vres[:, :, :nr] = v[:, :, nb * 128:]
    o0 = polar_decode_attention_v4(q, *plain, kres, vres, *vq, nb, nr, rbits=rbits, tbits=tbits)
    o1 = polar_decode_attention_v4(q, *packed, kres, vres, *vq, nb, nr, rbits=rbits, tbits=tbits)
    assert torch.equal(o0, o1)


def test_packed_rows_are_refused_for_other_angle_widths(gpu):
    from polarquant_amd._ffi import PolarQuantError
    g = torch.Generator().manual_seed(63)
    k = wl.make_keys(1, 1, 128, 1e4, g).to(gpu)
    q = wl.make_half((1, 1, 1, 128), g).to(gpu)
    packed = quantize_and_pack_nbit(k, 2, 4, packed=True)          # the quantizer packs any rbits + tbits <= 6 ...
    with pytest.raises(PolarQuantError):                           # ... the decode kernels unpack tbits == 3 only
        attention_decode_forward_triton_impl(q, *packed, rbits=2, tbits=4)


def test_attention_class_with_packed_codes_equals_the_plain_one(gpu):
    """config.packed_codes: the cache tuple carries [B,Nk,Nb,128,48] indices; outputs and every other
    tuple slot are bit-identical to the byte-per-code cache, across a flush."""
    from polarquant_amd.modeling_common import PolarConfig
    from polarquant_amd.modeling_qwen_polar import Qwen2PolarForCausalLM, Qwen2PolarGroupAttention
    kw = dict(hidden_size=7 * 128, num_attention_heads=7, num_key_value_heads=1, num_hidden_layers=1, intermediate_size=256,
              vocab_size=100, rope_theta=1e6, rbits=3, tbits=3, attention_bias=True)
    torch.manual_seed(3)
    a = Qwen2PolarGroupAttention(PolarConfig(**kw), 0).half().to(gpu)
    b = Qwen2PolarGroupAttention(PolarConfig(packed_codes=True, **kw), 0).half().to(gpu)
    b.load_state_dict(a.state_dict())
    L, steps = 200, 70
    x = (torch.randn(2, L + steps, 7 * 128) * 0.5).half().to(gpu)
    inv = 1.0 / (1e6 ** (torch.arange(0, 128, 2, dtype=torch.float32) / 128))

    def rope(start, n):
        ang = torch.arange(start, start + n, dtype=torch.float32)[:, None] * inv[None]
        emb = torch.cat([ang, ang], -1)[None]
        return emb.cos().half().to(gpu), emb.sin().half().to(gpu)
    with torch.no_grad():
        oa, ca = a(x[:, :L], None, None, rope(0, L))
        ob, cb = b(x[:, :L], None, None, rope(0, L))
        assert torch.equal(oa, ob)
        for i in range(steps):
            oa, ca = a(x[:, L + i:L + i + 1], None, ca, rope(L + i, 1))
            ob, cb = b(x[:, L + i:L + i + 1], None, cb, rope(L + i, 1))
            assert torch.equal(oa, ob), i
    assert cb[1].shape[-1] == 48 and ca[1].shape[-1] == 64 and cb[1].shape[2] == ca[1].shape[2] == 2
    assert torch.equal(po.unpack_codes6(cb[1].cpu()), ca[1].cpu())
    for j in (0, 2, 3, 4, 5, 6):
        assert (ca[j] is None and cb[j] is None) or torch.equal(ca[j], cb[j])
    m = Qwen2PolarForCausalLM(PolarConfig(packed_codes=True, **kw))
    assert m.kv_cache_bytes_per_token() == 1 * 1 * (48 + 4 + 256)


def test_layout_converters_round_trip(gpu):
    from polarquant_amd.quantize import convert_codes6
    g = torch.Generator().manual_seed(64)
    codes = torch.randint(0, 64, (2, 3, 5, 128, 64), generator=g, dtype=torch.uint8)
    packed = convert_codes6(codes.to(gpu), pack=True)
    assert packed.shape == (2, 3, 5, 128, 48) and torch.equal(packed.cpu(), po.pack_codes6(codes))
    back = convert_codes6(packed, pack=False)
    assert torch.equal(back.cpu(), codes)
