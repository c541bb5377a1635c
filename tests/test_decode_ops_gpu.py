"""The fused elementwise kernels of the decode step against the eager torch ops they replace
(HF apply_rotary_pos_emb + cache writes, residual add + RMSNorm, SiLU * up)."""
import pytest
import torch
import torch.nn.functional as F

from polarquant_amd.decode_ops import rmsnorm, rope_append, silu_mul
from polarquant_amd.modeling_common import RMSNorm, apply_rotary_pos_emb

pytestmark = pytest.mark.gpu


def _ulps_off(got: torch.Tensor, ref: torch.Tensor) -> float:
    """Largest |got - ref| in units of the dtype's spacing at |ref|."""
    return float(((got.float() - ref.float()).abs() / _ulp(ref)).max())


def _ulp(ref: torch.Tensor) -> torch.Tensor:
    """Spacing of the dtype at |ref| (as float)."""
    bits = 10 if ref.dtype == torch.float16 else 7
    mag = ref.float().abs().clamp_min(2.0 ** -14)
    return torch.exp2(torch.floor(torch.log2(mag)) - bits)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("N,Nk", [(8, 2), (7, 1), (4, 4)])
def test_rope_append_is_bit_identical_to_the_eager_ops(gpu, dtype, N, Nk):
    torch.manual_seed(N * 10 + Nk)
    B, rows, max_pos = 3, 128, 700
    inv = 1.0 / (5e5 ** (torch.arange(0, 128, 2, dtype=torch.float32) / 128))
    ang = torch.arange(max_pos, dtype=torch.float32)[:, None] * inv[None]
    emb = torch.cat([ang, ang], -1)
    cos_t, sin_t = emb.cos().to(dtype).to(gpu), emb.sin().to(dtype).to(gpu)
    q_lin = torch.randn(B, 1, N * 128, device=gpu).to(dtype)
    k_lin = torch.randn(B, 1, Nk * 128, device=gpu).to(dtype)
    v_lin = torch.randn(B, 1, Nk * 128, device=gpu).to(dtype)
    for p, kr in [(0, 0), (321, 65), (699, 127)]:
        pos = torch.tensor([p], dtype=torch.int64, device=gpu)
        k_row = torch.tensor([kr], dtype=torch.int64, device=gpu)
        k_dst = torch.full((B, Nk, rows, 128), 7.0, dtype=dtype, device=gpu)
        v_dst = torch.full((B, Nk, max_pos, 128), 7.0, dtype=dtype, device=gpu)
        q = rope_append(q_lin, k_lin, v_lin, cos_t, sin_t, pos, k_dst, k_row, v_dst, pos, N, Nk)
        # the eager chain (reference :50-59, :77, :98)
        qe = q_lin.view(B, 1, N, 128).transpose(1, 2)
        ke = k_lin.view(B, 1, Nk, 128).transpose(1, 2)
        ve = v_lin.view(B, 1, Nk, 128).transpose(1, 2)
        qr, kr_ = apply_rotary_pos_emb(qe, ke, cos_t[p:p + 1][None], sin_t[p:p + 1][None])
        assert q.shape == (B, N, 1, 128) and torch.equal(q, qr)
        assert torch.equal(k_dst[:, :, kr], kr_[:, :, 0]) and torch.equal(v_dst[:, :, p], ve[:, :, 0])
        k_dst[:, :, kr] = 7.0
        v_dst[:, :, p] = 7.0
        assert bool((k_dst == 7.0).all()) and bool((v_dst == 7.0).all())     # nothing else was touched


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("hidden", [512, 4096, 3584, 16384])
def test_rmsnorm_matches_module(gpu, dtype, hidden):
    torch.manual_seed(hidden)
    mod = RMSNorm(hidden, 1e-5).to(dtype).to(gpu)
    with torch.no_grad():
        mod.weight.copy_((1 + 0.1 * torch.randn(hidden)).to(dtype))
    x = (torch.randn(5, 1, hidden, device=gpu) * 3).to(dtype)
    res = torch.randn(5, 1, hidden, device=gpu).to(dtype)
    with torch.no_grad():
        ref = mod(x)
        got = rmsnorm(x, mod.weight, mod.variance_epsilon)
        # w * dtype(x * inv): a last-bit difference of the fp32 inv can move the inner rounding by one
        # step, which the multiplication by w can turn into two steps of the result
        assert _ulps_off(got, ref) <= 2, _ulps_off(got, ref)
        assert (got != ref).float().mean().item() < 0.05                    # and such differences are rare
        s_ref = x + res
        ref2 = mod(s_ref)
        s = torch.empty_like(x)
        got2 = rmsnorm(x, mod.weight, mod.variance_epsilon, residual=res, sum_out=s)
        assert torch.equal(s, s_ref)
        assert _ulps_off(got2, ref2) <= 2, _ulps_off(got2, ref2)
        assert (got2 != ref2).float().mean().item() < 0.05
        xin = x.clone()
        got3 = rmsnorm(xin, mod.weight, mod.variance_epsilon, residual=res, sum_out=xin)      # in place
        assert torch.equal(xin, s_ref) and torch.equal(got3, got2)
        got4 = rmsnorm(x, mod.weight, mod.variance_epsilon, residual=res)                   # sum not wanted
        assert torch.equal(got4, got2)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_silu_mul_matches_eager(gpu, dtype):
    torch.manual_seed(1)
    g = (torch.randn(4, 1, 14336, device=gpu) * 3).to(dtype)
    u = torch.randn(4, 1, 14336, device=gpu).to(dtype)
    ref = F.silu(g) * u
    got = silu_mul(g, u)
    assert _ulps_off(got, ref) <= 2, _ulps_off(got, ref)
    assert (got != ref).float().mean().item() < 0.05
    # the two halves of one fused gate|up projection output
    gu = torch.cat([g, u], dim=-1)
    assert torch.equal(silu_mul(gu[..., :14336], gu[..., 14336:]), got)


def test_measurement_aids_launch_and_report_their_bytes(gpu):
    """pq_stream_read and pq_attn_load_replica read what they say (whole 16 KiB trips / whole pairs of tiles) and
    leave their inputs and the sink alone."""
    from polarquant_amd import _ffi
    from polarquant_amd.kernel4group import _stream_ptr
    lib = _ffi.bench_lib()
    planes, tokens = 6, 1000
    codes = torch.randint(0, 255, (planes, 1024, 64), dtype=torch.uint8, device=gpu)
    v = torch.randn(planes, tokens + 5, 128, device=gpu).half()
    before = (codes.clone(), v.clone())
    sink = torch.zeros(1, dtype=torch.int32, device=gpu)
    got = lib.pq_attn_load_replica(codes.data_ptr(), v.data_ptr(), planes, 1024, tokens + 5, tokens, 3, sink.data_ptr(), _stream_ptr(gpu))
    assert got == planes * 3 * 256 * 320            # 1000 // 3 = 333 tokens -> 256 per slice
    got = lib.pq_stream_read(v.data_ptr(), v.numel() * 2, 7, sink.data_ptr(), _stream_ptr(gpu))
    assert got == 7 * (v.numel() * 2 // 7 // 16384 * 16384)
    torch.cuda.synchronize()
    assert torch.equal(codes, before[0]) and torch.equal(v, before[1]) and int(sink) == 0


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("B,L,N,Nk,per_seq", [(2, 300, 4, 2, False), (3, 1, 7, 1, True), (1, 129, 32, 8, False), (2, 64, 28, 4, True)])
def test_rope_qk_is_the_eager_rotation_bit_for_bit(gpu, dtype, B, L, N, Nk, per_seq):
    from polarquant_amd.decode_ops import rope_qk
    from polarquant_amd.modeling_common import apply_rotary_pos_emb
    g = torch.Generator().manual_seed(B * 100 + L + N)
    fused = (torch.randn(B, L, (N + 2 * Nk) * 128, generator=g) * 3).to(dtype).to(gpu)      # slices of one projection output
    q_lin, k_lin = fused[..., :N * 128], fused[..., N * 128:(N + Nk) * 128]
    pos = torch.arange(L, dtype=torch.float32)[None].repeat(B if per_seq else 1, 1)
    if per_seq:
        pos = pos + torch.arange(pos.shape[0], dtype=torch.float32)[:, None] * 17
    ang = pos[..., None] * (5e5 ** (-torch.arange(0, 128, 2).float() / 128))
    emb = torch.cat([ang, ang], -1)
    cos, sin = emb.cos().to(dtype).to(gpu), emb.sin().to(dtype).to(gpu)
    q_ref, k_ref = apply_rotary_pos_emb(q_lin.reshape(B, L, N, 128).transpose(1, 2), k_lin.reshape(B, L, Nk, 128).transpose(1, 2), cos, sin)
    q, k = rope_qk(q_lin, k_lin, cos, sin, N, Nk)
    assert q.shape == (B, N, L, 128) and k.shape == (B, Nk, L, 128)
    assert torch.equal(q, q_ref) and torch.equal(k, k_ref)
    # dense inputs take the same path
    q2, k2 = rope_qk(q_lin.contiguous(), k_lin.contiguous(), cos, sin, N, Nk)
    assert torch.equal(q2, q_ref) and torch.equal(k2, k_ref)
