"""pq_linear_small_m (the decode step's projections at <= 16 rows) against fp32 torch matmuls of the
same half-precision operands.  Tolerance: the result is one rounding of an fp32 sum whose order differs
from the reference's, so at most one unit in the last place of the dtype, plus a little accumulation noise."""
import os
import random

import pytest
import torch
import torch.nn.functional as F

from polarquant_amd.decode_ops import linear_small_m

pytestmark = pytest.mark.gpu

EPS = {torch.float16: 2.0 ** -11, torch.bfloat16: 2.0 ** -8}


def _check(y, ref, dtype, ulps=1.0):
    y, ref = y.float().cpu(), ref.float().cpu()
    tol = ulps * 2 * EPS[dtype] * ref.abs() + 1e-3 * ref.abs().mean()
    bad = ((y - ref).abs() > tol).sum().item()
    assert bad == 0, "%d of %d outputs off; worst %.3e" % (bad, y.numel(), (y - ref).abs().max().item())


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M,N,K,bias", [(8, 6144, 4096, False), (1, 4096, 4096, False), (16, 4096, 14336, False), (8, 4096, 14336, False), (9, 256, 4096, True), (4, 64, 160, False),
                                        (5, 1024, 3584, True), (8, 64, 96, True), (3, 18944, 3584, False), (8, 4608, 3584, True)])
def test_linear_matches_fp32_matmul(gpu, dtype, M, N, K, bias):
    print("case", dtype, M, N, K, bias, flush=True)
    g = torch.Generator().manual_seed(M * 1000 + N + K)
    x = torch.randn(M, 1, K, generator=g).to(dtype)
    w = (torch.randn(N, K, generator=g) * 0.05).to(dtype)
    b = torch.randn(N, generator=g).to(dtype) if bias else None
    y = linear_small_m(x.to(gpu), w.to(gpu), None if b is None else b.to(gpu))
    assert y.shape == (M, 1, N) and y.dtype == dtype
    ref = F.linear(x.double(), w.double(), None if b is None else b.double())
    _check(y, ref, dtype)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_linear_reads_a_strided_slice(gpu, dtype):
    """x as columns [256, 768) of a wider activation: unit element stride, wider row stride."""
    g = torch.Generator().manual_seed(5)
    wide = torch.randn(8, 1024, generator=g).to(dtype).to(gpu)
    w = (torch.randn(128, 512, generator=g) * 0.05).to(dtype).to(gpu)
    y = linear_small_m(wide[:, 256:768], w)
    _check(y, F.linear(wide[:, 256:768].double().cpu(), w.double().cpu()), dtype)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", [(8, 14336, 4096), (2, 512, 256), (16, 1536, 3584)])
def test_gated_linear_follows_the_eager_roundings(gpu, dtype, M, N, K):
    """silu(x.Wg^T) * (x.Wu^T) with gate, up and silu(gate) each rounded to the dtype, as the eager MLP does."""
    print("case gated", dtype, M, N, K, flush=True)
    g = torch.Generator().manual_seed(N + K)
    x = torch.randn(M, K, generator=g).to(dtype)
    wg = (torch.randn(N, K, generator=g) * 0.03).to(dtype)
    wu = (torch.randn(N, K, generator=g) * 0.03).to(dtype)
    y = linear_small_m(x.to(gpu), wg.to(gpu), up_weight=wu.to(gpu))
    gate = F.linear(x.double(), wg.double()).to(dtype)
    up = F.linear(x.double(), wu.double()).to(dtype)
    act = (gate.double() * torch.sigmoid(gate.double())).to(dtype)
    ref = (act.double() * up.double())
    # a last-place difference in gate or up (summation order) moves the product by about one more unit
    _check(y, ref, dtype, ulps=3.0)


# more seeds: PQ_RANDOM_LINEAR_CASES=2000; another stretch of them: PQ_RANDOM_LINEAR_FIRST=1000
_SEEDS = range(int(os.environ.get("PQ_RANDOM_LINEAR_FIRST", "0")),
               int(os.environ.get("PQ_RANDOM_LINEAR_FIRST", "0")) + int(os.environ.get("PQ_RANDOM_LINEAR_CASES", "16")))


@pytest.mark.parametrize("seed", _SEEDS)
def test_random_linear_case(gpu, seed):
    """Random rows (1..16), outputs (any multiple of 16), inner size (any multiple of 32: every K-split and stage
    remainder), bias or gate, dtype, dense or strided x."""
    rnd = random.Random(9000 + seed)
    dtype = torch.bfloat16 if seed % 3 == 2 else torch.float16
    M = rnd.randint(1, 16)
    N = 16 * rnd.randint(1, 96)
    K = 32 * rnd.randint(1, rnd.choice([8, 64, 300]))
    gated = rnd.random() < 0.3
    bias = not gated and rnd.random() < 0.5
    strided = rnd.random() < 0.3
    print("case", dict(seed=seed, dtype=str(dtype), M=M, N=N, K=K, gated=gated, bias=bias, strided=strided), flush=True)
    g = torch.Generator().manual_seed(seed)
    wide = torch.randn(M, K + 64, generator=g).to(dtype)
    x = wide[:, 32:32 + K] if strided else wide[:, :K].contiguous()
    sc = 1.0 / (K ** 0.5)
    w = (torch.randn(N, K, generator=g) * sc).to(dtype)
    if gated:
        wu = (torch.randn(N, K, generator=g) * sc).to(dtype)
        y = linear_small_m(wide.to(gpu)[:, 32:32 + K] if strided else x.to(gpu), w.to(gpu), up_weight=wu.to(gpu))
        gate = F.linear(x.double(), w.double()).to(dtype)
        up = F.linear(x.double(), wu.double()).to(dtype)
        act = (gate.double() * torch.sigmoid(gate.double())).to(dtype)
        _check(y, act.double() * up.double(), dtype, ulps=3.0)
    else:
        b = torch.randn(N, generator=g).to(dtype) if bias else None
        y = linear_small_m(wide.to(gpu)[:, 32:32 + K] if strided else x.to(gpu), w.to(gpu), None if b is None else b.to(gpu))
        _check(y, F.linear(x.double(), w.double(), None if b is None else b.double()), dtype)
    assert y.shape == (M, N) and y.dtype == dtype


def test_linear_rejects_what_the_kernel_does_not_cover(gpu):
    x = torch.zeros(17, 64, dtype=torch.float16, device=gpu)
    w = torch.zeros(32, 64, dtype=torch.float16, device=gpu)
    with pytest.raises(RuntimeError):
        linear_small_m(x, w)                                    # 17 rows
    with pytest.raises(RuntimeError):
        linear_small_m(x[:4, :48].contiguous(), w[:, :48].contiguous())     # K not a multiple of 32
    with pytest.raises(RuntimeError):
        linear_small_m(x[:4], w[:24].contiguous())              # N not a multiple of 16
    with pytest.raises(RuntimeError):
        linear_small_m(x[:4].cpu(), w.cpu())


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("B,N,Nk,K,bias", [(8, 32, 8, 4096, False), (3, 4, 2, 512, True), (1, 7, 1, 896, True),
                                            (5, 8, 8, 8192, False), (8, 2, 1, 192, False)])
def test_qkv_rope_append_equals_projection_then_rotation(gpu, dtype, B, N, Nk, K, bias):
    """One launch against the two it replaces: the rotated query, the key row and the value row are the same bits;
    rows of the caches other than the written ones are untouched."""
    from polarquant_amd.decode_ops import linear_small_m, qkv_rope_append, rope_append
    g = torch.Generator().manual_seed(B * 1000 + N + K)
    x = torch.randn(B, 1, K, generator=g).to(dtype).to(gpu)
    w = (torch.randn((N + 2 * Nk) * 128, K, generator=g) / K ** 0.5).to(dtype).to(gpu)
    b = torch.randn((N + 2 * Nk) * 128, generator=g).to(dtype).to(gpu) if bias else None
    max_pos, k_rows, v_rows = 300, 128, 300
    ang = torch.arange(max_pos, dtype=torch.float32)[:, None] * (1e4 ** (-torch.arange(0, 128, 2).float() / 128))[None]
    emb = torch.cat([ang, ang], -1)
    cos, sin = emb.cos().to(dtype).to(gpu), emb.sin().to(dtype).to(gpu)
    pos = torch.tensor([257], device=gpu)
    k_row = torch.tensor([77], device=gpu)
    fill = torch.randn(B, Nk, k_rows, 128, generator=g).to(dtype).to(gpu)
    fillv = torch.randn(B, Nk, v_rows, 128, generator=g).to(dtype).to(gpu)
    k1, v1, k2, v2 = fill.clone(), fillv.clone(), fill.clone(), fillv.clone()
    qkv = linear_small_m(x, w, b)
    nq, nkv = N * 128, Nk * 128
    q_ref = rope_append(qkv[..., :nq], qkv[..., nq:nq + nkv], qkv[..., nq + nkv:], cos, sin, pos, k1, k_row, v1, pos, N, Nk)
    q_got = qkv_rope_append(x, w, b, cos, sin, pos, k2, k_row, v2, pos, N, Nk)
    torch.cuda.synchronize()
    assert q_got.shape == q_ref.shape and torch.equal(q_got, q_ref)
    assert torch.equal(k2, k1) and torch.equal(v2, v1)
    assert not torch.equal(k2[:, :, 77], fill[:, :, 77]) and torch.equal(k2[:, :, :77], fill[:, :, :77])
    # a strided x (rows of a wider tensor)
    wide = torch.zeros(B, 1, K + 64, dtype=dtype, device=gpu)
    wide[..., :K] = x
    k3, v3 = fill.clone(), fillv.clone()
    assert torch.equal(qkv_rope_append(wide[..., :K], w, b, cos, sin, pos, k3, k_row, v3, pos, N, Nk), q_ref)
    assert torch.equal(k3, k1) and torch.equal(v3, v1)
