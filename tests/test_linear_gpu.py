"""pq_linear_small_m (the decode step's projections at <= 16 rows) against fp32 torch matmuls of the
same half-precision operands.  Tolerance: the result is one rounding of an fp32 sum whose order differs
from the reference's, so at most one unit in the last place of the dtype, plus a little accumulation noise."""
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
