"""GPU parity of pq_decode_scores (through the C ABI) against the CPU oracle.

Tolerance: scores within 1e-3 relative in fp32 (the path's stated bar), taken
relative to the largest |score| of the (batch, head) row, and in practice met
with two orders of magnitude to spare (asserted at 2e-5).
"""
import pytest
import torch

from oracle import polar_oracle as po
from polarquant_amd import workloads as wl
from polarquant_amd.kernel4group import attention_decode_forward_triton_impl

pytestmark = pytest.mark.gpu


def _rel_err(got, ref):
    scale = ref.abs().amax(dim=-1, keepdim=True).clamp_min(1e-30)
    return ((got.double() - ref.double()).abs() / scale).max().item()


def _run(gpu, q, quant, rbits, tbits):
    dev = [t.to(gpu) for t in (q,) + tuple(quant)]
    out = attention_decode_forward_triton_impl(*dev, rbits=rbits, tbits=tbits)
    torch.cuda.synchronize()
    return out.cpu()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("heads,kv,rbits,tbits", [(32, 32, 4, 4), (32, 8, 4, 4), (28, 4, 3, 3), (16, 8, 4, 4),
                                                  (8, 1, 5, 3), (6, 2, 2, 2), (5, 1, 4, 4), (12, 2, 4, 4), (3, 1, 4, 1),
                                                  # more than 16 angle bins: the wide table (32-128 KiB)
                                                  (8, 1, 2, 6), (32, 8, 3, 5), (6, 2, 2, 5), (7, 1, 1, 6), (2, 2, 2, 6),
                                                  # 128 angle bins: four heads per table, more heads in two launches
                                                  (4, 1, 1, 7), (3, 1, 1, 7), (8, 1, 1, 7), (14, 2, 1, 7), (10, 2, 1, 7), (2, 2, 1, 7)])
def test_scores_match_oracle(gpu, dtype, heads, kv, rbits, tbits):
    print("case", dtype, heads, kv, rbits, tbits, flush=True)
    g = torch.Generator().manual_seed(7)
    B, L = 2, 512
    k = wl.make_keys(B, kv, L, 1e4, g, dtype)
    q = wl.make_half((B, heads, 1, 128), g, dtype)
    quant = po.quantize_and_pack_nbit(k, rbits, tbits)
    ref = po.decode_scores(q, *quant, rbits=rbits, tbits=tbits, dtype=torch.float64)
    got = _run(gpu, q, quant, rbits, tbits)
    assert got.shape == (B, heads, 1, L) and got.dtype == torch.float32
    assert _rel_err(got, ref) < 2e-5


def test_scores_cfg0_full(gpu):
    """Workload configs[0]: batch 1, 32 heads MHA, context 4096, 4/4 bits."""
    sh = wl.CONFIGS[0]
    inp = wl.make_decode_inputs(sh)
    quant = po.quantize_and_pack_nbit(inp.k, sh.rbits, sh.tbits)
    ref = po.decode_scores(inp.q, *quant, dtype=torch.float64)
    got = _run(gpu, inp.q, quant, 4, 4)
    assert got.shape == (1, 32, 1, 4096)
    assert _rel_err(got, ref) < 2e-5


def test_scores_random_codes_and_metadata(gpu):
    """The reference micro-benchmark feeds random codes in [0,250) and randn
    metadata, negative scales included (benchmark/benchmark_matmul.py:94-99)."""
    g = torch.Generator().manual_seed(11)
    B, N, Nk, Nb = 2, 32, 8, 3
    codes = torch.randint(0, 250, (B, Nk, Nb, 128, 64), generator=g, dtype=torch.uint8)
    meta = [torch.randn(B, Nk, Nb, 1, 64, generator=g).half() for _ in range(4)]
    meta[0][0, 0, 0, 0, :8] = 0          # rscale == 0: degenerate radius range
    meta[2][0, 0, 0, 0, 8:16] = 0        # tscale == 0: degenerate angle range
    q = torch.randn(B, N, 1, 128, generator=g).half()
    ref = po.decode_scores(q, codes, *meta, dtype=torch.float64)
    got = _run(gpu, q, (codes, *meta), 4, 4)
    assert _rel_err(got, ref) < 2e-5


def test_scores_linearity_in_query(gpu):
    """Size-independent property: scores are linear in q (q1+q2 exact in half)."""
    g = torch.Generator().manual_seed(3)
    k = wl.make_keys(1, 8, 2048, 5e5, g)
    quant = po.quantize_and_pack_nbit(k)
    q1 = (torch.randint(-8, 9, (1, 32, 1, 128), generator=g).float() / 4).half()
    q2 = (torch.randint(-8, 9, (1, 32, 1, 128), generator=g).float() / 4).half()
    s1, s2, s12 = (_run(gpu, q, quant, 4, 4) for q in (q1, q2, q1 + q2))
    assert _rel_err(s1 + s2, s12) < 1e-5
