"""The hand-over between the scorer and the accumulator wavefront of the default decode-attention kernels when it
FAILS: with PQ_TEST_SILENT_SCORER the scorers publish no tile and the bounded waits give up after 1000 polls.  The
call must return (no wavefront waits for ever), its output must be NaN everywhere (a failed hand-over cannot pass
for a result), and the next ordinary call must be right again (nothing lingers in the library or on the device).
Nothing here makes the GPU fault or hang: every kernel runs to its normal end."""
import math
import time

import pytest
import torch

from oracle import polar_oracle as po
from polarquant_amd import _ffi
from polarquant_amd import workloads as wl
from polarquant_amd.kernel4group import _stream_ptr

pytestmark = pytest.mark.gpu


def _inputs(gpu, B, N, Nk, n_groups, n_resid, seed):
    g = torch.Generator().manual_seed(seed)
    L = n_groups * 128 + n_resid
    k = wl.make_keys(B, Nk, L, 5e5, g, torch.float16)
    q = wl.make_half((B, N, 1, 128), g, torch.float16)
    v = wl.make_half((B, Nk, L, 128), g, torch.float16)
    quant = po.quantize_and_pack_nbit(k[:, :, :n_groups * 128].contiguous(), 4, 4)
    kres = k[:, :, n_groups * 128:].contiguous()
    ref64 = po.decode_attention_exact(q, kres, *quant, v, None, 4, 4)
    return [t.to(gpu).contiguous() for t in (q.reshape(B, N, 128), *quant, kres, v)], ref64


def _call(dev, B, N, Nk, n_groups, n_resid, n_splits, gpu, flags, counts=None):
    q, codes, rs, rm, ts, tm, kres, v = dev
    out = torch.zeros((B, N, 128), dtype=torch.float16, device=gpu)
    lib = _ffi.lib()
    nbytes = lib.pq_decode_attn_workspace_bytes(B, N, n_splits)
    ws = torch.zeros((nbytes // 4,), dtype=torch.float32, device=gpu)
    gp, rp = (None, None) if counts is None else (counts[0].data_ptr(), counts[1].data_ptr())
    rc = lib.pq_decode_attn(q.data_ptr(), codes.data_ptr(), rs.data_ptr(), rm.data_ptr(), ts.data_ptr(), tm.data_ptr(),
                            n_groups, n_groups, gp, kres.data_ptr(), kres.shape[2], n_resid, rp, v.data_ptr(), v.shape[2],
                            None, 0, 1.0 / math.sqrt(128), B, N, Nk, 4, 4, _ffi.PQ_F16, n_splits, 0, ws.data_ptr(), nbytes,
                            out.data_ptr(), flags, _stream_ptr(gpu))
    assert rc == 0, _ffi.STATUS_NAMES.get(rc, rc)
    torch.cuda.synchronize()
    return out.cpu()


@pytest.mark.parametrize("balanced", [False, True])
def test_a_silent_scorer_times_out_and_poisons_the_result(gpu, balanced):
    shape = dict(B=2, N=32, Nk=8, n_groups=6, n_resid=37, n_splits=3)
    dev, ref64 = _inputs(gpu, shape["B"], shape["N"], shape["Nk"], shape["n_groups"], shape["n_resid"], 21)
    counts = None
    flags = 0
    if balanced:
        flags = _ffi.PQ_BALANCED_SLICES
        counts = (torch.full((2,), 6, dtype=torch.int32, device=gpu), torch.full((2,), 37, dtype=torch.int32, device=gpu))
    print("silent scorer, balanced =", balanced, flush=True)
    t0 = time.perf_counter()
    bad = _call(dev, gpu=gpu, flags=flags | _ffi.PQ_TEST_SILENT_SCORER, counts=counts, **shape)
    took = time.perf_counter() - t0
    assert bool(torch.isnan(bad.float()).all()), "a failed hand-over produced numbers"
    assert took < 5.0, took                     # 1000 polls per wait: milliseconds, not the half second of the real limit
    good = _call(dev, gpu=gpu, flags=flags, counts=counts, **shape)
    err = (good.double().reshape(ref64.shape) - ref64).abs()
    assert bool((err <= 1e-3 + 1e-2 * ref64.abs()).all()), float(err.max())


def test_the_hook_is_refused_where_it_means_nothing(gpu):
    # the score op has no hand-over
    P = 4096
    assert _ffi.lib().pq_validate_decode_scores(P, P, P, P, P, P, P, 2, 32, 8, 4, 4, 4, 0, _ffi.PQ_TEST_SILENT_SCORER) == -2
