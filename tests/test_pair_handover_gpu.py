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
                            max(n_groups, 1), n_groups, gp, kres.data_ptr(), kres.shape[2], n_resid, rp, v.data_ptr(), v.shape[2],
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


@pytest.mark.parametrize("N,Nk,n_groups,n_resid", [(32, 8, 6, 37), (28, 4, 3, 0), (8, 8, 0, 5), (16, 8, 2, 128)])
def test_one_slice_per_plane_writes_the_output_without_a_merge(gpu, N, Nk, n_groups, n_resid):
    """With n_splits == 1 the default kernels of pq_decode_attn write the finished output themselves.  It must be, bit
    for bit, what the two-step form (pq_decode_attn_partials, then pq_decode_attn_merge) makes of the same call."""
    B = 3
    dev, ref64 = _inputs(gpu, B, N, Nk, max(n_groups, 1), n_resid, 31)
    q, codes, rs, rm, ts, tm, kres, v = dev
    if n_groups == 0:                                   # no quantized groups: only the residual window
        v = v[:, :, 128:].contiguous()
        g = torch.Generator().manual_seed(32)
        kres_cpu, v_cpu = kres.cpu(), v.cpu()
        ref64 = po.decode_attention_exact(q.cpu().reshape(B, N, 1, 128), kres_cpu, None, None, None, None, None, v_cpu, None, 4, 4)
        dev = [q, codes, rs, rm, ts, tm, kres, v]
    if n_resid == 0:
        dev[6] = torch.zeros(B, Nk, 128, 128, dtype=torch.float16, device=gpu)
    direct = _call(dev, B=B, N=N, Nk=Nk, n_groups=n_groups, n_resid=n_resid, n_splits=1, gpu=gpu, flags=0)
    # the same call in two steps
    q, codes, rs, rm, ts, tm, kres, v = dev
    lib = _ffi.lib()
    nbytes = lib.pq_decode_attn_workspace_bytes(B, N, 1)
    ws = torch.zeros((nbytes // 4,), dtype=torch.float32, device=gpu)
    out = torch.zeros((B, N, 128), dtype=torch.float16, device=gpu)
    rc = lib.pq_decode_attn_partials(q.data_ptr(), codes.data_ptr(), rs.data_ptr(), rm.data_ptr(), ts.data_ptr(), tm.data_ptr(),
                                     max(n_groups, 1), n_groups, None, kres.data_ptr(), kres.shape[2], n_resid, None, v.data_ptr(),
                                     v.shape[2], None, 0, 1.0 / math.sqrt(128), B, N, Nk, 4, 4, _ffi.PQ_F16, 1, 0, ws.data_ptr(),
                                     nbytes, 0, _stream_ptr(gpu))
    assert rc == 0
    rc = lib.pq_decode_attn_merge(ws.data_ptr(), nbytes, B, N, 1, _ffi.PQ_F16, out.data_ptr(), _stream_ptr(gpu))
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.equal(direct.view(torch.int16), out.cpu().view(torch.int16))
    err = (direct.double().reshape(ref64.shape) - ref64).abs()
    assert bool((err <= 1e-3 + 1e-2 * ref64.abs()).all()), float(err.max())


def test_a_silent_scorer_poisons_the_directly_written_output_too(gpu):
    shape = dict(B=2, N=32, Nk=8, n_groups=3, n_resid=9, n_splits=1)
    dev, _ = _inputs(gpu, 2, 32, 8, 3, 9, 33)
    bad = _call(dev, gpu=gpu, flags=_ffi.PQ_TEST_SILENT_SCORER, **shape)
    assert bool(torch.isnan(bad.float()).all())


def test_directly_written_output_under_a_replayed_graph(gpu):
    """One slice per plane inside a captured HIP graph: replays, with the inputs changed in place between them, must give
    what the eager call gives for the same inputs."""
    from polarquant_amd.attention import new_workspace, polar_decode_attention
    B, N, Nk, ng, nr = 2, 32, 8, 3, 9
    dev, _ = _inputs(gpu, B, N, Nk, ng, nr, 41)
    q, codes, rs, rm, ts, tm, kres, v = dev
    q = q.reshape(B, N, 1, 128).contiguous()
    ws = new_workspace(B, N, 1, gpu)
    out = torch.zeros(B, N, 1, 128, dtype=torch.float16, device=gpu)
    call = lambda o: polar_decode_attention(q, codes, rs, rm, ts, tm, kres, v, ng, nr, n_splits=1, out=o, workspace=ws)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call(out)                                            # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(out)
    g = torch.Generator(device=gpu).manual_seed(42)
    for i in range(3):
        q.copy_(torch.randn(q.shape, generator=g, device=gpu).half())
        v.mul_(0.5 + i)
        graph.replay()
        torch.cuda.synchronize()
        eager = torch.zeros_like(out)
        call(eager)
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), eager.view(torch.int16)), i
