"""The hand-over between the scorer and the accumulator wavefront of the default decode-attention kernels when it
FAILS: with PQ_TEST_SILENT_SCORER (honoured by the test build of the library only, libpolarquant_hip_testhooks.so)
the scorers publish no tile and the bounded waits give up after 1000 polls.  The call must return (no wavefront
waits for ever), its output must be NaN everywhere (a failed hand-over cannot pass for a result), the caller's
status word must say so, and the next ordinary call must be right again (nothing lingers in the library or on the
device).  Also here: the hand-over while another kernel of the same process shares the GPU on a second stream.
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


def _call(dev, gpu, **kw):
    """_launch, then wait for the device -> the output on the host."""
    out = _launch(dev, gpu=gpu, **kw)[0]
    torch.cuda.synchronize()
    return out.cpu()


def _launch(dev, B, N, Nk, n_groups, n_resid, n_splits, gpu, flags, counts=None, lib=None, status=None, ws_fill=0.0):
    """One pq_decode_attn call through the C ABI of `lib` (default: the shipping library), not waited for
    -> (output, workspace), both on the device.
    `status`: an int32 device tensor passed as the call's status word; `ws_fill`: what the workspace holds before."""
    q, codes, rs, rm, ts, tm, kres, v = dev
    out = torch.zeros((B, N, 128), dtype=torch.float16, device=gpu)
    lib = lib or _ffi.lib()
    nbytes = lib.pq_decode_attn_workspace_bytes(B, N, n_splits)
    ws = torch.full((nbytes // 4,), ws_fill, dtype=torch.float32, device=gpu)
    gp, rp = (None, None) if counts is None else (counts[0].data_ptr(), counts[1].data_ptr())
    rc = lib.pq_decode_attn(q.data_ptr(), codes.data_ptr(), rs.data_ptr(), rm.data_ptr(), ts.data_ptr(), tm.data_ptr(),
                            max(n_groups, 1), n_groups, gp, kres.data_ptr(), kres.shape[2], n_resid, rp, v.data_ptr(), v.shape[2],
                            None, 0, 1.0 / math.sqrt(128), B, N, Nk, 4, 4, _ffi.PQ_F16, n_splits, 0, ws.data_ptr(), nbytes,
                            out.data_ptr(), flags, None if status is None else status.data_ptr(), _stream_ptr(gpu))
    assert rc == 0, _ffi.STATUS_NAMES.get(rc, rc)
    return out, ws


@pytest.mark.parametrize("balanced", [False, True])
def test_a_silent_scorer_times_out_and_poisons_the_result(gpu, hooks_lib, balanced):
    shape = dict(B=2, N=32, Nk=8, n_groups=6, n_resid=37, n_splits=3)
    dev, ref64 = _inputs(gpu, shape["B"], shape["N"], shape["Nk"], shape["n_groups"], shape["n_resid"], 21)
    counts = None
    flags = 0
    if balanced:
        flags = _ffi.PQ_BALANCED_SLICES
        counts = (torch.full((2,), 6, dtype=torch.int32, device=gpu), torch.full((2,), 37, dtype=torch.int32, device=gpu))
    print("silent scorer, balanced =", balanced, flush=True)
    status = torch.zeros(1, dtype=torch.int32, device=gpu)
    t0 = time.perf_counter()
    bad = _call(dev, gpu=gpu, flags=flags | _ffi.PQ_TEST_SILENT_SCORER, counts=counts, lib=hooks_lib, status=status, **shape)
    took = time.perf_counter() - t0
    assert bool(torch.isnan(bad.float()).all()), "a failed hand-over produced numbers"
    assert int(status) == _ffi.PQ_STATUS_HANDOVER_TIMEOUT, "the host was not told of the failed hand-over"
    assert took < 5.0, took                     # 1000 polls per wait: milliseconds, not the half second of the real limit
    # the same call without the hook, through both builds: right again, and the status word stays clear
    for lib in (hooks_lib, None):
        status.zero_()
        good = _call(dev, gpu=gpu, flags=flags, counts=counts, lib=lib, status=status, **shape)
        assert int(status) == 0
        err = (good.double().reshape(ref64.shape) - ref64).abs()
        assert bool((err <= 1e-3 + 1e-2 * ref64.abs()).all()), float(err.max())


def test_a_failed_pair_poisons_every_plane_of_its_segment(gpu, hooks_lib):
    """Balanced slices over short ragged sequences: one segment holds pieces of several planes.  When the pair that
    works through it fails, EVERY one of those planes must come out NaN -- also the pieces after the one in which the
    wait gave up, whose partials would otherwise be whatever an earlier call left in the workspace (here: finite
    numbers, so that a piece nobody wrote would show as a finite output row)."""
    B, N, Nk = 3, 28, 4
    lens = [5, 130, 77]
    g = torch.Generator().manual_seed(51)
    k = wl.make_keys(B, Nk, 256, 1e6, g, torch.float16)
    q = wl.make_half((B, N, 1, 128), g, torch.float16)
    v = wl.make_half((B, Nk, 256, 128), g, torch.float16).to(gpu)
    # plane capacities: 1 group, 128 residual keys; sequence b holds lens[b] // 128 groups and lens[b] % 128 residual keys
    quant = po.quantize_and_pack_nbit(k[:, :, :128].contiguous(), 4, 4)
    kres = torch.zeros(B, Nk, 128, 128, dtype=torch.float16)
    for b, L in enumerate(lens):
        ng = L // 128
        kres[b, :, :L % 128] = k[b, :, ng * 128:L]
    counts = (torch.tensor([L // 128 for L in lens], dtype=torch.int32, device=gpu),
              torch.tensor([L % 128 for L in lens], dtype=torch.int32, device=gpu))
    dev = [t.to(gpu).contiguous() for t in (q.reshape(B, N, 128), *quant, kres)] + [v]
    shape = dict(B=B, N=N, Nk=Nk, n_groups=1, n_resid=0, n_splits=2)
    print("silent scorer, several planes per segment", flush=True)
    status = torch.zeros(1, dtype=torch.int32, device=gpu)
    bad = _call(dev, gpu=gpu, flags=_ffi.PQ_BALANCED_SLICES | _ffi.PQ_TEST_SILENT_SCORER, counts=counts, lib=hooks_lib,
                status=status, ws_fill=0.25, **shape)
    assert bool(torch.isnan(bad.float()).all()), "rows of a failed segment came out finite: %d of %d" % (
        int(torch.isfinite(bad.float()).sum()), bad.numel())
    assert int(status) == _ffi.PQ_STATUS_HANDOVER_TIMEOUT
    # and the ordinary call on the same inputs against the oracle, sequence by sequence
    status.zero_()
    good = _call(dev, gpu=gpu, flags=_ffi.PQ_BALANCED_SLICES, counts=counts, status=status, ws_fill=0.25, **shape)
    assert int(status) == 0
    for b, L in enumerate(lens):
        ng, nr = L // 128, L % 128
        qb = [t[b:b + 1, :, :ng] for t in quant] if ng else [None] * 5
        args = (q[b:b + 1], kres[b:b + 1, :, :nr] if nr else None, *qb, v[b:b + 1, :, :L].cpu(), None, 4, 4)
        ref = po.decode_attention_exact(*args)
        # (the reference rounds the scores of the un-quantized keys to fp16, :79, which these short sequences consist of)
        band = 1e-3 + 1e-2 * ref.abs() + po.residual_score_rounding_band(*args)
        err = (good[b:b + 1].double().reshape(ref.shape) - ref).abs()
        assert bool((err <= band).all()), (b, float(err.max()))


def test_the_hook_is_refused_where_it_means_nothing(gpu, hooks_lib):
    P = 4096
    for lib in (_ffi.lib(), hooks_lib):
        # the score op has no hand-over
        assert lib.pq_validate_decode_scores(P, P, P, P, P, P, P, 2, 32, 8, 4, 4, 4, 0, _ffi.PQ_TEST_SILENT_SCORER) == -2
    # the shipping library refuses the hook outright: its ABI cannot be asked for NaN
    dev, _ = _inputs(gpu, 1, 32, 8, 2, 3, 22)
    q, codes, rs, rm, ts, tm, kres, v = dev
    out = torch.zeros(1, 32, 128, dtype=torch.float16, device=gpu)
    ws = torch.zeros(_ffi.lib().pq_decode_attn_workspace_bytes(1, 32, 2) // 4, dtype=torch.float32, device=gpu)
    rc = _ffi.lib().pq_decode_attn(q.data_ptr(), codes.data_ptr(), rs.data_ptr(), rm.data_ptr(), ts.data_ptr(), tm.data_ptr(),
                                   2, 2, None, kres.data_ptr(), kres.shape[2], 3, None, v.data_ptr(), v.shape[2], None, 0, 0.088,
                                   1, 32, 8, 4, 4, _ffi.PQ_F16, 2, 0, ws.data_ptr(), ws.numel() * 4, out.data_ptr(),
                                   _ffi.PQ_TEST_SILENT_SCORER, None, _stream_ptr(gpu))
    assert rc == -2


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
                                     nbytes, 0, None, _stream_ptr(gpu))
    assert rc == 0
    rc = lib.pq_decode_attn_merge(ws.data_ptr(), nbytes, B, N, 1, _ffi.PQ_F16, out.data_ptr(), _stream_ptr(gpu))
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.equal(direct.view(torch.int16), out.cpu().view(torch.int16))
    err = (direct.double().reshape(ref64.shape) - ref64).abs()
    assert bool((err <= 1e-3 + 1e-2 * ref64.abs()).all()), float(err.max())


def test_a_silent_scorer_poisons_the_directly_written_output_too(gpu, hooks_lib):
    shape = dict(B=2, N=32, Nk=8, n_groups=3, n_resid=9, n_splits=1)
    dev, _ = _inputs(gpu, 2, 32, 8, 3, 9, 33)
    status = torch.zeros(1, dtype=torch.int32, device=gpu)
    bad = _call(dev, gpu=gpu, flags=_ffi.PQ_TEST_SILENT_SCORER, lib=hooks_lib, status=status, **shape)
    assert bool(torch.isnan(bad.float()).all())
    assert int(status) == _ffi.PQ_STATUS_HANDOVER_TIMEOUT


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


def test_pairs_with_another_kernel_sharing_the_gpu(gpu):
    """The scorer / accumulator kernels while a second stream of the same process keeps the GPU busy with another
    kernel (a loop of plain streaming reads whose workgroups take and leave compute units all the time): the placement
    of a workgroup's eight wavefronts and the bounded waits of the hand-over must not depend on having the device to
    themselves.  Every call is held to the oracle and to a clear status word; the test stops at the first failure."""
    B, N, Nk, ng, nr = 4, 32, 8, 24, 37
    dev, ref64 = _inputs(gpu, B, N, Nk, ng, nr, 61)
    blib = _ffi.bench_lib()
    filler = torch.empty(256 << 20, dtype=torch.uint8, device=gpu).fill_(1)
    sink = torch.zeros(1, dtype=torch.int32, device=gpu)
    side = torch.cuda.Stream()
    status = torch.zeros(1, dtype=torch.int32, device=gpu)
    torch.cuda.synchronize()
    print("co-tenancy: attention on the current stream, streaming reads on a second one", flush=True)
    for rnd, (n_waves, flags, counts) in enumerate([
            (256, 0, None), (1024, 0, None), (3072, 0, None),
            (1024, _ffi.PQ_BALANCED_SLICES, (torch.full((B,), ng, dtype=torch.int32, device=gpu),
                                             torch.full((B,), nr, dtype=torch.int32, device=gpu)))]):
        # both queues are filled without waiting for the device: 12 streaming reads of 256 MiB (~40 us each) on the side
        # stream for every attention call (~30 us) on the main one, 24 times over; then one wait, and every output checked
        held = []
        for rep in range(24):
            for _ in range(12):
                got = blib.pq_stream_read(filler.data_ptr(), filler.numel(), n_waves, sink.data_ptr(), side.cuda_stream)
                assert got > 0
            held.append(_launch(dev, B=B, N=N, Nk=Nk, n_groups=ng, n_resid=nr, n_splits=8, gpu=gpu, flags=flags,
                                counts=counts, status=status))
        torch.cuda.synchronize()
        assert int(status) == 0, rnd
        for rep, (out, _) in enumerate(held):
            err = (out.cpu().double().reshape(ref64.shape) - ref64).abs()
            assert bool((err <= 1e-3 + 1e-2 * ref64.abs()).all()), (rnd, rep, float(err.max()))
    torch.cuda.synchronize()
