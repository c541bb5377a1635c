"""pq_decode_attn_static (the entry point that allocates nothing: split partials in a device array
inside the library) against pq_decode_attn with a caller's workspace, both through the C ABI.

The two run the same kernels on the same inputs with the same split count, so the outputs must be
the same bits.  Two calls in a row, the second on a smaller input with fewer slices: the library's
buffer then still holds the first call's partials, which must not leak into the second result.
The first output is also held to the stated bar against the fp64 oracle (rtol 1e-2 / atol 1e-3).
"""
import math

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
    dev = [t.to(gpu).contiguous() for t in (q.reshape(B, N, 128), *quant, kres, v)]
    return dev, ref64


def _call(static, dev, B, N, Nk, n_groups, n_resid, n_splits, gpu, flags=0):
    q, codes, rs, rm, ts, tm, kres, v = dev
    out = torch.full((B, N, 128), float("nan"), dtype=torch.float16, device=gpu)
    head = [q.data_ptr(), codes.data_ptr(), rs.data_ptr(), rm.data_ptr(), ts.data_ptr(), tm.data_ptr(), n_groups,
            n_groups, None, kres.data_ptr(), kres.shape[2], n_resid, None, v.data_ptr(), v.shape[2], None, 0,
            1.0 / math.sqrt(128), B, N, Nk, 4, 4, _ffi.PQ_F16, n_splits, 0]
    lib = _ffi.lib()
    if static:
        rc = lib.pq_decode_attn_static(*head, out.data_ptr(), flags, None, _stream_ptr(gpu))
    else:
        nbytes = lib.pq_decode_attn_workspace_bytes(B, N, n_splits)
        ws = torch.full((nbytes // 4,), float("nan"), dtype=torch.float32, device=gpu)
        rc = lib.pq_decode_attn(*head, ws.data_ptr(), nbytes, out.data_ptr(), flags, None, _stream_ptr(gpu))
    assert rc == 0, _ffi.STATUS_NAMES.get(rc, rc)
    torch.cuda.synchronize()
    return out.cpu()


def test_static_entry_point_matches_workspace_entry_point(gpu):
    # first call: 2 sequences x 8 KV heads, 24 groups + 37 residual keys, 9 slices of 3 groups, so the last slice
    # holds nothing and takes the empty-partial path
    big = dict(B=2, N=32, Nk=8, n_groups=24, n_resid=37, n_splits=9)
    small = dict(B=1, N=32, Nk=8, n_groups=5, n_resid=3, n_splits=2)
    for i, (shape, seed) in enumerate(((big, 11), (small, 12))):
        print("pq_decode_attn_static call", i, shape, flush=True)
        dev, ref64 = _inputs(gpu, shape["B"], shape["N"], shape["Nk"], shape["n_groups"], shape["n_resid"], seed)
        got = _call(True, dev, gpu=gpu, **shape)
        want = _call(False, dev, gpu=gpu, **shape)
        assert torch.isfinite(got.float()).all()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), "call %d: outputs differ" % i
        err = (got.double().reshape(ref64.shape) - ref64).abs()
        assert bool((err <= 1e-3 + 1e-2 * ref64.abs()).all()), "call %d: off the oracle by %g" % (i, err.max().item())


def test_static_entry_point_with_balanced_slices(gpu):
    """The flags pass through: slices cut on the device (PQ_BALANCED_SLICES) leave some partial slots of the library's
    buffer unused, which the second, smaller call must not read as results of the first."""
    for i, (shape, seed) in enumerate(((dict(B=3, N=32, Nk=8, n_groups=9, n_resid=100, n_splits=6), 14),
                                       (dict(B=1, N=32, Nk=8, n_groups=2, n_resid=0, n_splits=3), 15))):
        print("pq_decode_attn_static balanced call", i, shape, flush=True)
        dev, ref64 = _inputs(gpu, shape["B"], shape["N"], shape["Nk"], shape["n_groups"], shape["n_resid"], seed)
        got = _call(True, dev, gpu=gpu, flags=_ffi.PQ_BALANCED_SLICES, **shape)
        want = _call(False, dev, gpu=gpu, flags=_ffi.PQ_BALANCED_SLICES, **shape)
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), "call %d: outputs differ" % i
        err = (got.double().reshape(ref64.shape) - ref64).abs()
        assert bool((err <= 1e-3 + 1e-2 * ref64.abs()).all()), "call %d: off the oracle by %g" % (i, err.max().item())


def test_static_entry_point_rejects_sizes_beyond_its_buffer(gpu):
    dev, _ = _inputs(gpu, 1, 32, 8, 2, 1, 13)
    q, codes, rs, rm, ts, tm, kres, v = dev
    out = torch.zeros(1, 32, 128, dtype=torch.float16, device=gpu)
    # 1 * 32 * 513 partials > 16384
    rc = _ffi.lib().pq_decode_attn_static(
        q.data_ptr(), codes.data_ptr(), rs.data_ptr(), rm.data_ptr(), ts.data_ptr(), tm.data_ptr(), 2, 2, None,
        kres.data_ptr(), kres.shape[2], 1, None, v.data_ptr(), v.shape[2], None, 0, 0.088, 1, 32, 8, 4, 4, _ffi.PQ_F16,
        513, 0, out.data_ptr(), 0, None, _stream_ptr(gpu))
    assert rc == -7          # PQ_ERR_WORKSPACE
