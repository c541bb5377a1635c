"""The C ABI without a GPU: the library loads, exports every symbol that
include/polarquant.h declares, and its host-side argument checks return the
documented error codes.  No kernel is launched here."""
import ctypes
import os
import re

import pytest

from polarquant_amd import _ffi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
P = 0x7f0000000000          # a fake, 4 KiB-aligned "device pointer": the validators never dereference


@pytest.fixture(scope="module")
def lib():
    return _ffi.lib()


def _declared_functions(header="polarquant.h"):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(pq_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound(lib):
    names = _declared_functions()
    assert len(names) >= 12
    raw = ctypes.CDLL(_ffi.LIB_PATH)
    for n in names:
        assert hasattr(raw, n), "libpolarquant_hip.so does not export %s" % n
        assert n in _ffi.SIGNATURES, "%s is declared in the header but has no ctypes signature" % n
    assert set(_ffi.SIGNATURES) == set(names)
    # the measurement aids live in a library of their own, not in the product ABI
    bench_names = _declared_functions("polarquant_bench.h")
    assert bench_names == sorted(_ffi.BENCH_SIGNATURES) and not set(bench_names) & set(names)
    raw_bench = ctypes.CDLL(_ffi.BENCH_LIB_PATH)
    for n in bench_names:
        assert hasattr(raw_bench, n) and not hasattr(raw, n)


def test_version_and_status_strings(lib):
    assert lib.pq_version() >= 100
    for code in range(0, -10, -1):
        assert lib.pq_status_string(code)
    assert b"unknown" in lib.pq_status_string(-99)


def test_validate_decode_scores(lib):
    ok = [P, P, P, P, P, P, P, 2, 32, 8, 4, 4, 4, 0, 0]
    assert lib.pq_validate_decode_scores(*ok) == 0

    def bad(i, v):
        a = list(ok); a[i] = v
        return lib.pq_validate_decode_scores(*a)
    assert bad(0, None) == -1 and bad(6, None) == -1                 # null pointers
    assert bad(7, 0) == -2 and bad(9, 5) == -2 and bad(10, 0) == -2   # B<=0, N % Nk, Nb<=0
    assert bad(8, 72) == -2                                          # rep 9 > 8
    assert bad(11, 5) == -3 and bad(12, 5) == -3 and bad(12, 0) == -3  # r+t>8 (twice), tbits<1
    # every split the reference takes (rbits + tbits <= 8), 1/7 included
    for rb, tb, want in ((3, 5, 0), (2, 6, 0), (1, 6, 0), (4, 1, 0), (7, 1, 0), (1, 7, 0), (2, 7, -3), (1, 8, -3), (0, 4, -3)):
        assert lib.pq_validate_decode_scores(*ok[:11], rb, tb, 0, 0) == want, (rb, tb)
    assert b"rbits + tbits <= 8" in lib.pq_status_string(-3)
    assert bad(13, 2) == -4                                          # dtype
    assert bad(1, P + 4) == -5 and bad(6, P + 2) == -5               # misaligned codes / out
    # the launching entry point runs the same checks before touching the device
    assert lib.pq_decode_scores(*ok[:11], 5, 4, 0, 0, None) == -3
    # packed 6-bit code rows: tbits == 3 and rbits <= 3 only; unknown flag bits are refused
    assert lib.pq_validate_decode_scores(*ok[:11], 3, 3, 0, 4) == 0
    assert lib.pq_validate_decode_scores(*ok[:11], 4, 4, 0, 4) == -3 and lib.pq_validate_decode_scores(*ok[:11], 4, 3, 0, 4) == -3
    assert lib.pq_validate_decode_scores(*ok[:11], 3, 3, 0, 8) == -2


def test_validate_quantize_groups(lib):
    strides = (ctypes.c_int64 * 4)(8 * 256 * 128, 256 * 128, 128, 1)
    sp = ctypes.cast(strides, ctypes.c_void_p)
    ok = [P, sp, 0, 2, 8, 2, 4, 4, 0, P, P, P, P, P, 2, 0]
    assert lib.pq_validate_quantize_groups(*ok) == 0

    def bad(i, v):
        a = list(ok); a[i] = v
        return lib.pq_validate_quantize_groups(*a)
    assert bad(0, None) == -1 and bad(1, None) == -1 and bad(9, None) == -1
    assert bad(3, 0) == -2 and bad(5, 0) == -2
    assert bad(6, 5) == -3 and bad(7, 0) == -3
    # the quantizer takes every split the decode entry points read
    a = list(ok); a[6], a[7] = 2, 5
    assert lib.pq_validate_quantize_groups(*a) == 0
    a[6], a[7] = 2, 6
    assert lib.pq_validate_quantize_groups(*a) == 0
    a[6], a[7] = 1, 7
    assert lib.pq_validate_quantize_groups(*a) == 0
    a[6], a[7] = 2, 7
    assert lib.pq_validate_quantize_groups(*a) == -3
    assert bad(2, 7) == -4
    assert bad(8, 1) == 0 and bad(8, 2) == 0 and bad(8, 3) == 0   # PQ_WRAP_FP32, PQ_ANGLE_UNIFORM
    assert bad(8, 4) == -3                           # packed 6-bit codes need rbits + tbits <= 6
    a = list(ok); a[6], a[7], a[8] = 3, 3, 4
    assert lib.pq_validate_quantize_groups(*a) == 0
    assert bad(8, 8) == 0 and bad(8, 9) == 0         # PQ_DEVICE_ATAN2, PQ_EAGER_GPU
    assert bad(8, 16) == -2                          # unknown flag bit
    assert bad(14, 1) == -6 and bad(15, 1) == -6     # capacity < offset + Nb
    assert bad(0, P + 2) == -5                       # key pointer not 8-byte aligned
    for i, s in enumerate([(8 * 256 * 128, 256 * 128, 128, 2), (8 * 256 * 128, 256 * 128, 64, 1),
                           (8 * 256 * 128 + 2, 256 * 128, 128, 1)]):
        st = (ctypes.c_int64 * 4)(*s)
        a = list(ok); a[1] = ctypes.cast(st, ctypes.c_void_p)
        assert lib.pq_validate_quantize_groups(*a) == (-6 if i < 2 else -5)
    # transposed [B,L,Nk,128] view: token stride Nk*128
    st = (ctypes.c_int64 * 4)(256 * 8 * 128, 128, 8 * 128, 1)
    a = list(ok); a[1] = ctypes.cast(st, ctypes.c_void_p)
    assert lib.pq_validate_quantize_groups(*a) == 0


def test_validate_decode_attn_and_plan(lib, hooks_lib):
    B, N, Nk, ns = 2, 32, 8, 4
    wsb = lib.pq_decode_attn_workspace_bytes(B, N, ns)
    assert wsb == B * N * ns * 132 * 4
    ok = [P, P, P, P, P, P, 4, 3, None, P, 128, 5, None, P, 1024, None, 0, 0.088, B, N, Nk, 4, 4, 0, ns, 0, P, wsb, P, 0]
    assert lib.pq_validate_decode_attn(*ok) == 0
    a = list(ok); a[21], a[22], a[29] = 3, 3, 4
    assert lib.pq_validate_decode_attn(*a) == 0                      # packed 6-bit codes with 3/3 bits
    a[21] = 4
    assert lib.pq_validate_decode_attn(*a) == -3
    for rb, tb, want in ((3, 5, 0), (2, 6, 0), (1, 7, 0), (2, 7, -3)):
        a = list(ok); a[21], a[22] = rb, tb
        assert lib.pq_validate_decode_attn(*a) == want, (rb, tb)

    def bad(i, v):
        a = list(ok); a[i] = v
        return lib.pq_validate_decode_attn(*a)
    assert bad(0, None) == -1 and bad(13, None) == -1 and bad(26, None) == -1 and bad(28, None) == -1
    assert bad(1, None) == -1            # groups > 0 but no codes
    assert bad(9, None) == -1            # residual > 0 but no residual keys
    assert bad(7, 5) == -6               # n_groups > capacity
    assert bad(11, 129) == -6            # n_resid > capacity
    assert bad(14, 3 * 128 + 4) == -6    # V capacity below tokens
    assert bad(24, 0) == -7 and bad(27, wsb - 1) == -7 and bad(25, -1) == -7
    assert bad(20, 5) == -2 and bad(22, 5) == -3 and bad(23, 3) == -4
    assert bad(13, P + 8) == -5
    assert bad(14, (1 << 24) + 1) == -2 and bad(6, (1 << 17) + 1) == -2      # plane too large for 32-bit offsets
    # the value plane's byte size is a 32-bit field (2^24 rows of 256 bytes would read as 0 bytes: every value
    # a silent zero) and the parking offset 0xFFFF0000 of loads that must read nothing has to lie past it
    max_rows = (1 << 24) - 256
    assert max_rows * 256 == 0xFFFF0000
    assert bad(14, max_rows) == 0 and bad(14, max_rows + 1) == -2 and bad(14, 1 << 24) == -2
    assert bad(10, max_rows) == 0 and bad(10, max_rows + 1) == -2 and bad(10, 1 << 24) == -2
    # slices cut on the device: a flag of the attention entry points only, and at least two partial slots per head
    a = list(ok); a[29] = 16
    assert lib.pq_validate_decode_attn(*a) == 0
    a[24], a[27] = 1, lib.pq_decode_attn_workspace_bytes(B, N, 1)
    assert lib.pq_validate_decode_attn(*a) == -7
    a = list(ok); a[29] = 32
    assert lib.pq_validate_decode_attn(*a) == 0                      # PQ_SINGLE_WAVEFRONT, alone or with balanced slices
    a[29] = 32 | 16
    assert lib.pq_validate_decode_attn(*a) == 0
    assert lib.pq_validate_decode_scores(P, P, P, P, P, P, P, 2, 32, 8, 4, 4, 4, 0, 32) == -2
    # PQ_TEST_SILENT_SCORER, the hook that turns a call's output into NaN: the shipping library refuses it like any
    # unknown flag; the test build takes it, but not where there is no hand-over to silence
    a = list(ok); a[29] = 0x40000000
    assert lib.pq_validate_decode_attn(*a) == -2
    hooks = hooks_lib
    assert hooks.pq_validate_decode_attn(*a) == 0
    a[29] = 0x40000000 | 32
    assert hooks.pq_validate_decode_attn(*a) == -2                   # with PQ_SINGLE_WAVEFRONT
    a[29] = 0x40000000 | 16
    assert hooks.pq_validate_decode_attn(*a) == 0                    # with balanced slices
    # balanced slices count the batch's units in 32 bits: capacities that could hold 2^31 of them are refused
    a = list(ok); a[29] = 16; a[6] = 1 << 17; a[18], a[19], a[20] = 4095, 16, 16; a[27] = lib.pq_decode_attn_workspace_bytes(4095, 16, 4)
    assert lib.pq_validate_decode_attn(*a) == -2
    a[29] = 0
    assert lib.pq_validate_decode_attn(*a) == 0                      # even slices have no such line
    a[29], a[21], a[22] = 0x40000000, 3, 5
    assert hooks.pq_validate_decode_attn(*a) == -2                   # 5 angle bits run the one-wavefront kernels
    a = list(ok); a[29] = 64
    assert lib.pq_validate_decode_attn(*a) == -2                     # unknown flag bit
    assert lib.pq_validate_decode_scores(P, P, P, P, P, P, P, 2, 32, 8, 4, 4, 4, 0, 16) == -2
    assert bad(0, P + 8) == -5                                       # q rows are read as 16-byte pieces
    a = list(ok); a[15] = P; a[16] = 100          # mask row shorter than the context
    assert lib.pq_validate_decode_attn(*a) == -6
    # no quantized groups yet: codes may be NULL
    a = list(ok); a[1:6] = [None] * 5; a[6] = 0; a[7] = 0
    assert lib.pq_validate_decode_attn(*a) == 0
    # plan: fills 4 wavefront slots per CU exactly once, never more splits than groups
    assert lib.pq_decode_attn_plan(16, 8, 256, 256) == 8
    assert lib.pq_decode_attn_plan(1, 8, 1024, 256) == 128
    assert lib.pq_decode_attn_plan(64, 4, 64, 256) == 4
    assert lib.pq_decode_attn_plan(1, 8, 3, 256) == 3
    assert lib.pq_decode_attn_plan(512, 8, 64, 256) == 1
    assert lib.pq_decode_attn_merge(None, 0, 1, 1, 1, 0, None, None) == -1


def test_validate_value_quantizer_and_v4_attention(lib, hooks_lib):
    strides = (ctypes.c_int64 * 4)(8 * 300 * 128, 300 * 128, 128, 1)
    sp = ctypes.cast(strides, ctypes.c_void_p)
    ok = [P, sp, 0, 2, 8, 300, P, P, P, 512, 100]
    assert lib.pq_validate_quantize_values(*ok) == 0

    def bad(i, v):
        a = list(ok); a[i] = v
        return lib.pq_validate_quantize_values(*a)
    assert bad(0, None) == -1 and bad(1, None) == -1 and bad(6, None) == -1 and bad(7, None) == -1 and bad(8, None) == -1
    assert bad(3, 0) == -2 and bad(5, 0) == -2 and bad(2, 3) == -4
    assert bad(9, 399) == -6 and bad(10, -1) == -6          # capacity < offset + T
    assert bad(0, P + 8) == -5                               # rows are read as 16-byte pieces
    st = (ctypes.c_int64 * 4)(8 * 300 * 128, 300 * 128, 132, 1)
    a = list(ok); a[1] = ctypes.cast(st, ctypes.c_void_p)
    assert lib.pq_validate_quantize_values(*a) == -5
    st = (ctypes.c_int64 * 4)(300 * 8 * 128, 128, 8 * 128, 1)   # transposed [B,T,Nk,128] view
    a = list(ok); a[1] = ctypes.cast(st, ctypes.c_void_p)
    assert lib.pq_validate_quantize_values(*a) == 0

    B, N, Nk, ns = 2, 32, 8, 4
    wsb = lib.pq_decode_attn_workspace_bytes(B, N, ns)
    ok = [P, P, P, P, P, P, 4, 3, None, P, 128, 5, None, P, P, P, P, 512, None, 0, 0.088, B, N, Nk, 4, 4, 0, ns, 0, P, wsb, P, 0]
    assert lib.pq_validate_decode_attn_v4(*ok) == 0

    def bad4(i, v):
        a = list(ok); a[i] = v
        return lib.pq_validate_decode_attn_v4(*a)
    assert bad4(13, None) == -1                               # residual window without values
    assert bad4(14, None) == -1 and bad4(15, None) == -1 and bad4(16, None) == -1   # groups without 4-bit values
    assert bad4(17, 3 * 128 - 1) == -6                        # value-code capacity below the quantized tokens
    assert bad4(0, None) == -1 and bad4(1, None) == -1 and bad4(7, 5) == -6 and bad4(27, 0) == -7
    assert bad4(13, P + 8) == -5
    a = list(ok); a[1:6] = [None] * 5; a[6] = 0; a[7] = 0; a[14:17] = [None] * 3; a[17] = 0
    assert lib.pq_validate_decode_attn_v4(*a) == 0            # nothing quantized yet
    # balanced slices and the choice of the kernel form as for half-precision values; the test hook into the hand-over
    # exists for the half-precision-value entry points only and is refused here instead of silently ignored (in the test
    # build too)
    assert bad4(32, 16) == 0 and bad4(32, 32) == 0 and bad4(32, 0x40000000) == -2
    # the largest stores: 2^24 - 256 rows of packed values, as many whole groups of codes as fit under that
    a = list(ok); a[6], a[17] = ((1 << 24) - 256) // 128, (1 << 24) - 256
    assert lib.pq_validate_decode_attn_v4(*a) == 0
    a[17] += 1
    assert lib.pq_validate_decode_attn_v4(*a) == -2
    a = list(ok); a[32] = 0x40000000
    assert hooks_lib.pq_validate_decode_attn_v4(*a) == -2
    # two wavefronts per SIMD for up to 4 query heads per KV head, one beyond
    assert lib.pq_decode_attn_v4_plan(16, 32, 8, 256, 256) == 16
    assert lib.pq_decode_attn_v4_plan(64, 28, 4, 64, 256) == 4
    assert lib.pq_decode_attn_v4_plan(1, 32, 8, 3, 256) == 3


def test_fused_decode_ops_reject_bad_arguments(lib):
    """Argument checks of the elementwise entry points run before any launch."""
    ok = [P, P, P, P, P, 4096, P, P, P, 128, P, P, 4096, P, 2, 32, 8, 0, 0, 0, None]
    def bad(i, v):
        a = list(ok); a[i] = v
        return lib.pq_rope_append(*a)
    for i in (0, 1, 2, 3, 4, 6, 7, 8, 10, 11, 13):
        assert bad(i, None) == -1, i
    assert bad(14, 0) == -2 and bad(15, 0) == -2 and bad(16, 0) == -2
    assert bad(17, 2) == -4
    assert bad(5, 0) == -6 and bad(9, 0) == -6 and bad(12, 0) == -6
    assert bad(18, 100) == -6 and bad(19, 100) == -6                 # row strides shorter than a row
    assert lib.pq_rmsnorm(None, None, P, P, None, 2, 4096, 1e-5, 0, None) == -1
    assert lib.pq_rmsnorm(P, None, None, P, None, 2, 4096, 1e-5, 0, None) == -1
    assert lib.pq_rmsnorm(P, None, P, P, None, 0, 4096, 1e-5, 0, None) == -2
    assert lib.pq_rmsnorm(P, None, P, P, None, 2, 4100, 1e-5, 0, None) == -2      # hidden % 8
    assert lib.pq_rmsnorm(P, None, P, P, None, 2, 4096, 1e-5, 5, None) == -4
    assert lib.pq_rmsnorm(P + 2, None, P, P, None, 2, 4096, 1e-5, 0, None) == -5
    assert lib.pq_silu_mul(None, P, P, 2, 64, 0, 0, None) == -1
    assert lib.pq_silu_mul(P, P, P, 0, 64, 0, 0, None) == -2 and lib.pq_silu_mul(P, P, P, 2, 12, 0, 0, None) == -2
    assert lib.pq_silu_mul(P, P, P, 2, 64, 0, 9, None) == -4 and lib.pq_silu_mul(P, P + 4, P, 2, 64, 0, 0, None) == -5
    assert lib.pq_silu_mul(P, P, P, 2, 64, 32, 0, None) == -6                      # rows would overlap


def test_linear_small_m_rejects_bad_arguments(lib):
    ok = [P, 4096, P, None, None, P, 4096, 8, 4096, 4096, 1]
    assert lib.pq_validate_linear_small_m(*ok) == 0
    def bad(i, v):
        a = list(ok)
        a[i] = v
        return lib.pq_validate_linear_small_m(*a)
    assert bad(0, None) == -1 and bad(2, None) == -1 and bad(5, None) == -1
    assert bad(10, 2) == -4                                             # dtype
    assert bad(7, 0) == -2 and bad(7, 17) == -2                         # rows
    assert bad(8, 4100) == -2 and bad(9, 4100) == -2 and bad(9, 16) == -2   # N % 16, K % 32
    assert bad(1, 4000) == -6 and bad(1, 4100) == -6 and bad(6, 4000) == -6 and bad(6, 4098) == -6   # strides
    assert bad(0, P + 8) == -5 and bad(2, P + 2) == -5 and bad(5, P + 4) == -5 and bad(3, P + 8) == -5
    gated_with_bias = list(ok)
    gated_with_bias[3], gated_with_bias[4] = P, P
    assert lib.pq_validate_linear_small_m(*gated_with_bias) == -2
    assert lib.pq_linear_small_m(None, 4096, P, None, None, P, 4096, 8, 4096, 4096, 1, None) == -1


def test_qkv_rope_append_rejects_bad_arguments(lib):
    #     x  stride  w  bias  M  K     dt cos sin rows pos q  k  krows krow v  vrows vrow N   Nk
    ok = [P, 4096, P, None, 8, 4096, 0, P, P, 4096, P, P, P, 128, P, P, 4096, P, 32, 8]
    assert lib.pq_validate_qkv_rope_append(*ok) == 0
    def bad(i, v):
        a = list(ok)
        a[i] = v
        return lib.pq_validate_qkv_rope_append(*a)
    for i in (0, 2, 7, 8, 10, 11, 12, 14, 15, 17):
        assert bad(i, None) == -1, i
    assert bad(6, 3) == -4
    assert bad(4, 0) == -2 and bad(4, 9) == -2 and bad(5, 4128) == -2 and bad(5, 0) == -2     # rows, K % 64
    assert bad(18, 0) == -2 and bad(19, 0) == -2
    assert bad(1, 4000) == -6 and bad(1, 4100) == -6 and bad(9, 0) == -6 and bad(13, 0) == -6 and bad(16, -1) == -6
    assert bad(0, P + 8) == -5 and bad(2, P + 2) == -5 and bad(11, P + 4) == -5 and bad(10, P + 4) == -5 and bad(3, P + 1) == -5
    assert lib.pq_qkv_rope_append(*(ok[:2] + [None] + ok[3:] + [None])) == -1


def test_stream_read_rejects_bad_arguments():
    lib = _ffi.bench_lib()
    assert lib.pq_stream_read(None, 1 << 30, 1024, P, None) == 0 and lib.pq_stream_read(P, 1 << 30, 1024, None, None) == 0
    assert lib.pq_stream_read(P, 1 << 30, 0, P, None) == 0 and lib.pq_stream_read(P + 8, 1 << 30, 1024, P, None) == 0
    assert lib.pq_stream_read(P, 1000, 1024, P, None) == 0          # less than one 16 KiB trip per wavefront


def test_rope_qk_rejects_bad_arguments(lib):
    ok = [P, 0, P, 0, P, P, 0, P, P, 2, 300, 32, 8, 1]
    def call(a):
        return lib.pq_rope_qk(*a, None)
    def bad(i, v):
        a = list(ok)
        a[i] = v
        return call(a)
    for i in (0, 2, 4, 5, 7, 8):
        assert bad(i, None) == -1, i
    assert bad(13, 2) == -4
    assert bad(9, 0) == -2 and bad(10, 0) == -2 and bad(11, 0) == -2 and bad(12, 0) == -2
    assert bad(1, 4000) == -6 and bad(1, 4100) == -6 and bad(3, 1000) == -6 and bad(6, 128) == -6 and bad(6, 300 * 128 + 4) == -6
    assert bad(0, P + 8) == -5 and bad(4, P + 2) == -5 and bad(8, P + 4) == -5


def test_attn_load_replica_rejects_bad_arguments():
    lib = _ffi.bench_lib()
    ok = [P, P, 128, 32768, 32769, 32768, 8, P]
    def bad(i, v):
        a = list(ok)
        a[i] = v
        return lib.pq_attn_load_replica(*a, None)
    assert bad(0, None) == 0 and bad(1, None) == 0 and bad(7, None) == 0 and bad(0, P + 8) == 0
    assert bad(2, 0) == 0 and bad(6, 0) == 0 and bad(5, 0) == 0
    assert bad(5, 40000) == 0                       # more tokens than a plane holds
    assert bad(4, 1 << 24) == 0 and bad(3, 1 << 26) == 0   # a plane a 32-bit byte offset cannot span
    assert bad(6, 512) == 0                         # slices shorter than two tiles


def test_convert_codes6_rejects_bad_arguments(lib):
    assert lib.pq_convert_codes6(None, P, 4, 1, None) == -1 and lib.pq_convert_codes6(P, None, 4, 0, None) == -1
    assert lib.pq_convert_codes6(P, P, 0, 1, None) == -2
    assert lib.pq_convert_codes6(P + 4, P, 4, 1, None) == -5 and lib.pq_convert_codes6(P, P + 4, 4, 0, None) == -5


def test_python_wrappers_refuse_cpu_tensors():
    import torch
    from polarquant_amd.attention import polar_decode_attention
    from polarquant_amd.kernel4group import attention_decode_forward_triton_impl
    from polarquant_amd.quantize import quantize_and_pack_nbit
    k = torch.zeros(1, 1, 128, 128, dtype=torch.float16)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        quantize_and_pack_nbit(k)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        attention_decode_forward_triton_impl(k[:, :, :1], torch.zeros(1, 1, 1, 128, 64, dtype=torch.uint8), *[k[:, :, :1, :64].unsqueeze(2)] * 4)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        polar_decode_attention(k[:, :, :1], None, None, None, None, None, k, k, 0, 1)


def test_header_compiles_as_c_and_library_links_without_python(tmp_path):
    """gcc -std=c11 against include/polarquant.h, linked with the shared library only."""
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    libdir = os.path.join(root, "polarquant_amd")
    if not os.path.exists(os.path.join(libdir, "libpolarquant_hip.so")):
        pytest.skip("library not built")
    exe = str(tmp_path / "capi_link")
    cmd = ["gcc", "-std=c11", "-Wall", "-Wextra", "-Werror", "-pedantic", "-I", os.path.join(root, "include"),
           os.path.join(root, "tests", "capi_link_main.c"), "-o", exe, "-L", libdir, "-lpolarquant_hip",
           "-Wl,-rpath," + libdir, "-Wl,-rpath,/opt/rocm/lib", "-Wl,--allow-shlib-undefined"]
    build = subprocess.run(cmd, capture_output=True, text=True)
    assert build.returncode == 0, build.stderr[-3000:]
    run = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert run.returncode == 0, (run.returncode, run.stdout, run.stderr[-2000:])
    assert run.stdout.startswith("capi ok")
