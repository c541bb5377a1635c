"""ctypes binding of libpolarquant_hip.so (the C ABI declared in include/polarquant.h).

The library is loaded from the package directory; it is never built implicitly
on import of this module when a built library exists.  If it is missing the
loader raises: there is no CPU fallback for any op of this package.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_uint, c_void_p

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libpolarquant_hip.so")

PQ_F16, PQ_BF16 = 0, 1
PQ_WRAP_FP32 = 1
PQ_ANGLE_UNIFORM = 2
PQ_CODES_PACKED6 = 4
PQ_DEVICE_ATAN2 = 8
PQ_BALANCED_SLICES = 16
PQ_SINGLE_WAVEFRONT = 32
PQ_TEST_SILENT_SCORER = 0x40000000      # honoured by the test build of the library only; the one loaded here refuses it
PQ_STATUS_HANDOVER_TIMEOUT = 1
PQ_EAGER_GPU = PQ_WRAP_FP32 | PQ_DEVICE_ATAN2

STATUS_NAMES = {
    0: "PQ_OK", -1: "PQ_ERR_NULL_POINTER", -2: "PQ_ERR_BAD_SHAPE", -3: "PQ_ERR_BAD_BITS", -4: "PQ_ERR_BAD_DTYPE",
    -5: "PQ_ERR_MISALIGNED", -6: "PQ_ERR_BAD_STRIDE", -7: "PQ_ERR_WORKSPACE", -8: "PQ_ERR_LAUNCH",
    -9: "PQ_ERR_NO_DEVICE",
}

# name -> (restype, argtypes); every symbol of include/polarquant.h
SIGNATURES = {
    "pq_version": (c_int, []),
    "pq_status_string": (c_char_p, [c_int]),
    "pq_decode_scores": (c_int, [c_void_p] * 7 + [c_int] * 7 + [c_uint, c_void_p]),
    "pq_validate_decode_scores": (c_int, [c_void_p] * 7 + [c_int] * 7 + [c_uint]),
    "pq_quantize_groups": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_uint]
                           + [c_void_p] * 5 + [c_int, c_int, c_void_p]),
    "pq_validate_quantize_groups": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_uint]
                                    + [c_void_p] * 5 + [c_int, c_int]),
    "pq_selftest_quantizer_math": (c_int, [c_int, c_void_p, c_void_p]),
    "pq_decode_attn": (c_int, [c_void_p] * 6 + [c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p,
                                                c_void_p, c_int64, c_void_p, c_int64, c_float]
                       + [c_int] * 8 + [c_void_p, c_size_t, c_void_p, c_uint, c_void_p, c_void_p]),
    "pq_decode_attn_static": (c_int, [c_void_p] * 6 + [c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p,
                                                       c_void_p, c_int64, c_void_p, c_int64, c_float]
                              + [c_int] * 8 + [c_void_p, c_uint, c_void_p, c_void_p]),
    "pq_validate_decode_attn": (c_int, [c_void_p] * 6 + [c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p,
                                                         c_void_p, c_int64, c_void_p, c_int64, c_float]
                                + [c_int] * 8 + [c_void_p, c_size_t, c_void_p, c_uint]),
    "pq_decode_attn_partials": (c_int, [c_void_p] * 6 + [c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p,
                                                         c_void_p, c_int64, c_void_p, c_int64, c_float]
                                + [c_int] * 8 + [c_void_p, c_size_t, c_uint, c_void_p, c_void_p]),
    "pq_decode_attn_merge": (c_int, [c_void_p, c_size_t, c_int, c_int, c_int, c_int, c_void_p, c_void_p]),
    "pq_quantize_values": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p,
                                   c_int64, c_int64, c_void_p]),
    "pq_validate_quantize_values": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p,
                                            c_int64, c_int64]),
    "pq_decode_attn_v4": (c_int, [c_void_p] * 6 + [c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p,
                                                   c_void_p, c_void_p, c_void_p, c_void_p, c_int64,
                                                   c_void_p, c_int64, c_float]
                          + [c_int] * 8 + [c_void_p, c_size_t, c_void_p, c_uint, c_void_p, c_void_p]),
    "pq_validate_decode_attn_v4": (c_int, [c_void_p] * 6 + [c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p,
                                                            c_void_p, c_void_p, c_void_p, c_void_p, c_int64,
                                                            c_void_p, c_int64, c_float]
                                   + [c_int] * 8 + [c_void_p, c_size_t, c_void_p, c_uint]),
    "pq_rope_append": (c_int, [c_void_p] * 5 + [c_int64, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_int64,
                                               c_void_p, c_int, c_int, c_int, c_int, c_int64, c_int64, c_void_p]),
    "pq_rmsnorm": (c_int, [c_void_p] * 5 + [c_int, c_int, c_float, c_int, c_void_p]),
    "pq_silu_mul": (c_int, [c_void_p] * 3 + [c_int, c_int, c_int64, c_int, c_void_p]),
    "pq_linear_small_m": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int, c_int, c_int, c_void_p]),
    "pq_validate_linear_small_m": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int, c_int, c_int]),
    "pq_rope_qk": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_void_p, c_void_p,
                           c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "pq_qkv_rope_append": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_int64,
                                   c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_void_p, c_int, c_int, c_void_p]),
    "pq_validate_qkv_rope_append": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_int64,
                                            c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_void_p, c_int, c_int]),
    "pq_convert_codes6": (c_int, [c_void_p, c_void_p, c_size_t, c_int, c_void_p]),
    "pq_decode_attn_plan": (c_int, [c_int] * 4),
    "pq_decode_attn_v4_plan": (c_int, [c_int] * 5),
    "pq_decode_attn_workspace_bytes": (c_size_t, [c_int] * 3),
}


# the bench-only library (include/polarquant_bench.h): measurement aids, loaded by bench.py and its tests
BENCH_LIB_PATH = os.path.join(HERE, "libpolarquant_bench.so")
BENCH_SIGNATURES = {
    "pq_stream_read": (c_size_t, [c_void_p, c_size_t, c_int, c_void_p, c_void_p]),
    "pq_attn_load_replica": (c_size_t, [c_void_p, c_void_p, c_int, c_int64, c_int64, c_int64, c_int, c_void_p, c_void_p]),
}


class PolarQuantError(RuntimeError):
    def __init__(self, status: int, where: str):
        self.status = status
        msg = STATUS_NAMES.get(status, str(status))
        try:
            msg += ": " + lib().pq_status_string(status).decode()
        except Exception:
            pass
        super().__init__("%s failed with %s" % (where, msg))


_LIB = None


def lib() -> ctypes.CDLL:
    """The loaded HIP library.  Raises if it has not been built."""
    global _LIB
    if _LIB is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "polarquant_amd: %s is missing; build it with `python -m polarquant_amd.build` "
                "(there is no CPU fallback)" % LIB_PATH)
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _LIB = handle
    return _LIB


_BENCH_LIB = None


def bench_lib() -> ctypes.CDLL:
    """The measurement-aid library.  Raises if it has not been built."""
    global _BENCH_LIB
    if _BENCH_LIB is None:
        if not os.path.exists(BENCH_LIB_PATH):
            raise RuntimeError("polarquant_amd: %s is missing; build it with `python -m polarquant_amd.build`" % BENCH_LIB_PATH)
        handle = ctypes.CDLL(BENCH_LIB_PATH)
        for name, (res, args) in BENCH_SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _BENCH_LIB = handle
    return _BENCH_LIB


def check(status: int, where: str) -> None:
    if status != 0:
        raise PolarQuantError(status, where)
