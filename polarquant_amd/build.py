"""Build recipe of the HIP library: hipcc for gfx950, in-tree.

    python -m polarquant_amd.build                    # (re)build polarquant_amd/libpolarquant_hip.so, its test build and libpolarquant_bench.so
    python -m polarquant_amd.build --phase-timers     # the measuring build (benchmarks/phase_timing.py)
    python -m polarquant_amd.build --probe no_values  # a probe build (benchmarks/probe_bench.py)

hipcc cross-compiles without a GPU.  Flags that matter:
  -ffp-contract=off            the quantizer reproduces eager half-precision torch
                               arithmetic op by op; FMAs are written explicitly
  -packed-fp32-ops disabled    no v_pk_*_f32 instructions
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "build")
LIB = os.path.join(HERE, "libpolarquant_hip.so")
# (source, defines, object tag): the two attention sources are compiled once per dtype, so that the halves of their
# many template instantiations build side by side
UNITS = [("pq_attn.hip", ("PQ_DTYPE=0",), ".f16"), ("pq_attn.hip", ("PQ_DTYPE=1",), ".bf16"),
         ("pq_attn_pair.hip", ("PQ_DTYPE=0",), ".f16"), ("pq_attn_pair.hip", ("PQ_DTYPE=1",), ".bf16"),
         ("pq_scores.hip", (), ""), ("pq_quantize.hip", (), ""), ("pq_linear.hip", (), ""), ("pq_attn_common.hip", (), ""),
         ("pq_capi.hip", (), ""), ("pq_values.hip", (), ""), ("pq_decode_ops.hip", (), "")]
SOURCES = sorted({u[0] for u in UNITS})
# measurement aids (a plain streaming read, the attention kernel's loads without its arithmetic): a library of
# their own, loaded by bench.py and its tests only
BENCH_LIB = os.path.join(HERE, "libpolarquant_bench.so")
BENCH_SOURCES = ["pq_stream.hip"]
ARCH = "gfx950"
FLAGS = ["--offload-arch=" + ARCH, "-O3", "-fPIC", "-std=c++17", "-ffp-contract=off",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall", "-Wno-unused-function"]


def _hipcc() -> str:
    for c in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if c and (os.path.isabs(c) and os.path.exists(c) or not os.path.isabs(c)):
            return c
    raise RuntimeError("hipcc not found")


TIMERS_LIB = os.path.join(HERE, "libpolarquant_hip_timers.so")
# the test build: the same library with -DPQ_TEST_HOOKS, which alone honours PQ_TEST_SILENT_SCORER (a hook that turns
# the output into NaN on purpose).  Loaded by tests/test_pair_handover_gpu.py only, never by the package.
HOOKS_LIB = os.path.join(HERE, "libpolarquant_hip_testhooks.so")
# the units that read the define: the C ABI's flag check and the paired kernels (float16 only: the hook is honoured for
# that dtype, which is what its test uses; the bfloat16 kernels of the test build are the shipping ones)
HOOKS_UNITS = {("pq_capi.hip", ""): ("pq_capi.hip", ("PQ_TEST_HOOKS",), ".hooks"),
               ("pq_attn_pair.hip", ".f16"): ("pq_attn_pair.hip", ("PQ_DTYPE=0", "PQ_TEST_HOOKS"), ".f16.hooks")}


def _compile(src: str, defines=(), tag: str = "") -> str:
    obj = os.path.join(OBJ, os.path.splitext(src)[0] + tag + ".o")
    cmd = [_hipcc()] + FLAGS + ["-D" + d for d in defines] + ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def _link(objs, lib: str) -> None:
    tmp = lib + ".tmp"
    r = subprocess.run([_hipcc(), "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", tmp] + list(objs),
                       capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    os.replace(tmp, lib)


# probe builds: the library with one unit compiled for a timing-only experiment (results wrong on purpose); loaded by
# polarquant_amd/benchmarks/probe_bench.py only
PROBE_LIB = os.path.join(HERE, "libpolarquant_hip_probe.so")
PROBES = {"no_values": {("pq_attn.hip", ".f16"): ("pq_attn.hip", ("PQ_DTYPE=0", "PQ_PROBE_NO_VALUES"), ".f16.no_values")},
          "direct_bins": {("pq_quantize.hip", ""): ("pq_quantize.hip", ("PQ_PROBE_DIRECT_BINS",), ".direct_bins")}}


def build_probe(name: str, verbose: bool = True) -> str:
    """libpolarquant_hip_probe.so for probe `name`: the shipping objects (built if missing) with the probe's units
    recompiled."""
    os.makedirs(OBJ, exist_ok=True)
    swap = PROBES[name]
    units = [swap.get((src, tag), (src, defs, tag)) for src, defs, tag in UNITS]
    todo = [u for u in units if u in swap.values() or not os.path.exists(os.path.join(OBJ, os.path.splitext(u[0])[0] + u[2] + ".o"))]
    with ThreadPoolExecutor(max_workers=min(8, max(len(todo), 1))) as ex:
        list(ex.map(lambda j: _compile(*j), todo))
    _link([os.path.join(OBJ, os.path.splitext(u[0])[0] + u[2] + ".o") for u in units], PROBE_LIB)
    if verbose:
        print("built", PROBE_LIB, "(probe %s)" % name)
    return PROBE_LIB


def build(verbose: bool = True, phase_timers: bool = False) -> str:
    """The library the package loads; or, with phase_timers, a second library (same ABI, not loaded by default)
    whose attention kernel times its phases with the wall clock and prints them: a measuring build for
    `python -m polarquant_amd.benchmarks.phase_timing`, a few percent slower than the real one."""
    os.makedirs(OBJ, exist_ok=True)
    if phase_timers:
        main = [(src, defs + ("PQ_ATTN_PHASE_TIMERS",), tag + ".timers") for src, defs, tag in UNITS]
        jobs = list(main)
    else:
        main = list(UNITS)
        hooks = [HOOKS_UNITS.get((src, tag), (src, defs, tag)) for src, defs, tag in UNITS]
        bench = [(s_, (), "") for s_ in BENCH_SOURCES]
        jobs = main + [u for u in hooks if u not in main] + bench
    # the units are listed longest compilation first
    with ThreadPoolExecutor(max_workers=min(8, len(jobs))) as ex:
        built = dict(zip(jobs, ex.map(lambda j: _compile(*j), jobs)))
    lib = TIMERS_LIB if phase_timers else LIB
    _link([built[u] for u in main], lib)
    if not phase_timers:
        _link([built[u] for u in hooks], HOOKS_LIB)
        _link([built[u] for u in bench], BENCH_LIB)
        if verbose:
            print("built", HOOKS_LIB)
            print("built", BENCH_LIB)
    if verbose:
        print("built", lib)
    return lib


if __name__ == "__main__":
    if "--probe" in sys.argv[1:]:
        build_probe(sys.argv[sys.argv.index("--probe") + 1])
    else:
        build(phase_timers="--phase-timers" in sys.argv[1:])
