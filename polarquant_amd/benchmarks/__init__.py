"""Measurement modules (timing harnesses, sweeps, the measuring build's reader): what bench.py and the
profiles' commands run.  Nothing in the importable product (the drop-in classes, the ops, the C-ABI binding)
imports from here.

    python -m polarquant_amd.benchmarks.config_bench      configs[0], [2], [3]
    python -m polarquant_amd.benchmarks.e2e_bench         configs[4], the end-to-end greedy decode
    python -m polarquant_amd.benchmarks.memory_bench      the reference's peak-memory protocol
    python -m polarquant_amd.benchmarks.microbench        the reference's score-op micro-benchmark shapes
    python -m polarquant_amd.benchmarks.shape_bench       decode attention at other head layouts and batch shapes
    python -m polarquant_amd.benchmarks.linear_bench      the decode step's linear layers
    python -m polarquant_amd.benchmarks.phase_timing      per-phase wall-clock times of the attention kernels (measuring build)
"""
