// Instrumentation of the MEASURING build of the decode-attention kernels (-DPQ_ATTN_PHASE_TIMERS,
// `python -m polarquant_amd.build --phase-timers` -> libpolarquant_hip_timers.so, read by
// polarquant_amd/benchmarks/phase_timing.py).  In the shipping build every macro below expands to nothing.
#pragma once

// ---- probe builds (timing only: their results are wrong on purpose) ----
// -DPQ_PROBE_NO_VALUES (`python -m polarquant_amd.build --probe no_values` -> libpolarquant_hip_probe.so, timed by
// polarquant_amd/benchmarks/probe_bench.py): the 4-bit-value kernels without their value path -- no value loads, no
// nibble unpacking, no matrix products, no zero-point term; codes, tables, scores, mask and the softmax sums remain.
// What is left is the floor the score side alone sets for that kernel.
#ifdef PQ_PROBE_NO_VALUES
constexpr bool kProbeNoValues = true;
#else
constexpr bool kProbeNoValues = false;
#endif

// ---- one wavefront per slice (pq_attn.hip) ----
// Measuring build only (-DPQ_ATTN_PHASE_TIMERS, `python -m polarquant_amd.build --phase-timers`): wall-clock
// (100 MHz) time of each phase of the group loop, summed per wavefront and printed by a few of them.
#ifdef PQ_ATTN_PHASE_TIMERS
#define PQ_T_ENTRY const long long pt_entry_ = wall_clock64(); long long pt_loop0_ = pt_entry_, pt_first_ = 0, pt_loop1_ = pt_entry_, pt_sum_[6] = {0, 0, 0, 0, 0, 0}; int pt_groups_ = 0
#define PQ_T_DECL long long pt_[6] = {0, 0, 0, 0, 0, 0}, pt_mark_ = 0; pt_loop0_ = wall_clock64()
#define PQ_T_MARK() pt_mark_ = wall_clock64()
#define PQ_T_ADD(i) do { const long long pt_now_ = wall_clock64(); pt_[i] += pt_now_ - pt_mark_; pt_mark_ = pt_now_; } while (0)
#define PQ_T_KEEP(x) asm volatile("" ::"v"(x))
#define PQ_T_FIRST_GROUP_DONE() do { if (pt_first_ == 0) pt_first_ = wall_clock64() - pt_loop0_; } while (0)
#define PQ_T_REPORT(n_groups)                                                                                        \
    do {                                                                                                             \
        pt_loop1_ = wall_clock64();                                                                                  \
        pt_groups_ = n_groups;                                                                                       \
        for (int i_ = 0; i_ < 6; i_++) pt_sum_[i_] = pt_[i_];                                                        \
    } while (0)
// Printed once per piece, after its partial has been handed to the memory system (a device printf takes
// milliseconds, so none may sit inside what is timed): the phase sums of the group loop, then the absolute entry
// and exit clocks (the 100 MHz counter is common to the chip, so the spread of entries and exits over the
// wavefronts can be read off), entry -> loop, the first group, the loop, loop -> exit.
#define PQ_T_EXIT()                                                                                                  \
    do {                                                                                                             \
        const long long pt_exit_ = wall_clock64();                                                                   \
        const int pt_block_ = static_cast<int>((blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x);      \
        if (threadIdx.x == 0 && pt_block_ % 97 == 0) {                                                               \
            printf("pq_phase block %d groups %d total %lld table %lld value_issue %lld code_wait %lld code_issue %lld score %lld softmax_pv %lld\n", \
                   pt_block_, pt_groups_, pt_loop1_ - pt_loop0_, pt_sum_[0], pt_sum_[1], pt_sum_[2], \
                   pt_sum_[3], pt_sum_[4], pt_sum_[5]);                                                              \
            printf("pq_piece block %d groups %d entry %lld exit %lld before_loop %lld first_group %lld loop %lld after_loop %lld\n", \
                   pt_block_, pt_groups_, pt_entry_, pt_exit_, pt_loop0_ - pt_entry_, pt_first_,   \
                   pt_loop1_ - pt_loop0_, pt_exit_ - pt_loop1_);                                                     \
        }                                                                                                            \
    } while (0)
#else
#define PQ_T_ENTRY
#define PQ_T_DECL
#define PQ_T_MARK()
#define PQ_T_ADD(i)
#define PQ_T_KEEP(x)
#define PQ_T_FIRST_GROUP_DONE()
#define PQ_T_REPORT(n_groups)
#define PQ_T_EXIT()
#endif

// ---- scorer / accumulator pairs (pq_attn_pair.hip) ----
// Measuring build only (-DPQ_ATTN_PHASE_TIMERS): every wavefront adds up the wall-clock time (100 MHz) it spends in
// pair_wait and notes the clock at its entry, at its first and last hand-over and at its exit; the wavefronts of every
// 97th workgroup print them with their role when their kernel ends.  From these the reader takes a pair's start-up
// (entry -> first tile handed over), its pace in the steady state and its tail (last hand-over -> exit).
struct PairTimes { long long waited = 0, first = 0, last = 0, mark[3] = {0, 0, 0}; };
#ifdef PQ_ATTN_PHASE_TIMERS
#define PQ_PAIR_T_DECL const long long pw_entry_ = wall_clock64()
#define PQ_PAIR_T_WAIT(call) [&]() { const long long t0_ = wall_clock64(); const bool r_ = (call); pw_times_.waited += wall_clock64() - t0_; return r_; }()
#define PQ_PAIR_T_TILE() do { pw_times_.last = wall_clock64(); if (pw_times_.first == 0) pw_times_.first = pw_times_.last; } while (0)
// the clock the first time a wavefront passes a point of its start-up (scorer: 0 = role known, 1 = first loads have
// arrived, which the measuring build waits for at this point, 2 = first table built; accumulator: 0 = role known)
#define PQ_PAIR_T_MARK(i, drain)                                                                                     \
    do {                                                                                                             \
        if (pw_times_.mark[i] == 0) {                                                                                \
            if (drain) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");                                              \
            pw_times_.mark[i] = wall_clock64();                                                                      \
        }                                                                                                            \
    } while (0)
#define PQ_PAIR_T_REPORT(role, tiles, times)                                                                         \
    do {                                                                                                             \
        const long long pw_exit_ = wall_clock64();                                                                   \
        if ((threadIdx.x & 63) == 0 && blockIdx.x % 97 == 0)                                                         \
            printf("pq_pair block %d wave %d role %d tiles %d entry %lld first %lld last %lld exit %lld waited %lld " \
                   "marks %lld %lld %lld\n",                                                                         \
                   static_cast<int>(blockIdx.x), static_cast<int>(threadIdx.x >> 6), role, tiles, pw_entry_,         \
                   (times).first, (times).last, pw_exit_, (times).waited, (times).mark[0], (times).mark[1],          \
                   (times).mark[2]);                                                                                 \
    } while (0)
#else
#define PQ_PAIR_T_DECL
#define PQ_PAIR_T_WAIT(call) (call)
#define PQ_PAIR_T_TILE()
#define PQ_PAIR_T_MARK(i, drain)
#define PQ_PAIR_T_REPORT(role, tiles, times)
#endif
