// Host-side launcher prototypes shared between the C-ABI translation unit and
// the kernel translation units.  Each returns a hipError_t cast to int (0 = ok).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace pq {

int launch_scores(const void* q, const uint8_t* codes, const void* rscale, const void* rmn, const void* tscale,
                  const void* tmn, float* out, int B, int N, int Nk, int Nb, int tbits, int dtype, bool packed6, hipStream_t st);

int launch_quantize(const void* k, const int64_t* strides, int dtype, int B, int Nk, int Nb, int rbits, int tbits,
                    unsigned flags, uint8_t* codes, void* rscale, void* rmn, void* tscale, void* tmn,
                    int cap, int off, hipStream_t st);

int launch_selftest(int dtype, unsigned long long* counters, hipStream_t st);

int launch_quantize_values(const void* v, const int64_t* strides, int dtype, int B, int Nk, int T,
                           int32_t* codes, void* scale, void* mn, int64_t cap, int64_t off, hipStream_t st);

int launch_rope_qk(const void* q_lin, int64_t q_stride, const void* k_lin, int64_t k_stride, const void* cos_t,
                   const void* sin_t, int64_t cs_batch_stride, void* q_out, void* k_out, int B, int L, int N, int Nk,
                   int dtype, hipStream_t st);
int launch_rope_append(const void* q_lin, const void* k_lin, const void* v_lin, const void* cos_tab, const void* sin_tab,
                       const int64_t* pos, void* q_out, void* k_dst, int64_t k_rows, const int64_t* k_row,
                       void* v_dst, int64_t v_rows, const int64_t* v_row, int B, int N, int Nk, int64_t max_pos, int dtype,
                       int64_t q_stride, int64_t kv_stride, hipStream_t st);
int launch_rmsnorm(const void* x, const void* res, const void* w, void* y, void* sum_out, int rows, int hidden, float eps,
                   int dtype, hipStream_t st);
int launch_silu_mul(const void* gate, const void* up, void* y, int rows, int cols, int64_t in_stride, int dtype, hipStream_t st);

int launch_convert_codes6(const uint8_t* src, uint8_t* dst, size_t n_rows, bool pack, hipStream_t st);

int launch_small_m_linear(const void* x, int64_t x_stride, const void* w, const void* w_up, const void* bias, void* y,
                          int64_t y_stride, int M, int N, int K, int dtype, hipStream_t st);

int launch_qkv_rope_append(const void* x, int64_t x_stride, const void* w, const void* bias, int M, int K, int dtype,
                           const void* cos_tab, const void* sin_tab, int64_t max_pos, const int64_t* pos, void* q_out,
                           void* k_dst, int64_t k_rows, const int64_t* k_row, void* v_dst, int64_t v_rows,
                           const int64_t* v_row, int N, int Nk, hipStream_t st);

struct AttnArgs {
    const void* q;
    const uint8_t* codes;
    const void *rscale, *rmn, *tscale, *tmn;
    int group_capacity, n_groups;
    const int32_t* n_groups_per_seq;
    const void* k_resid;
    int resid_capacity, n_resid;
    const int32_t* n_resid_per_seq;
    const void* v;
    int64_t v_capacity;
    // 4-bit values (Mixed variant): when v4_codes is set, `v` holds only the residual window's rows
    const void *v4_codes = nullptr, *v4_scale = nullptr, *v4_zero = nullptr;
    int64_t v4_capacity = 0;
    const uint8_t* mask;
    int64_t mask_stride;
    float sm_scale;
    int B, N, Nk, tbits, dtype, n_splits, min_groups_per_split;
    int rep_count = 0;           // query heads per KV head this launch works on (0: all N / Nk), see launch_attn_partials
    bool packed6 = false;        // code rows are 48 bytes of packed 6-bit codes (tbits == 3 only)
    bool balanced = false;       // slices cut on the device from the per-sequence counts (PQ_BALANCED_SLICES)
    bool single_wave = false;    // one wavefront per slice instead of a scorer / accumulator pair (PQ_SINGLE_WAVEFRONT)
    bool silent_scorer = false;  // PQ_TEST_SILENT_SCORER (honoured by the test build only)
    int32_t* status = nullptr;   // optional device word the paired kernels set when a hand-over gives up
    float* workspace;
    void* out;
};
// pq_attn_common.hip: picks the kernel family and the grid, then calls one of the four launchers below
int launch_attn_partials(const AttnArgs& a, hipStream_t st);
int launch_attn_merge(const float* ws, int B, int N, int n_splits, int dtype, void* out, hipStream_t st);
// The attention kernels are compiled once per key / value dtype (-DPQ_DTYPE=0: float16, 1: bfloat16), each into an
// object of its own, so that the two halves of the instantiations build side by side.  `total`: slices (even split:
// n_splits * B * Nk) or segments (balanced slices: what the device holds at once).
//   pq_attn_pair.hip: a scorer / accumulator pair of wavefronts per slice, the default for half-precision values
int launch_attn_pair_f16(const AttnArgs& a, int total, hipStream_t st);
int launch_attn_pair_bf16(const AttnArgs& a, int total, hipStream_t st);
//   pq_attn.hip: one wavefront per slice (PQ_SINGLE_WAVEFRONT, 4-bit values, more than 16 angle bins)
int launch_attn_one_f16(const AttnArgs& a, int total, hipStream_t st);
int launch_attn_one_bf16(const AttnArgs& a, int total, hipStream_t st);

// Device address, on the current device, of the library's own buffer for split partials
// (kStaticMaxPartials partials of 132 floats); 0 or a hipError_t.
constexpr int kStaticMaxPartials = 16384;
int attn_static_scratch(float** ptr);

// The one-wavefront kernels are instantiated for 1, 2, 4 and 8 query heads per KV head and run other ratios with the
// next of those (the heads that do not exist are zero queries whose results are dropped); the paired kernels and the
// score op are instantiated for every ratio 1..8.
inline int rep_pad(int rep) { return rep <= 1 ? 1 : rep <= 2 ? 2 : rep <= 4 ? 4 : 8; }
// More than 16 angle bins (tbits 5, 6): the table is 32-128 KiB, too large for the four tables of a paired workgroup;
// those bit widths run the one-wavefront kernels.
constexpr int kMaxPairTbits = 4;
// 128 angle bins (tbits 7): 64 pairs x 128 bins x 16 bytes = 128 KiB for up to four query heads, which is all the LDS
// a workgroup can have; KV heads with more query heads are worked through four heads at a time.
constexpr int kMaxHeadsWidestTable = 4;
// Units a plane's start-up counts for when the slices are cut on the device (query, first table, first loads, the
// partial's write).  Measured at configs[2]: one wavefront per slice, 0 / 1 / 2 / 3 units: 92.8 / 89.6 / 87.9 / 88.6 us;
// a pair per slice, whose tiles are faster and whose start-up is not, 1 / 2 / 3 / 4 / 5 units: 81.0 / 79.5 / 77.9 / 77.3 /
// 77.3 us.
constexpr int kStartUnits = 3;

// Which family a call runs: the scorer / accumulator pairs (the only kernels that can write the finished output
// themselves when a plane has a single slice) or the one-wavefront kernels.  One predicate for the launcher and for
// the entry point that decides whether a merge launch follows.
inline bool attn_runs_pairs(bool v4_codes, bool single_wave, int tbits) {
    return !v4_codes && !single_wave && tbits <= kMaxPairTbits;
}

}  // namespace pq
