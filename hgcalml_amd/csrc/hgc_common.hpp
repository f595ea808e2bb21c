// Shared host/device helpers of the gfx950 kernels (wave64 only).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "hgcalml_amd.h"

namespace hgc {

constexpr int kWave = 64;
constexpr int kNumXcd = 8;  // MI355X: 8 accelerator complex dies, one L2 each

// ---- error plumbing -------------------------------------------------------

char *last_error_buffer();  // thread local, 512 bytes

// device status word of the calling thread (hgc_set_status_word), or nullptr
int *status_word();

inline int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(last_error_buffer(), 512, fmt, ap);
    va_end(ap);
    return code;
}

#define HGC_REQUIRE(cond, ...)                                         \
    do {                                                               \
        if (!(cond)) return ::hgc::fail(HGC_ERR_INVALID_ARGUMENT, __VA_ARGS__); \
    } while (0)

#define HGC_HIP(expr)                                                              \
    do {                                                                           \
        hipError_t e_ = (expr);                                                    \
        if (e_ != hipSuccess)                                                      \
            return ::hgc::fail(HGC_ERR_LAUNCH, "%s: %s", #expr, hipGetErrorString(e_)); \
    } while (0)

inline int check_launch(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(HGC_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
    return HGC_OK;
}

inline hipStream_t as_stream(hgc_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

inline int ceil_div(long long a, long long b) { return (int)((a + b - 1) / b); }

inline size_t align_up(size_t x, size_t a = 256) { return (x + a - 1) / a * a; }

inline bool aligned256(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 255u) == 0; }

// Carves 256-byte aligned pieces out of a caller supplied workspace.
struct Carver {
    char *base;
    size_t used = 0;
    explicit Carver(void *p) : base(static_cast<char *>(p)) {}
    template <typename T>
    T *take(size_t count) {
        T *p = reinterpret_cast<T *>(base + used);
        used += align_up(count * sizeof(T));
        return p;
    }
};

// ---- internal entry points shared between translation units -----------------

// Ascending sort of n pairwise different 64-bit keys (none of them all ones;
// d_keys is overwritten, d_spare holds n more keys): the low `value_bits` bits of
// the i-th smallest key go to d_values[i]. `stage` = 0 or, for tests, the number of
// keys a workgroup sorts in LDS at once (a power of two up to 8192).
bool sample_sort_supported(long long n);
size_t sample_sort_workspace_bytes();
int sample_sort_values(uint64_t *d_keys, uint64_t *d_spare, long long n, int value_bits, int *d_values,
                       void *workspace, size_t workspace_bytes, int stage, hipStream_t s);

// Groups the points by bin for the kNN search in a handful of launches: grid from
// the bounding box, bin of every point, bin boundary table and the inputs moved
// into bin order (`d_sorting[i]` = original index of the i-th point). Unlike
// hgc_sort_by_bin the order inside a bin is not specified (it can differ from
// run to run). `n_bins_bound` bounds the number of bins of all events. The
// boundary of bin b is d_boundaries[b << shift] with shift =
// bin_grouping_sub_shift(...); the table has (n_bins_bound << shift) + 1 entries.
// spatial (granted where bin_grouping_spatial says so: 2 to 4 binned dimensions, table
// within bounds): shift = n_bin_dims, the points of a bin come grouped by the half of the
// bin they lie in per dimension (sub-cell bits: dimension i at bit n_bin_dims - 1 - i),
// every table entry is the boundary of such a sub-cell, and d_sflat holds sub-cell indices
// (bin << n_bin_dims | bits) instead of bin indices.
// d_bin_starts (may be null): n_bins_bound + 1 entries, the boundary of every bin without a stride.
bool bin_grouping_spatial(int n_bins_bound, int n_bin_dims);
int bin_grouping_sub_shift(int n_bins_bound, int n_bin_dims, bool spatial);
size_t bin_grouping_workspace_bytes(int n_vert, int n_bins_bound, int n_bin_dims, bool spatial);
int bin_grouping(const float *d_coords, const int *d_row_splits, const int *d_direction, int n_vert, int n_coords,
                 int n_bin_dims, int n_rs, int n_bins_scalar, int n_bins_bound, float *d_shift, float *d_bin_width,
                 int *d_n_bins, int *d_boundaries, int *d_sorting, float *d_scoords, int *d_sflat, int *d_sbinass,
                 int *d_sdir, bool spatial, int *d_bin_starts, void *workspace, size_t workspace_bytes,
                 hipStream_t s);

int launch_fill_i32(int *p, int value, long long n, hipStream_t s);

// The front end of the condensate wrapper (modules/assign_condensate_op.py:269-274) in one pass:
// d_shifted = d_coords minus the column minima (all n_coords columns), the grid of n_bins_scalar
// bins over the first n_bin_dims shifted columns (what BinByCoordinates derives with
// pre_normalized=True), and the bin of every hit. d_min_bits / d_max_bits_inverted [n_coords]:
// column minima as order-preserving bit patterns, maxima as the complement of theirs.
int shift_and_bin(const float *d_coords, const uint32_t *d_min_bits, const uint32_t *d_max_bits_inverted,
                  const int *d_row_splits, int n_vert, int n_coords, int n_bin_dims, int n_rs, int n_bins_scalar,
                  int n_total_bins, float *d_shifted, float *d_bin_width, int *d_n_bins, int *d_assigned_bin,
                  int *d_flat_bin, hipStream_t s);

// Stable sort of `total` items by integer key (split_sort.hip). Item i has the key
// d_keys[d_values ? d_values[i] : i] and the value d_values ? d_values[i] : i; keys outside
// [0, n_keys) count as n_keys and sort last. d_order [total] receives the values in key order,
// d_offsets (may be null) [n_keys + 1] the first position of every key. `per_key_hint`: items
// expected per key (sizes the tiles). Not every shape is supported (key ranges of 2^22 and more).
bool stable_key_sort_supported(long long total, int n_keys, int per_key_hint);
size_t stable_key_sort_workspace_bytes(long long total, int n_keys, int per_key_hint);
int stable_key_sort(const int *d_keys, const int *d_values, long long total, int n_keys, int per_key_hint,
                    int *d_offsets, int *d_order, void *workspace, size_t workspace_bytes, hipStream_t s);

// hgc_binned_select_knn_fused over a boundary table with stride 2^boundary_shift.
// fine_bits > 0 (= n_bin_dim): d_bin_idx holds the half-bin cells of bin_grouping's spatial mode
// and d_cell_boundaries is that mode's table (one entry per cell); a query whose bin holds more
// than fine_min_population points then walks the nested grid of half the bin width instead of
// the bins.
int binned_select_knn_strided(const float *d_coord, const int *d_bin_idx, const int *d_direction,
                              const int *d_dim_bin_idx, const int *d_bin_boundaries, int boundary_shift,
                              const int *d_n_bins, const float *d_bin_width, const int *d_sorting,
                              const float *d_shift, float max_radius, int *d_indices, float *d_dist, int n_vert,
                              int n_neigh, int n_coords, int n_bin_dim, int n_bboundaries, int tf_compat,
                              int use_direction, const int *d_cell_boundaries, int fine_bits,
                              int fine_min_population, hipStream_t s);

// hgc_binned_assign_to_condensates with two more arguments: with d_high set, the *_h
// arrays are the arrays of all hits themselves (n_vert_h == n_vert, d_indices_to_filtered[i]
// = i or -1, d_row_splits_h = d_row_splits) and d_high [n_vert] says which hits form the
// high-beta subset; d_quirk = {index of the first of them, its no_condensation_mask, the
// second one's} then stands for the first two entries of the filtered mask.
size_t condensates_workspace_bytes(int n_vert, int n_vert_h, int num_rows, int dimensions);
int condensates_assign(int dimensions, int dimensions_binning, int *d_condensates_assigned_h,
                       const float *d_ccoords_h, const float *d_dist_h, const float *d_beta_h,
                       const int *d_no_condensation_mask_h, int *d_high_assigned_status_h,
                       const int *d_original_indices_h, const int *d_row_splits_h, const float *d_ccoords,
                       const int *d_no_condensation_mask, const int *d_indices_to_filtered,
                       float *d_assignment_min_distance, int *d_assignment, int *d_association,
                       int *d_n_condensates, int *d_alpha_indices, const int *d_bin_splits, const int *d_n_bins,
                       const float *d_bin_widths, const int *d_row_splits, int num_rows, int assign_by_max_beta,
                       int n_vert, int n_vert_h, int *d_error, const int *d_high, const int *d_quirk,
                       void *workspace, size_t workspace_bytes, hipStream_t s);

// ---- device helpers -------------------------------------------------------

#ifdef __HIPCC__

__device__ __forceinline__ int lane_id() { return threadIdx.x & (kWave - 1); }

// Consecutive workgroups are dealt round-robin to the 8 XCDs. This maps the
// hardware block index to a logical tile index such that each XCD works on one
// contiguous range of tiles (neighbouring tiles then share that XCD's L2).
__device__ __forceinline__ int xcd_contiguous_block(int bid, int nblocks) {
    const int per = nblocks / kNumXcd;
    const int body = per * kNumXcd;
    if (bid >= body) return bid;  // ragged tail keeps its index
    return (bid % kNumXcd) * per + bid / kNumXcd;
}

// Same idea in chunks: tiles [c*CHUNK, (c+1)*CHUNK) go to XCD c % 8, so that an
// XCD's concurrent workgroups still work on neighbouring tiles while every XCD
// gets its share of every part of the tile range. For work whose cost varies
// along the range (one XCD-sized contiguous piece would finish long after
// another).
template <int CHUNK>
__device__ __forceinline__ int xcd_chunked_block(int bid, int nblocks) {
    const int body = nblocks / (kNumXcd * CHUNK) * (kNumXcd * CHUNK);
    if (bid >= body) return bid;  // ragged tail keeps its index
    const int xcd = bid % kNumXcd, k = bid / kNumXcd;  // the k-th block this XCD receives
    return ((k / CHUNK) * kNumXcd + xcd) * CHUNK + k % CHUNK;
}

__device__ __forceinline__ int readlane_i32(int v, int lane) {
    return __builtin_amdgcn_readlane(v, lane);
}

__device__ __forceinline__ uint64_t readlane_u64(uint64_t v, int lane) {
    uint32_t lo = __builtin_amdgcn_readlane((int)(uint32_t)v, lane);
    uint32_t hi = __builtin_amdgcn_readlane((int)(uint32_t)(v >> 32), lane);
    return ((uint64_t)hi << 32) | lo;
}

// lane i receives v from lane i-1; lane 0 receives `into_lane0`
__device__ __forceinline__ uint32_t wave_shift_up1(uint32_t v, uint32_t into_lane0) {
    // DPP wave_shr:1 (0x138): whole-wave shift right by one lane; lanes without
    // a source keep the first operand.
    return (uint32_t)__builtin_amdgcn_update_dpp((int)into_lane0, (int)v, 0x138, 0xf, 0xf, false);
}

__device__ __forceinline__ uint64_t wave_shift_up1_u64(uint64_t v, uint64_t into_lane0) {
    uint32_t lo = wave_shift_up1((uint32_t)v, (uint32_t)into_lane0);
    uint32_t hi = wave_shift_up1((uint32_t)(v >> 32), (uint32_t)(into_lane0 >> 32));
    return ((uint64_t)hi << 32) | lo;
}

// DPP controls (gfx9 encoding): shift right by n lanes inside each row of 16,
// broadcast of lane 15 of each row to the next row, of lane 31 to the upper half.
constexpr int kDppRowShr = 0x110;
constexpr int kDppRowBcast15 = 0x142;
constexpr int kDppRowBcast31 = 0x143;

// v of the lane `CTRL` names, 0 where that lane does not exist or the row is masked off
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint32_t dpp_or_zero(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, ROW_MASK, 0xf, false);
}

// inclusive prefix sum over the 64 lanes (wrapping arithmetic)
__device__ __forceinline__ int wave_inclusive_sum(int x) {
    uint32_t v = (uint32_t)x;
    v += dpp_or_zero<kDppRowShr + 1, 0xf>(v);
    v += dpp_or_zero<kDppRowShr + 2, 0xf>(v);
    v += dpp_or_zero<kDppRowShr + 4, 0xf>(v);
    v += dpp_or_zero<kDppRowShr + 8, 0xf>(v);
    v += dpp_or_zero<kDppRowBcast15, 0xa>(v);
    v += dpp_or_zero<kDppRowBcast31, 0xc>(v);
    return (int)v;
}

// inclusive prefix maximum over the 64 lanes
__device__ __forceinline__ uint32_t wave_inclusive_max(uint32_t v) {
    v = max(v, dpp_or_zero<kDppRowShr + 1, 0xf>(v));
    v = max(v, dpp_or_zero<kDppRowShr + 2, 0xf>(v));
    v = max(v, dpp_or_zero<kDppRowShr + 4, 0xf>(v));
    v = max(v, dpp_or_zero<kDppRowShr + 8, 0xf>(v));
    v = max(v, dpp_or_zero<kDppRowBcast15, 0xa>(v));
    v = max(v, dpp_or_zero<kDppRowBcast31, 0xc>(v));
    return v;
}

// LDS traffic of one wave stays in program order; this keeps the compiler from
// moving the wave's own accesses across the point where lanes exchange data.
__device__ __forceinline__ void wave_lds_fence() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

#endif  // __HIPCC__

}  // namespace hgc
