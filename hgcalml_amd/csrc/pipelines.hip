// Whole-wrapper entry points: the complete device-side sequence of a reference
// Python wrapper behind one C call, so that a caller pays one launch sequence
// and one workspace instead of a dozen framework ops.
//
//   hgc_binned_select_knn_pipeline  modules/binned_select_knn_op.py:33-104
//     (bounding box and grid, bin assignment, grouping by bin with the inputs
//      moved along, search, un-sort)
//   hgc_build_and_assign_condensates  modules/assign_condensate_op.py:210-373
//     (coordinates shifted to their minimum, grid, bin assignment, stable sort
//      into bin order, high-beta subset, assignment, back to the caller's order)
#include "hgc_common.hpp"

#include <algorithm>
#include <cmath>
#include <mutex>

namespace hgc {
int launch_fill_i32(int *p, int value, long long n, hipStream_t s);
}

using namespace hgc;

// Scratch memory of hgc_binned_select_knn_pipeline_static, part of the library's
// device image: every GPU the library runs on holds its own copy at its own
// address from the first use to the end of the process. In host code this name
// is only a handle for hipGetSymbolAddress, never a device address.
static __device__ __align__(256) unsigned char scratch[HGC_STATIC_SCRATCH_BYTES];

namespace {

// The grid the kNN pipeline searches on. The neighbour sets do not depend on it (the search is
// exact), only the run time does, so by default the pipeline does not take the caller's grid
// (the reference wrapper's n_bins over min(3, C) dimensions) but its own.
//   * Up to four binned dimensions: binning the fourth coordinate of 4-D points too removes the
//     candidates that are close in three coordinates and far in the fourth.
//   * n_bins = 0.9 (points per event * 64 / K)^(1/dimensions) with K taken inside 32 .. 64 (0.85
//     under a nested grid, below): a bit
//     more than one point per bin at K = 64, and finer for fewer neighbours (16 events of 20,000 to
//     120,000 3-D points, K = 32, radius 0.1: 1.72 ms -> 1.59 ms). For more than 64 neighbours a
//     coarser grid did not pay (150,000 clustered 4-D points, K = 129 / 257: 0.96 / 2.23 ms on the
//     grid for 64, 1.02 / 2.49 ms on one scaled further).
//   * Where every coordinate is binned (2 to 4 of them) and the table stays small, a nested grid of
//     half the bin width for the queries of crowded bins (bin_grouping's spatial mode,
//     KnnParams::fine_bits): with it the bins themselves can be wider than a single grid would
//     want them, which is what sparse regions like (their shells are mostly empty bins). Measured
//     kernel times, 150,000 points in 4-D, K = 64, single grid of 20 bins -> nested grid on 18 bins:
//     clusters + noise 450 -> 425 us, Gaussian blob 825 -> 515 us, uniform 418 -> 351 us. The whole
//     call with and without it on the same bins, in ms (150,000 points; the nested grid's table is
//     2^dimensions times larger, and few neighbours come from few candidates either way):
//                               K = 8          16            32            64            129
//       4-D clusters + noise  0.43 / 0.28   0.38 / 0.31   0.40 / 0.37   0.47 / 0.47   0.86 / 0.86
//       4-D Gaussian blob     0.35 / 0.32   0.38 / 0.38   0.44 / 0.52   0.56 / 0.82   1.04 / 1.86
//       3-D clusters + noise  0.31 / 0.23   0.30 / 0.25   0.32 / 0.30   0.36 / 0.36   0.61 / 0.64
//       3-D uniform           0.33 / 0.21   0.29 / 0.24   0.33 / 0.29   0.35 / 0.32   0.55 / 0.53
//       3-D Gaussian blob     0.26 / 0.25   0.29 / 0.29   0.33 / 0.36   0.37 / 0.52   0.70 / 0.96
//       2-D clusters + noise  0.28 / 0.22   0.30 / 0.27   0.36 / 0.33   0.36 / 0.35   0.60 / 0.59
//     so it is taken from 48 neighbours on and three binned dimensions on.
//   * Points with more than four coordinates bin the first four, on the same rule (their bins hold
//     every point along the other coordinates, so the neighbourhood is wide in bin widths however
//     fine the grid; a nested grid does not pay there). 150,000 points, K = 64, three binned
//     dimensions at 32 bins -> four at 18: 5-D Gaussian 2.07 -> 1.45 ms, 6-D Gaussian 2.91 -> 2.20 ms,
//     6-D uniform 2.24 -> 1.62 ms, 8-D Gaussian 7.40 -> 5.85 ms. (Gaussians like more bins still,
//     uniform boxes fewer: 24 / 11 bins give 1.17 / 2.32, 2.08 / 3.71, 2.71 / 1.23, 5.95 / 7.70 ms.)
//   * Small events want fewer bins than that (most of a small grid is boundary): 200,000 uniform
//     4-D points in 1000 events, K = 64: 0.80 ms at 4 bins, 0.52 at 3; in 4000 events 1.07 ms at
//     4 bins, 0.31 at 2.
thread_local int g_callers_knn_grid = 0;

struct SearchGrid {
    int n_bin_dims, n_bins;
    bool nested;  // ask for the nested grid of half the bin width (granted where the boundary table stays small)
};

SearchGrid callers_grid(int n_coords, int n_bins_scalar, int max_bin_dims) {
    return {std::min(max_bin_dims, n_coords), n_bins_scalar, false};
}

// kSmallestGridK: the grid for this many neighbours or fewer is the finest one (it sizes the workspace)
constexpr int kSmallestGridK = 32, kLargestGridK = 64;
// a bin with more than (K - 1) / kCrowdedBinFraction points sends its queries to the nested grid
constexpr int kCrowdedBinFraction = 3;  // 2 .. 6 measured: 3 is best by 1 to 3 % on clustered, Gaussian and uniform points
// fewer neighbours than this search on the single grid (see the table above own_grid)
constexpr int kSmallestNestedK = 48;

SearchGrid own_grid(int n_vert, int n_coords, int n_rs, int n_neigh) {
    const int dims = std::min(n_coords, 4);
    const double per_event = std::max(1.0, (double)n_vert / std::max(1, n_rs - 1));
    // small events: 0.75 of the rule up to 5,000 points per event, rising to 1 at 50,000
    const double small = std::min(1.0, std::max(0.75, 0.75 + 0.25 * (std::log10(per_event) - 3.7)));
    const double k = std::min(std::max(n_neigh, kSmallestGridK), kLargestGridK);
    const bool nested = dims == n_coords && dims >= 3 && n_neigh >= kSmallestNestedK;
    // under a nested grid the bins can be a little wider still (150,000 points, K = 64, factor 0.9 -> 0.85:
    // clusters + noise and Gaussian blob unchanged, 4-D uniform 0.40 -> 0.385 ms, 3-D clusters 0.354 -> 0.346 ms;
    // at 0.8 and below the blob loses 2 to 4 %)
    const double n_bins = (nested ? 0.85 : 0.9) * small * std::pow(per_event * 64.0 / k, 1.0 / dims);
    return {dims, std::max(2, std::min((int)std::lround(n_bins), dims >= 4 ? 40 : dims == 3 ? 128 : 1024)), nested};
}

SearchGrid search_grid(int n_vert, int n_coords, int n_rs, int n_neigh, int n_bins_scalar, int max_bin_dims) {
    const SearchGrid asked = callers_grid(n_coords, n_bins_scalar, max_bin_dims);
    // a request the reference op refuses stays refused
    if (g_callers_knn_grid || asked.n_bin_dims < 2 || asked.n_bin_dims > 5 || n_bins_scalar < 1) return asked;
    return own_grid(n_vert, n_coords, n_rs, n_neigh);
}

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices] = {};  // device address of `scratch` per device, looked up once

// the current device's copy of `scratch` (nullptr + error text on failure)
int static_scratch(void **out) {
    int dev = -1;
    HGC_HIP(hipGetDevice(&dev));
    HGC_REQUIRE(dev >= 0 && dev < kMaxDevices, "device ordinal %d beyond the %d this library keeps scratch for", dev,
                kMaxDevices);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *ptr = nullptr;
        HGC_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        if (!ptr || !aligned256(ptr)) return fail(HGC_ERR_LAUNCH, "static scratch array has no usable device address");
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return HGC_OK;
}

struct KnnPipelineLayout {
    size_t shift, bin_width, n_bins, sorting, bounds, bin_starts, scoords, sflat, sbinass, sdir, grouping_ws, total;
    int total_bins_bound;
    bool nested;
    int boundary_shift;
};

KnnPipelineLayout knn_layout(int n_vert, int n_coords, const SearchGrid &grid, int n_rs, int use_direction) {
    KnnPipelineLayout L{};
    const int n_bin_dims = grid.n_bin_dims, n_bins_scalar = grid.n_bins;
    // every per-dimension bin count is at most n_bins_scalar + 1
    long long bound = n_rs - 1;
    for (int i = 0; i < n_bin_dims; ++i) bound = std::min<long long>(bound * (n_bins_scalar + 1), 1ll << 40);
    L.total_bins_bound = (int)std::min<long long>(bound, (1ll << 31) - 2);
    L.nested = grid.nested && bin_grouping_spatial(L.total_bins_bound, n_bin_dims);
    L.boundary_shift = bin_grouping_sub_shift(L.total_bins_bound, n_bin_dims, L.nested);
    const size_t n = std::max(n_vert, 1);
    size_t off = 0;
    auto take = [&](size_t bytes) {
        size_t at = off;
        off += align_up(bytes);
        return at;
    };
    L.shift = take(8 * sizeof(float));
    L.bin_width = take(sizeof(float));
    L.n_bins = take(8 * sizeof(int));
    L.sorting = take(n * sizeof(int));
    L.bounds = take((((size_t)L.total_bins_bound << L.boundary_shift) + 1) * sizeof(int));
    L.bin_starts = take(((size_t)L.total_bins_bound + 1) * sizeof(int));
    L.scoords = take(n * n_coords * sizeof(float));
    L.sflat = take(n * sizeof(int));
    L.sbinass = take(n * (n_bin_dims + 1) * sizeof(int));
    L.sdir = take(use_direction ? n * sizeof(int) : 0);
    L.grouping_ws = take(bin_grouping_workspace_bytes(n_vert, L.total_bins_bound, n_bin_dims, L.nested));
    L.total = off;
    return L;
}

// ---- condensates ------------------------------------------------------------

constexpr int kMaxCoordDims = 16;

__device__ __forceinline__ uint32_t ordered_bits(float x) {
    const uint32_t u = __float_as_uint(x);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float from_ordered_bits(uint32_t u) {
    return __uint_as_float((u & 0x80000000u) ? (u & 0x7fffffffu) : ~u);
}

// Column minima and maxima (NaN ignored) as order-preserving bit patterns, combined with
// atomicMin: range[c] = pattern of the minimum, range[kMaxCoordDims + c] = complement of the
// pattern of the maximum. Both start at 0xffffffff.
__global__ __launch_bounds__(256) void column_range_kernel(const float *__restrict__ x, int n, int C,
                                                           uint32_t *__restrict__ range) {
    __shared__ uint32_t s_range[2 * kMaxCoordDims];
    if (threadIdx.x < 2 * kMaxCoordDims) s_range[threadIdx.x] = 0xffffffffu;
    __syncthreads();
    uint32_t lo[kMaxCoordDims], hi[kMaxCoordDims];
#pragma unroll
    for (int c = 0; c < kMaxCoordDims; ++c) lo[c] = hi[c] = 0xffffffffu;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x)
#pragma unroll
        for (int c = 0; c < kMaxCoordDims; ++c)
            if (c < C) {
                const float v = x[(size_t)i * C + c];
                if (v == v) {
                    lo[c] = min(lo[c], ordered_bits(v));
                    hi[c] = min(hi[c], ~ordered_bits(v));
                }
            }
#pragma unroll
    for (int c = 0; c < kMaxCoordDims; ++c) {
        if (c < C) {
            uint32_t a = lo[c], b = hi[c];
            for (int off = 32; off > 0; off >>= 1) {
                a = min(a, (uint32_t)__shfl_xor((int)a, off, kWave));
                b = min(b, (uint32_t)__shfl_xor((int)b, off, kWave));
            }
            if (lane_id() == 0) {
                atomicMin(&s_range[c], a);
                atomicMin(&s_range[kMaxCoordDims + c], b);
            }
        }
    }
    __syncthreads();
    if (threadIdx.x < C) {
        atomicMin(&range[threadIdx.x], s_range[threadIdx.x]);
        atomicMin(&range[kMaxCoordDims + threadIdx.x], s_range[kMaxCoordDims + threadIdx.x]);
    }
}

// inputs moved into bin order, local radii scaled, the high-beta subset marked
__global__ __launch_bounds__(256) void condensate_inputs_kernel(const float *__restrict__ shifted,
                                                                const float *__restrict__ betas,
                                                                const float *__restrict__ dist,
                                                                const int *__restrict__ mask,
                                                                const int *__restrict__ sorting, int n, int C,
                                                                float beta_threshold, float distance_threshold,
                                                                float *__restrict__ coords_s,
                                                                float *__restrict__ betas_s,
                                                                float *__restrict__ dist_s, int *__restrict__ mask_s,
                                                                int *__restrict__ high, int *__restrict__ to_filtered) {
    const int at = blockIdx.x * blockDim.x + threadIdx.x;
    if (at >= n) return;
    const int i = sorting[at];
    for (int c = 0; c < C; ++c) coords_s[(size_t)at * C + c] = shifted[(size_t)i * C + c];
    const float b = betas[i];
    const int m = mask ? mask[i] : 0;
    betas_s[at] = b;
    dist_s[at] = dist[i] / distance_threshold;
    mask_s[at] = m;
    const bool is_high = b > beta_threshold || m > 0;
    high[at] = is_high;
    to_filtered[at] = is_high ? at : -1;
}

// {first hit of the high-beta subset, its mask, the second one's mask}
__global__ __launch_bounds__(1024) void first_two_high_kernel(const int *__restrict__ high,
                                                              const int *__restrict__ mask_s, int n,
                                                              int *__restrict__ quirk) {
    __shared__ int s_count[16], s_found[2];
    if (threadIdx.x < 2) s_found[threadIdx.x] = -1;
    __syncthreads();
    int found = 0;
    for (int base = 0; base < n && found < 2; base += 1024) {
        const int i = base + threadIdx.x;
        const bool h = i < n && high[i] != 0;
        const uint64_t m = __ballot(h);
        if (lane_id() == 0) s_count[threadIdx.x >> 6] = __popcll(m);
        __syncthreads();
        int before = 0, total = 0;
        for (int w = 0; w < 16; ++w) {
            if (w < (int)(threadIdx.x >> 6)) before += s_count[w];
            total += s_count[w];
        }
        const int nth = found + before + __popcll(m & ((1ull << lane_id()) - 1ull));
        if (h && nth < 2) s_found[nth] = i;
        found += total;
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        quirk[0] = s_found[0];
        quirk[1] = s_found[0] >= 0 ? mask_s[s_found[0]] : 0;
        quirk[2] = s_found[1] >= 0 ? mask_s[s_found[1]] : 0;
    }
}

// results back in the caller's order; the condensation points of all events as one list
__global__ __launch_bounds__(256) void condensate_outputs_kernel(const int *__restrict__ sorting,
                                                                 const int *__restrict__ assignment_s,
                                                                 const int *__restrict__ association_s,
                                                                 const int *__restrict__ is_alpha,
                                                                 const int *__restrict__ alpha_indices,
                                                                 const int *__restrict__ row_splits,
                                                                 const int *__restrict__ n_condensates, int n,
                                                                 int num_rows, int *__restrict__ assignment,
                                                                 int *__restrict__ association,
                                                                 unsigned char *__restrict__ is_cond,
                                                                 int *__restrict__ alpha_idx) {
    const int at = blockIdx.x * blockDim.x + threadIdx.x;
    if (at >= n) return;
    const int i = sorting[at];
    assignment[i] = assignment_s[at];
    association[i] = association_s[at];
    is_cond[i] = is_alpha[at] != 0;
    int lo = 1, hi = num_rows + 1;  // event = last r with row_splits[r] <= at
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (row_splits[mid] > at)
            hi = mid;
        else
            lo = mid + 1;
    }
    const int r = min(lo - 1, num_rows - 1);
    const int nth = at - row_splits[r];
    if (nth < n_condensates[r + 1] - n_condensates[r]) alpha_idx[n_condensates[r] + nth] = alpha_indices[at];
}

struct CondPipelineLayout {
    size_t mins, shifted, shift, bin_width, n_bins, binass, flat, sorting, bin_splits, coords_s, betas_s, dist_s,
        mask_s, high, to_filtered, quirk, taken, is_alpha, best, assignment_s, association_s, alpha_indices, setup_ws,
        sort_ws, core_ws, total;
    size_t setup_bytes, sort_bytes, core_bytes;
    int cells_bound, n_bin_dims;
};

bool cond_layout(int n_vert, int n_coords, int num_rows, int n_bins_scalar, int nbin_dims, CondPipelineLayout &L) {
    L = CondPipelineLayout{};
    L.n_bin_dims = std::min(n_coords, nbin_dims);
    long long cells = std::max(num_rows, 1);
    for (int d = 0; d < L.n_bin_dims; ++d) cells = std::min<long long>(cells * (n_bins_scalar + 1), 1ll << 40);
    if (cells >= (1ll << 31) - 2) return false;
    L.cells_bound = (int)cells;
    const size_t n = std::max(n_vert, 1);
    size_t off = 0;
    auto take = [&](size_t bytes) {
        size_t at = off;
        off += align_up(bytes);
        return at;
    };
    L.mins = take(2 * kMaxCoordDims * sizeof(uint32_t));
    L.shifted = take(n * n_coords * sizeof(float));
    L.shift = take(8 * sizeof(float));
    L.bin_width = take(sizeof(float));
    L.n_bins = take(8 * sizeof(int));
    L.binass = take(n * (L.n_bin_dims + 1) * sizeof(int));
    L.flat = take(n * sizeof(int));
    L.sorting = take(n * sizeof(int));
    L.bin_splits = take(((size_t)L.cells_bound + 1) * sizeof(int));
    L.coords_s = take(n * n_coords * sizeof(float));
    L.betas_s = take(n * sizeof(float));
    L.dist_s = take(n * sizeof(float));
    L.mask_s = take(n * sizeof(int));
    L.high = take(n * sizeof(int));
    L.to_filtered = take(n * sizeof(int));
    L.quirk = take(4 * sizeof(int));
    L.taken = take(n * sizeof(int));
    L.is_alpha = take(n * sizeof(int));
    L.best = take(n * sizeof(float));
    L.assignment_s = take(n * sizeof(int));
    L.association_s = take(n * sizeof(int));
    L.alpha_indices = take(n * sizeof(int));
    L.setup_bytes = hgc_bin_setup_workspace_bytes(n_vert, L.n_bin_dims);
    L.sort_bytes = hgc_sort_by_bin_workspace_bytes(n_vert, L.cells_bound);
    L.core_bytes = condensates_workspace_bytes(n_vert, n_vert, num_rows, n_coords);
    L.setup_ws = take(L.setup_bytes);
    L.sort_ws = take(L.sort_bytes);
    L.core_ws = take(L.core_bytes);
    L.total = off;
    return true;
}

}  // namespace

extern "C" {

size_t hgc_build_and_assign_condensates_workspace_bytes(int n_vert, int n_coords, int num_rows, int n_bins_scalar,
                                                        int nbin_dims) {
    CondPipelineLayout L;
    if (n_vert < 0 || n_coords < 1 || n_coords > kMaxCoordDims || num_rows < 0 || n_bins_scalar < 1 || nbin_dims < 1 ||
        nbin_dims > 6 || !cond_layout(n_vert, n_coords, num_rows, n_bins_scalar, nbin_dims, L))
        return 0;
    return L.total;
}

int hgc_build_and_assign_condensates(const float *d_ccoords, const float *d_betas, const float *d_dist,
                                     const int *d_no_condensation_mask, const int *d_row_splits, int n_vert,
                                     int n_coords, int num_rows, float beta_threshold, float distance_threshold,
                                     int assign_by_max_beta, int nbin_dims, int n_bins_scalar, int *d_assignment,
                                     int *d_association, int *d_alpha_idx, unsigned char *d_is_cond,
                                     int *d_n_condensates, void *workspace, size_t workspace_bytes,
                                     hgc_stream_t stream) {
    HGC_REQUIRE(n_vert >= 0 && num_rows >= 0, "bad sizes");
    HGC_REQUIRE(n_coords >= 1 && n_coords <= kMaxCoordDims, "1 <= coordinate dimensions <= %d", kMaxCoordDims);
    HGC_REQUIRE(nbin_dims >= 1 && nbin_dims <= 6, "1 <= nbin_dims <= 6");
    HGC_REQUIRE(n_bins_scalar >= 1, "n_bins must be positive");
    HGC_REQUIRE(distance_threshold > 0.f, "distance_threshold must be positive");
    HGC_REQUIRE(d_row_splits && d_n_condensates, "null pointer");
    hipStream_t s = as_stream(stream);
    if (n_vert == 0) return launch_fill_i32(d_n_condensates, 0, (long long)num_rows + 1, s);
    HGC_REQUIRE(num_rows >= 1, "hits without an event");
    HGC_REQUIRE(d_ccoords && d_betas && d_dist && d_assignment && d_association && d_alpha_idx && d_is_cond,
                "null pointer");
    CondPipelineLayout L;
    HGC_REQUIRE(cond_layout(n_vert, n_coords, num_rows, n_bins_scalar, nbin_dims, L),
                "bin table overflows int32: fewer bins or events per call");
    if (!workspace || !aligned256(workspace) || workspace_bytes < L.total)
        return fail(HGC_ERR_WORKSPACE, "condensates workspace missing, misaligned or too small");
    char *ws = static_cast<char *>(workspace);
    auto F = [&](size_t off) { return reinterpret_cast<float *>(ws + off); };
    auto I = [&](size_t off) { return reinterpret_cast<int *>(ws + off); };
    uint32_t *mins = reinterpret_cast<uint32_t *>(ws + L.mins);
    const int B = L.n_bin_dims;
    int rc;

    if ((rc = launch_fill_i32(reinterpret_cast<int *>(mins), -1, 2 * kMaxCoordDims, s))) return rc;
    column_range_kernel<<<std::max(1, std::min(512, ceil_div(n_vert, 1024))), 256, 0, s>>>(d_ccoords, n_vert,
                                                                                            n_coords, mins);
    if ((rc = check_launch("column_range"))) return rc;
    // coordinates shifted to their minimum, grid over the shifted coordinates, bin of every hit
    if ((rc = shift_and_bin(d_ccoords, mins, mins + kMaxCoordDims, d_row_splits, n_vert, n_coords, B, num_rows + 1,
                            n_bins_scalar, L.cells_bound, F(L.shifted), F(L.bin_width), I(L.n_bins), I(L.binass),
                            I(L.flat), s)))
        return rc;
    if ((rc = hgc_sort_by_bin(I(L.flat), n_vert, L.cells_bound, I(L.sorting), I(L.bin_splits), ws + L.sort_ws,
                              L.sort_bytes, stream)))
        return rc;
    condensate_inputs_kernel<<<ceil_div(n_vert, 256), 256, 0, s>>>(
        F(L.shifted), d_betas, d_dist, d_no_condensation_mask, I(L.sorting), n_vert, n_coords, beta_threshold,
        distance_threshold, F(L.coords_s), F(L.betas_s), F(L.dist_s), I(L.mask_s), I(L.high), I(L.to_filtered));
    if ((rc = check_launch("condensate_inputs"))) return rc;
    first_two_high_kernel<<<1, 1024, 0, s>>>(I(L.high), I(L.mask_s), n_vert, I(L.quirk));
    if ((rc = check_launch("first_two_high"))) return rc;
    // every hit is its own entry of the "high-beta" arrays; `high` says which ones count
    if ((rc = condensates_assign(n_coords, B, I(L.taken), F(L.coords_s), F(L.dist_s), F(L.betas_s), I(L.mask_s),
                                 I(L.is_alpha), I(L.sorting), d_row_splits, F(L.coords_s), I(L.mask_s),
                                 I(L.to_filtered), F(L.best), I(L.assignment_s), I(L.association_s), d_n_condensates,
                                 I(L.alpha_indices), I(L.bin_splits), I(L.n_bins), F(L.bin_width), d_row_splits,
                                 num_rows, assign_by_max_beta, n_vert, n_vert, nullptr, I(L.high), I(L.quirk),
                                 ws + L.core_ws, L.core_bytes, s)))
        return rc;
    condensate_outputs_kernel<<<ceil_div(n_vert, 256), 256, 0, s>>>(
        I(L.sorting), I(L.assignment_s), I(L.association_s), I(L.is_alpha), I(L.alpha_indices), d_row_splits,
        d_n_condensates, n_vert, num_rows, d_assignment, d_association, d_is_cond, d_alpha_idx);
    return check_launch("condensate_outputs");
}

int hgc_set_knn_grid(int use_callers_grid) {
    g_callers_knn_grid = use_callers_grid != 0;
    return HGC_OK;
}

int hgc_get_knn_grid(void) { return g_callers_knn_grid; }

size_t hgc_binned_select_knn_pipeline_workspace_bytes(int n_vert, int n_coords, int n_rs, int n_bins_scalar,
                                                      int max_bin_dims, int use_direction) {
    const SearchGrid asked = callers_grid(n_coords, n_bins_scalar, max_bin_dims);
    if (n_vert < 0 || n_coords < 1 || n_rs < 2 || n_bins_scalar < 1 || asked.n_bin_dims < 1 || asked.n_bin_dims > 5)
        return 0;
    // enough for either grid, whichever hgc_set_knn_grid selects at the time of the call, and for
    // the library's own grid at any number of neighbours (the coarser grids of larger numbers can be
    // nested ones where the finest is not)
    size_t bytes = knn_layout(n_vert, n_coords, asked, n_rs, use_direction).total;
    for (int k = kSmallestGridK; k <= kLargestGridK; k *= 2)
        bytes = std::max(bytes, knn_layout(n_vert, n_coords, own_grid(n_vert, n_coords, n_rs, k), n_rs, use_direction).total);
    return bytes;
}

int hgc_binned_select_knn_pipeline_static(const float *d_coords, const int *d_row_splits, const int *d_direction,
                                          int n_vert, int n_coords, int n_rs, int n_neigh, int n_bins_scalar,
                                          int max_bin_dims, int tf_compat, float max_radius, int *d_indices,
                                          float *d_dist, int *d_out_sorting, hgc_stream_t stream) {
    const size_t need = hgc_binned_select_knn_pipeline_workspace_bytes(n_vert, n_coords, n_rs, n_bins_scalar,
                                                                       max_bin_dims, d_direction != nullptr);
    if (need > (size_t)HGC_STATIC_SCRATCH_BYTES)
        return fail(HGC_ERR_WORKSPACE,
                    "this call needs %zu bytes of scratch, the built-in array holds %zu: use "
                    "hgc_binned_select_knn_pipeline with a workspace of your own", need,
                    (size_t)HGC_STATIC_SCRATCH_BYTES);
    void *ptr = nullptr;
    if (int rc = static_scratch(&ptr)) return rc;
    return hgc_binned_select_knn_pipeline(d_coords, d_row_splits, d_direction, n_vert, n_coords, n_rs, n_neigh,
                                          n_bins_scalar, max_bin_dims, tf_compat, max_radius, d_indices, d_dist,
                                          d_out_sorting, ptr, HGC_STATIC_SCRATCH_BYTES, stream);
}

int hgc_binned_select_knn_pipeline(const float *d_coords, const int *d_row_splits, const int *d_direction,
                                   int n_vert, int n_coords, int n_rs, int n_neigh, int n_bins_scalar,
                                   int max_bin_dims, int tf_compat, float max_radius, int *d_indices,
                                   float *d_dist, int *d_out_sorting, void *workspace, size_t workspace_bytes,
                                   hgc_stream_t stream) {
    HGC_REQUIRE(n_vert >= 0 && n_rs >= 2, "bad sizes");
    HGC_REQUIRE(n_bins_scalar >= 1, "n_bins must be positive");
    HGC_REQUIRE(std::min(max_bin_dims, n_coords) > 1, "BinnedSelectKnnOp expects at least 2 binning dimensions.");
    HGC_REQUIRE(std::min(max_bin_dims, n_coords) < 6, "BinnedSelectKnnOp expects maximum 5 binning dimensions.");
    const SearchGrid grid = search_grid(n_vert, n_coords, n_rs, n_neigh, n_bins_scalar, max_bin_dims);
    const int n_bin_dims = grid.n_bin_dims;
    n_bins_scalar = grid.n_bins;
    {   // the rows of bins of the grid (all dimensions but the last), which bound the rows of a shell, stay below 2^22
        long long rows = 1;
        for (int i = 0; i < n_bin_dims - 1; ++i) rows = std::min(rows * (n_bins_scalar + 1ll), 1ll << 40);
        HGC_REQUIRE(rows < (1ll << 22), "n_bins = %d is too fine for %d binned dimensions (the grid would have %lld "
                    "rows of bins, the limit is 2^22)", n_bins_scalar, n_bin_dims, rows);
    }
    if (n_vert == 0) return HGC_OK;
    HGC_REQUIRE(d_coords && d_row_splits && d_indices && d_dist, "null pointer");
    const int use_direction = d_direction != nullptr;
    const KnnPipelineLayout L = knn_layout(n_vert, n_coords, grid, n_rs, use_direction);
    HGC_REQUIRE(L.total_bins_bound < (1ll << 31) - 2, "bin table overflows int32: fewer bins or events per call");
    if (!workspace || !aligned256(workspace) || workspace_bytes < L.total)
        return fail(HGC_ERR_WORKSPACE, "kNN pipeline workspace missing, misaligned or too small");
    char *ws = static_cast<char *>(workspace);
    float *shift = reinterpret_cast<float *>(ws + L.shift);
    float *bin_width = reinterpret_cast<float *>(ws + L.bin_width);
    int *n_bins = reinterpret_cast<int *>(ws + L.n_bins);
    int *sorting = d_out_sorting ? d_out_sorting : reinterpret_cast<int *>(ws + L.sorting);
    int *bounds = reinterpret_cast<int *>(ws + L.bounds);
    int *bin_starts = reinterpret_cast<int *>(ws + L.bin_starts);
    float *scoords = reinterpret_cast<float *>(ws + L.scoords);
    int *sflat = reinterpret_cast<int *>(ws + L.sflat);
    int *sbinass = reinterpret_cast<int *>(ws + L.sbinass);
    int *sdir = use_direction ? reinterpret_cast<int *>(ws + L.sdir) : nullptr;

    // The search needs the points grouped by bin, not a particular order inside a
    // bin: its results are in the caller's index space and in canonical order.
    const int rc = bin_grouping(d_coords, d_row_splits, d_direction, n_vert, n_coords, n_bin_dims, n_rs, n_bins_scalar,
                                L.total_bins_bound, shift, bin_width, n_bins, bounds, sorting, scoords, sflat, sbinass,
                                sdir, L.nested, bin_starts, ws + L.grouping_ws, L.total - L.grouping_ws, as_stream(stream));
    if (rc) return rc;
    return binned_select_knn_strided(scoords, sflat, sdir, sbinass, bin_starts, 0, n_bins, bin_width,
                                     sorting, shift, max_radius, d_indices, d_dist, n_vert, n_neigh, n_coords,
                                     n_bin_dims, L.total_bins_bound + 1, tf_compat, use_direction,
                                     L.nested ? bounds : nullptr, L.nested ? n_bin_dims : 0, std::max(n_neigh - 1, 1) / kCrowdedBinFraction,
                                     as_stream(stream));
}

}  // extern "C"
