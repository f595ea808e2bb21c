// Object-condensation condensate assignment: greedy highest-beta-first
// selection of condensation points with radius claims, per event.
//
// Reference behaviour restated here:
//   modules/compiled/binned_assign_to_condensates_kernel.cc:23-125  (claim step)
//   modules/compiled/binned_assign_to_condensates_kernel.cc:128-241 (greedy loop)
//   modules/compiled/binstepper.h:100-165                           (box of bins)
//
// The reference picks, again and again, the unclaimed high-beta hit with the
// largest beta (first one in bin order on ties) by a linear scan. That order
// is static, so here the high-beta hits of every event are sorted ONCE by
// (event, beta descending, position ascending) with a stable radix sort, and
// one workgroup per event walks its list: the next hit that is still unclaimed
// becomes a condensation point and all 1024 threads test the hits of its box of
// bins (contiguous runs of the bin-sorted hits) in parallel. Only distances
// (serial fp32 over the coordinates, no FMA contraction) and comparisons are
// involved, so the result is the reference's bit for bit.
//
// This is latency-bound (a chain of a few hundred dependent claim steps per
// event), not bandwidth-bound: compulsory traffic is about N*(4C+16) bytes.
#include "hgc_common.hpp"

#include <cstring>
#include <algorithm>

#include <rocprim/rocprim.hpp>

namespace hgc {

int launch_fill_i32(int *p, int value, long long n, hipStream_t s);

namespace {

constexpr int kMaxDims = 16;     // coordinate dimensions
constexpr int kMaxBinDims = 6;   // binned dimensions
constexpr int kBlock = 1024;
constexpr int kWavesPerBlock = kBlock / kWave;

struct CondParams {
    int C, B;
    int *taken_h;
    const float *ccoords_h;
    const float *dist_h;
    const float *beta_h;
    const int *mask_h;
    int *is_alpha_h;
    const int *orig_h;
    const int *row_splits_h;
    const float *ccoords;
    const int *mask;
    const int *to_filtered;
    float *best_dsq;
    int *assignment;
    int *association;
    int *alpha_indices;
    const int *bin_splits;
    const int *n_bins;
    const float *bin_widths;
    const int *row_splits;
    int num_rows, by_max_beta, n_vert, n_vert_h;
    const int *order_h;   // high-beta hits in selection order, grouped by event
    int *event_count;     // condensates found per event
};

// the reference indexes the high-beta mask with the truth value of (q > 0)
__device__ __forceinline__ bool always_first(const int *mask_h, int n_vert_h, int q) {
    const int slot = q > 0 ? 1 : 0;
    return slot < n_vert_h && mask_h[slot] != 0;
}

// ascending sort key == selection order
__global__ __launch_bounds__(256) void selection_keys_kernel(const float *__restrict__ beta_h,
                                                             const int *__restrict__ mask_h,
                                                             const int *__restrict__ row_splits_h, int num_rows,
                                                             int n_vert_h, uint64_t *__restrict__ keys,
                                                             int *__restrict__ values) {
    const int q = blockIdx.x * blockDim.x + threadIdx.x;
    if (q >= n_vert_h) return;
    int lo = 1, hi = num_rows + 1;  // event = last r with row_splits_h[r] <= q
    while (lo < hi) {
        int mid = (lo + hi) >> 1;
        if (row_splits_h[mid] > q)
            hi = mid;
        else
            lo = mid + 1;
    }
    const uint64_t ev = (uint64_t)(lo - 1);
    uint64_t cls, low;
    if (always_first(mask_h, n_vert_h, q)) {
        cls = 0;  // chosen as soon as it is the first unclaimed one, in position order
        low = 0;
    } else {
        const float b = beta_h[q];
        uint32_t u = __float_as_uint(b);
        u = (u & 0x80000000u) ? ~u : (u | 0x80000000u);  // monotone map float -> uint
        low = (uint32_t)~u;                               // larger beta first
        cls = (b > -1.f) ? 1 : 2;                         // beta <= -1 (or NaN) is never picked
    }
    keys[q] = (ev << 34) | (cls << 32) | low;
    values[q] = q;
}

__global__ __launch_bounds__(kBlock) void condensate_event_kernel(const CondParams p) {
    const int r = blockIdx.x;
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid >> 6;
    const int first = p.row_splits[r], last = p.row_splits[r + 1];
    const int first_h = p.row_splits_h[r], last_h = p.row_splits_h[r + 1];

    for (int q = first_h + tid; q < last_h; q += kBlock) {
        p.is_alpha_h[q] = 0;
        p.taken_h[q] = 0;
        p.alpha_indices[q] = -1;
    }
    for (int i = first + tid; i < last; i += kBlock) {
        p.assignment[i] = -1;
        p.association[i] = -1;
        if (!p.by_max_beta) p.best_dsq[i] = 10e20f;
    }

    const int C = p.C, B = p.B;
    int nb[kMaxBinDims];
    int cells = 1;
#pragma unroll
    for (int d = 0; d < kMaxBinDims; ++d) {
        nb[d] = d < B ? p.n_bins[d] : 1;
        cells *= nb[d];
    }
    const int *bin_splits = p.bin_splits + (size_t)cells * r;
    const float bw = p.bin_widths[0];

    __shared__ int s_first[kWavesPerBlock];
    __shared__ int s_pick;
    __syncthreads();

    int cursor = first_h;  // everything before it in the order is claimed
    int shower = 0;
    while (cursor < last_h) {
        // ---- next unclaimed hit in selection order ----
        const int pos = cursor + tid;
        bool open = false;
        if (pos < last_h) {
            const int q = p.order_h[pos];
            open = p.taken_h[q] == 0 && (always_first(p.mask_h, p.n_vert_h, q) || p.beta_h[q] > -1.f);
        }
        const uint64_t b = __ballot(open);
        if (lane == 0) s_first[wave] = b ? wave * kWave + (__ffsll((long long)b) - 1) : kBlock;
        __syncthreads();
        if (tid == 0) {
            int best = kBlock;
            for (int w = 0; w < kWavesPerBlock; ++w) best = min(best, s_first[w]);
            s_pick = best;
        }
        __syncthreads();
        const int pick = s_pick;
        if (pick == kBlock) {  // nothing open in this window
            cursor += kBlock;
            __syncthreads();
            continue;
        }
        cursor += pick;
        const int alpha = p.order_h[cursor];

        // ---- claim step: all threads test the hits of alpha's box of bins ----
        float centre[kMaxDims];
#pragma unroll
        for (int c = 0; c < kMaxDims; ++c) centre[c] = c < C ? p.ccoords_h[(size_t)alpha * C + c] : 0.f;
        float radius = p.dist_h[alpha];
        const float radius_sq = radius * radius;
        const bool solitary = p.mask_h[alpha] > 0;
        if (solitary) radius = 0.f;

        int lo_bin[kMaxBinDims], width[kMaxBinDims];
        int n_rows = 1;
#pragma unroll
        for (int d = 0; d < kMaxBinDims; ++d) {
            lo_bin[d] = 0;
            width[d] = 1;
            if (d < B) {
                const float lo = centre[d] - radius;
                const float hi = centre[d] + radius;
                float fl = floorf(lo / bw), fh = ceilf(hi / bw);
                // keep the walk finite for absurd radii; the clamped range still
                // covers every bin of the grid in this dimension
                fl = fminf(fmaxf(fl, (float)(-nb[d])), (float)(2 * nb[d]));
                fh = fminf(fmaxf(fh, (float)(-nb[d])), (float)(2 * nb[d]));
                lo_bin[d] = (int)fl;
                width[d] = (int)fh - (int)fl + 1;
                if (d < B - 1) n_rows *= width[d];
            }
        }
        const int run_lo = lo_bin[B - 1], run_hi = lo_bin[B - 1] + width[B - 1] - 1;
        const int shower_orig = p.orig_h[alpha];

        for (int row = wave; row < n_rows; row += kWavesPerBlock) {
            // per-dimension indices are not range checked (only the flat index
            // is), like the reference
            long long base = 0;
            int rem = row;
            long long stride = nb[B - 1];
            for (int d = B - 2; d >= 0; --d) {
                const int k = lo_bin[d] + rem % width[d];
                rem /= width[d];
                base += (long long)k * stride;
                stride *= nb[d];
            }
            long long a = base + run_lo, z = base + run_hi;
            if (a < 0) a = 0;
            if (z > cells - 1) z = cells - 1;
            if (a > z) continue;
            const int hit_lo = bin_splits[a], hit_hi = bin_splits[z + 1];
            for (int i = hit_lo + lane; i < hit_hi; i += kWave) {
                if (p.by_max_beta && p.assignment[i] != -1) continue;
                float dsq = 0.f;
                for (int c = 0; c < C; ++c) {
                    const float t = centre[c] - p.ccoords[(size_t)i * C + c];
                    dsq = dsq + t * t;
                }
                const int filt = p.to_filtered[i];
                const bool inside = (dsq <= radius_sq && !solitary && p.mask[i] == 0) || (solitary && filt == alpha);
                if (!inside) continue;
                if (!p.by_max_beta) {
                    const float lhs = p.best_dsq[i] * radius_sq;
                    if (!(lhs >= dsq)) continue;
                    p.best_dsq[i] = dsq;
                }
                p.assignment[i] = shower;
                p.association[i] = shower_orig;
                if (filt != -1) p.taken_h[filt] = 1;
            }
        }
        if (tid == 0) {
            p.is_alpha_h[alpha] = 1;
            p.taken_h[alpha] = 1;
            p.alpha_indices[first_h + shower] = shower_orig;
        }
        ++shower;
        ++cursor;
        __syncthreads();  // claims visible to the whole workgroup before the next pick
    }
    if (tid == 0) p.event_count[r] = shower;
}

__global__ void cumulative_counts_kernel(const int *__restrict__ event_count, int num_rows,
                                         int *__restrict__ n_condensates, int *__restrict__ error) {
    if (blockIdx.x != 0 || threadIdx.x != 0) return;
    int run = 0;
    n_condensates[0] = 0;
    for (int r = 0; r < num_rows; ++r) {
        run += event_count[r];
        n_condensates[r + 1] = run;
    }
    if (error) *error = 0;
}

int selection_key_bits(int num_rows) {
    int bits = 1;
    while (bits < 30 && (1ll << bits) < (long long)num_rows) ++bits;
    return 34 + bits;
}

}  // namespace
}  // namespace hgc

using namespace hgc;

extern "C" {

size_t hgc_binned_assign_to_condensates_workspace_bytes(int n_vert, int n_vert_h, int num_rows) {
    (void)n_vert;
    const size_t nh = std::max(n_vert_h, 1);
    size_t temp = 0;
    (void)rocprim::radix_sort_pairs(nullptr, temp, (const uint64_t *)nullptr, (uint64_t *)nullptr,
                                    (const int *)nullptr, (int *)nullptr, nh, 0,
                                    selection_key_bits(std::max(num_rows, 1)), (hipStream_t) nullptr);
    return align_up(temp) + 2 * align_up(nh * sizeof(uint64_t)) + 2 * align_up(nh * sizeof(int)) +
           align_up((size_t)std::max(num_rows, 1) * sizeof(int));
}

int hgc_binned_assign_to_condensates(int dimensions, int dimensions_binning, int *d_condensates_assigned_h,
                                     const float *d_ccoords_h, const float *d_dist_h, const float *d_beta_h,
                                     const int *d_no_condensation_mask_h, int *d_high_assigned_status_h,
                                     const int *d_original_indices_h, const int *d_row_splits_h,
                                     const float *d_ccoords, const float *d_dist,
                                     const int *d_no_condensation_mask, const int *d_indices_to_filtered,
                                     float *d_assignment_min_distance, int *d_assignment, int *d_association,
                                     int *d_n_condensates, int *d_alpha_indices, const int *d_bin_splits,
                                     const int *d_n_bins, const float *d_bin_widths, const int *d_row_splits,
                                     int num_rows, int assign_by_max_beta, int n_vert, int n_vert_h, int *d_error,
                                     void *workspace, size_t workspace_bytes, hgc_stream_t stream) {
    (void)d_dist;  // carried by the reference functor, never read by its kernel
    HGC_REQUIRE(dimensions >= 1 && dimensions <= kMaxDims, "1 <= coordinate dimensions <= %d", kMaxDims);
    HGC_REQUIRE(dimensions_binning >= 1 && dimensions_binning <= kMaxBinDims && dimensions_binning <= dimensions,
                "1 <= binning dimensions <= min(%d, coordinate dimensions)", kMaxBinDims);
    HGC_REQUIRE(num_rows >= 0 && n_vert >= 0 && n_vert_h >= 0 && n_vert_h <= n_vert, "bad sizes");
    HGC_REQUIRE(d_n_condensates && d_row_splits && d_row_splits_h, "null pointer");
    hipStream_t s = as_stream(stream);
    if (!workspace || !aligned256(workspace) ||
        workspace_bytes < hgc_binned_assign_to_condensates_workspace_bytes(n_vert, n_vert_h, num_rows))
        return fail(HGC_ERR_WORKSPACE, "condensates workspace missing, misaligned or too small");
    if (n_vert > 0)
        HGC_REQUIRE(d_ccoords && d_no_condensation_mask && d_indices_to_filtered && d_assignment && d_association &&
                        d_bin_splits && d_n_bins && d_bin_widths && (assign_by_max_beta || d_assignment_min_distance),
                    "null pointer");
    if (n_vert_h > 0)
        HGC_REQUIRE(d_condensates_assigned_h && d_ccoords_h && d_dist_h && d_beta_h && d_no_condensation_mask_h &&
                        d_high_assigned_status_h && d_original_indices_h && d_alpha_indices,
                    "null pointer");

    const size_t nh = std::max(n_vert_h, 1);
    Carver carve(workspace);
    uint64_t *keys = carve.take<uint64_t>(nh);
    uint64_t *keys_sorted = carve.take<uint64_t>(nh);
    int *values = carve.take<int>(nh);
    int *order = carve.take<int>(nh);
    int *event_count = carve.take<int>(std::max(num_rows, 1));
    void *temp = carve.base + carve.used;
    size_t temp_bytes = workspace_bytes - carve.used;

    if (n_vert_h > 0) {
        selection_keys_kernel<<<ceil_div(n_vert_h, 256), 256, 0, s>>>(d_beta_h, d_no_condensation_mask_h,
                                                                      d_row_splits_h, num_rows, n_vert_h, keys, values);
        int rc = check_launch("selection_keys");
        if (rc) return rc;
        HGC_HIP(rocprim::radix_sort_pairs(temp, temp_bytes, keys, keys_sorted, values, order, (size_t)n_vert_h, 0,
                                          selection_key_bits(num_rows), s));
    }
    if (num_rows > 0) {
        CondParams p;
        p.C = dimensions;
        p.B = dimensions_binning;
        p.taken_h = d_condensates_assigned_h;
        p.ccoords_h = d_ccoords_h;
        p.dist_h = d_dist_h;
        p.beta_h = d_beta_h;
        p.mask_h = d_no_condensation_mask_h;
        p.is_alpha_h = d_high_assigned_status_h;
        p.orig_h = d_original_indices_h;
        p.row_splits_h = d_row_splits_h;
        p.ccoords = d_ccoords;
        p.mask = d_no_condensation_mask;
        p.to_filtered = d_indices_to_filtered;
        p.best_dsq = d_assignment_min_distance;
        p.assignment = d_assignment;
        p.association = d_association;
        p.alpha_indices = d_alpha_indices;
        p.bin_splits = d_bin_splits;
        p.n_bins = d_n_bins;
        p.bin_widths = d_bin_widths;
        p.row_splits = d_row_splits;
        p.num_rows = num_rows;
        p.by_max_beta = assign_by_max_beta;
        p.n_vert = n_vert;
        p.n_vert_h = n_vert_h;
        p.order_h = order;
        p.event_count = event_count;
        condensate_event_kernel<<<num_rows, kBlock, 0, s>>>(p);
        int rc = check_launch("condensate_event_kernel");
        if (rc) return rc;
    }
    cumulative_counts_kernel<<<1, 64, 0, s>>>(event_count, num_rows, d_n_condensates, d_error);
    return check_launch("cumulative_counts");
}

}  // extern "C"
