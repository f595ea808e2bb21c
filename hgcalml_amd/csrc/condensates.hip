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

// claimed flags of the event's high-beta hits: one bit each, in LDS when they
// fit (LDS_FLAGS), else the caller's int array in global memory
template <bool LDS_FLAGS>
struct TakenFlags {
    uint32_t *bits;  // LDS
    int *global;     // taken_h + first_h
    __device__ __forceinline__ bool test(int local) const {
        if (LDS_FLAGS) return (bits[local >> 5] >> (local & 31)) & 1u;
        return global[local] != 0;
    }
    __device__ __forceinline__ void set(int local) const {
        if (LDS_FLAGS)
            atomicOr(&bits[local >> 5], 1u << (local & 31));
        else
            global[local] = 1;
    }
};

constexpr int kHitsPerThread = 4;

// LDS_FLAGS: claimed flags of the high-beta hits in LDS. ASSIGNED_BITS (max-beta
// mode only, where an assigned hit is never looked at again): one bit per hit of
// the event in LDS says whether it is assigned, so that the claim step loads
// coordinates and masks of unassigned hits only; most hits of a box belong to
// earlier condensates, and one CU's load bandwidth is what the step waits for.
template <bool LDS_FLAGS, bool ASSIGNED_BITS>
__global__ __launch_bounds__(kBlock) void condensate_event_kernel(const CondParams p, int flag_words,
                                                                  int assigned_words) {
    extern __shared__ uint32_t s_bits[];
    __shared__ int s_first[kWavesPerBlock];
    __shared__ int s_pick, s_alpha, s_alpha_mask, s_alpha_orig;
    __shared__ float s_alpha_centre[kMaxDims], s_alpha_dist;
    __shared__ int s_row_off[kBlock + 1];
    __shared__ int s_row_start[kBlock];
    __shared__ int s_wave_tot[kWavesPerBlock];

    const int r = blockIdx.x;
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid >> 6;
    const int first = p.row_splits[r], last = p.row_splits[r + 1];
    const int first_h = p.row_splits_h[r], last_h = p.row_splits_h[r + 1];
    const TakenFlags<LDS_FLAGS> taken{s_bits, p.taken_h + first_h};

    for (int q = first_h + tid; q < last_h; q += kBlock) {
        p.is_alpha_h[q] = 0;
        p.taken_h[q] = 0;
        p.alpha_indices[q] = -1;
    }
    if (LDS_FLAGS)
        for (int i = tid; i < flag_words; i += kBlock) s_bits[i] = 0;
    uint32_t *const s_assigned = s_bits + flag_words;
    if (ASSIGNED_BITS)
        for (int i = tid; i < assigned_words; i += kBlock) s_assigned[i] = 0;
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
    const float edge_slack = 1e-3f * bw;  // bins are cut by a rounded fp32 divide
    __syncthreads();

    int cursor = first_h;  // everything before it in the selection order is claimed
    int window = -1;       // start of the 1024 order entries cached in registers
    int my_q = -1;
    bool my_selectable = false;
    // what a claim step needs of this thread's entry, fetched with the window so that
    // the step does not wait for a load that depends on the pick
    float my_centre[kMaxDims], my_dist = 0.f;
    int my_mask = 0, my_orig = -1;
#pragma unroll
    for (int c = 0; c < kMaxDims; ++c) my_centre[c] = 0.f;
    int shower = 0;
    while (cursor < last_h) {
        // ---- next unclaimed hit in selection order ----
        if (window < 0 || cursor >= window + kBlock) {
            window = cursor;
            const int pos = window + tid;
            my_q = pos < last_h ? p.order_h[pos] : -1;
            my_selectable = my_q >= 0 && (always_first(p.mask_h, p.n_vert_h, my_q) || p.beta_h[my_q] > -1.f);
            if (my_q >= 0) {
#pragma unroll
                for (int c = 0; c < kMaxDims; ++c)
                    if (c < C) my_centre[c] = p.ccoords_h[(size_t)my_q * C + c];
                my_dist = p.dist_h[my_q];
                my_mask = p.mask_h[my_q];
                my_orig = p.orig_h[my_q];
            }
        }
        const bool open = my_selectable && window + tid >= cursor && !taken.test(my_q - first_h);
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
            cursor = window + kBlock;
            __syncthreads();
            continue;
        }
        if (tid == pick) {
            s_alpha = my_q;
            s_alpha_dist = my_dist;
            s_alpha_mask = my_mask;
            s_alpha_orig = my_orig;
#pragma unroll
            for (int c = 0; c < kMaxDims; ++c) s_alpha_centre[c] = my_centre[c];
        }
        __syncthreads();
        cursor = window + pick;
        const int alpha = s_alpha;

        // ---- claim step ----
        float centre[kMaxDims];
#pragma unroll
        for (int c = 0; c < kMaxDims; ++c) centre[c] = s_alpha_centre[c];
        float radius = s_alpha_dist;
        const float radius_sq = radius * radius;
        const bool solitary = s_alpha_mask > 0;
        if (solitary) radius = 0.f;
        const float reach_sq = radius * radius * 1.0001f;  // pruning bound, slightly generous

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
        const int shower_orig = s_alpha_orig;

        for (int row0 = 0; row0 < n_rows; row0 += kBlock) {
            // -- every thread resolves one row of the box into a run of hits --
            int start = 0, len = 0;
            const int row = row0 + tid;
            if (row < n_rows) {
                // per-dimension indices are not range checked (only the flat index
                // is), like the reference
                long long base = 0;
                int rem = row;
                long long stride = nb[B - 1];
                bool in_grid = true;
                float gap_sq = 0.f;
                for (int d = B - 2; d >= 0; --d) {
                    const int k = lo_bin[d] + rem % width[d];
                    rem /= width[d];
                    base += (long long)k * stride;
                    stride *= nb[d];
                    in_grid = in_grid && k >= 0 && k < nb[d];
                    // distance from the centre to the slab of bin k in this dimension
                    const float below = (float)k * bw - edge_slack - centre[d];
                    const float above = centre[d] - ((float)(k + 1) * bw + edge_slack);
                    const float gap = fmaxf(0.f, fmaxf(below, above));
                    gap_sq += gap * gap;
                }
                int k_lo = run_lo, k_hi = run_hi;
                bool keep = true;
                if (in_grid && !solitary) {
                    // rows of real bins can be pruned against the sphere: no hit of a
                    // skipped bin can pass d^2 <= radius^2 (slack covers fp rounding)
                    const float rest = reach_sq - gap_sq;
                    if (rest < 0.f) {
                        keep = false;
                    } else {
                        const float half = sqrtf(rest) + edge_slack;
                        k_lo = max(k_lo, (int)floorf((centre[B - 1] - half) / bw) - 1);
                        k_hi = min(k_hi, (int)floorf((centre[B - 1] + half) / bw) + 1);
                    }
                }
                long long a = base + k_lo, z = base + k_hi;
                if (a < 0) a = 0;
                if (z > cells - 1) z = cells - 1;
                if (keep && a <= z) {
                    start = bin_splits[a];
                    len = bin_splits[z + 1] - start;
                }
            }
            // -- exclusive scan of the run lengths over the workgroup --
            const int incl = wave_inclusive_sum(len);
            if (lane == kWave - 1) s_wave_tot[wave] = incl;
            __syncthreads();
            int wave_off = 0, total = 0;
#pragma unroll
            for (int w = 0; w < kWavesPerBlock; ++w) {
                const int t = s_wave_tot[w];
                if (w < wave) wave_off += t;
                total += t;
            }
            s_row_off[tid] = wave_off + incl - len;
            s_row_start[tid] = start;
            if (tid == 0) s_row_off[kBlock] = total;
            __syncthreads();

            // -- all hits of all runs, kHitsPerThread per thread with their loads batched --
            for (int h0 = 0; h0 < total; h0 += kBlock * kHitsPerThread) {
                int hit[kHitsPerThread];
                bool live[kHitsPerThread];
#pragma unroll
                for (int k = 0; k < kHitsPerThread; ++k) {
                    const int h = h0 + k * kBlock + tid;
                    live[k] = h < total;
                    // last row whose offset is <= h (empty rows share their successor's offset)
                    int lo_r = 0;
#pragma unroll
                    for (int step = kBlock / 2; step > 0; step >>= 1) {
                        const int probe = lo_r + step;
                        if (s_row_off[probe] <= h) lo_r = probe;
                    }
                    hit[k] = live[k] ? s_row_start[lo_r] + (h - s_row_off[lo_r]) : first;
                }
                if (ASSIGNED_BITS) {
#pragma unroll
                    for (int k = 0; k < kHitsPerThread; ++k) {
                        const int local = hit[k] - first;
                        live[k] = live[k] && !((s_assigned[local >> 5] >> (local & 31)) & 1u);
                    }
                }
                int asg[kHitsPerThread], filt[kHitsPerThread], msk[kHitsPerThread];
                float dsq[kHitsPerThread];
#pragma unroll
                for (int k = 0; k < kHitsPerThread; ++k) {
                    const int i = hit[k];
                    asg[k] = -1;
                    filt[k] = -1;
                    msk[k] = 1;
                    dsq[k] = 0.f;
                    if (ASSIGNED_BITS && !live[k]) continue;
                    if (!ASSIGNED_BITS && p.by_max_beta) asg[k] = p.assignment[i];
                    filt[k] = p.to_filtered[i];
                    msk[k] = p.mask[i];
                    float acc = 0.f;
                    for (int c = 0; c < C; ++c) {
                        const float t = centre[c] - p.ccoords[(size_t)i * C + c];
                        acc = acc + t * t;
                    }
                    dsq[k] = acc;
                }
#pragma unroll
                for (int k = 0; k < kHitsPerThread; ++k) {
                    if (!live[k]) continue;
                    const int i = hit[k];
                    if (p.by_max_beta && asg[k] != -1) continue;
                    const bool inside = (dsq[k] <= radius_sq && !solitary && msk[k] == 0) || (solitary && filt[k] == alpha);
                    if (!inside) continue;
                    if (!p.by_max_beta) {
                        const float lhs = p.best_dsq[i] * radius_sq;
                        if (!(lhs >= dsq[k])) continue;
                        p.best_dsq[i] = dsq[k];
                    }
                    p.assignment[i] = shower;
                    p.association[i] = shower_orig;
                    if (ASSIGNED_BITS) atomicOr(&s_assigned[(i - first) >> 5], 1u << ((i - first) & 31));
                    if (filt[k] != -1) taken.set(filt[k] - first_h);
                }
            }
            __syncthreads();  // LDS row tables are reused by the next tile / condensate
        }
        if (tid == 0) {
            p.is_alpha_h[alpha] = 1;
            taken.set(alpha - first_h);
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
        // One claimed-flag bit per high-beta hit of an event and, in max-beta mode, one
        // assigned bit per hit live in LDS when they fit (n_vert_h and n_vert bound
        // every event; the event sizes themselves are device data).
        const int flag_words = ceil_div(std::max(n_vert_h, 1), 32);
        const int assigned_words = ceil_div(std::max(n_vert, 1), 32);
        constexpr size_t kDynamicLdsLimit = 144 * 1024;  // of 160 KB; the kernel has ~9 KB of static tables
        const size_t flag_bytes = (size_t)flag_words * 4, both_bytes = flag_bytes + (size_t)assigned_words * 4;
        // more than the default 64 KB of dynamic LDS has to be granted per kernel; without
        // the grant the variant without assigned bits runs
        const bool with_assigned_bits =
            assign_by_max_beta && both_bytes <= kDynamicLdsLimit &&
            (both_bytes <= 48 * 1024 ||
             hipFuncSetAttribute(reinterpret_cast<const void *>(&condensate_event_kernel<true, true>),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)kDynamicLdsLimit) == hipSuccess);
        (void)hipGetLastError();  // a refused grant is not an error of this call
        if (with_assigned_bits) {
            condensate_event_kernel<true, true><<<num_rows, kBlock, both_bytes, s>>>(p, flag_words, assigned_words);
        } else if (flag_bytes <= 48 * 1024) {
            condensate_event_kernel<true, false><<<num_rows, kBlock, flag_bytes, s>>>(p, flag_words, 0);
        } else {
            condensate_event_kernel<false, false><<<num_rows, kBlock, 0, s>>>(p, 0, 0);
        }
        int rc = check_launch("condensate_event_kernel");
        if (rc) return rc;
    }
    cumulative_counts_kernel<<<1, 64, 0, s>>>(event_count, num_rows, d_n_condensates, d_error);
    return check_launch("cumulative_counts");
}

}  // extern "C"
