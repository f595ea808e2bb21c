// Spatial binning: grid parameters, per-point bin assignment, stable sort into
// bin order, bin boundary table, row gather and index replacement.
//
// Reference behaviour restated here:
//   modules/bin_by_coordinates_op.py:46-71            (grid parameters)
//   modules/compiled/bin_by_coordinates_kernel.cc:46-114 (assignment)
//   modules/binned_select_knn_op.py:72-84             (sort + boundaries)
//   modules/compiled/index_replacer_kernel.cc:29-40
//
// All of this is HBM-bound integer/byte work over N points (a few bytes per
// point per pass); the sort and the scans use rocPRIM device primitives.
#include "hgc_common.hpp"

#include <cstring>
#include <algorithm>

#include <rocprim/rocprim.hpp>

#include <cfloat>
#include <cmath>

namespace hgc {

thread_local char g_last_error[512] = "";
char *last_error_buffer() { return g_last_error; }

thread_local int *g_status_word = nullptr;
int *status_word() { return g_status_word; }

namespace {

constexpr int kMaxBinDims = 8;

__global__ void fill_i32_kernel(int *p, int value, long long n) {
    long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long stride = (long long)gridDim.x * blockDim.x;
    for (; i < n; i += stride) p[i] = value;
}

__global__ void iota_i32_kernel(int *p, int n) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = i;
}

// ---- grid parameters --------------------------------------------------------

// stage 1: per-block column minima / maxima of the first n_dims columns
// (also zeroes `clear[0, n_clear)` on the way, for callers that need a cleared table next)
__global__ __launch_bounds__(256) void column_minmax_kernel(const float *__restrict__ coords, int stride,
                                                            int n_vert, int n_dims,
                                                            float *__restrict__ partial /*[blocks][2][8]*/,
                                                            int *__restrict__ clear, long long n_clear) {
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n_clear;
         i += (long long)gridDim.x * blockDim.x)
        clear[i] = 0;
    float lo[kMaxBinDims], hi[kMaxBinDims];
#pragma unroll
    for (int c = 0; c < kMaxBinDims; ++c) {
        lo[c] = FLT_MAX;
        hi[c] = -FLT_MAX;
    }
    for (int p = blockIdx.x * blockDim.x + threadIdx.x; p < n_vert; p += gridDim.x * blockDim.x) {
#pragma unroll
        for (int c = 0; c < kMaxBinDims; ++c) {
            if (c < n_dims) {
                float x = coords[(size_t)p * stride + c];
                lo[c] = fminf(lo[c], x);
                hi[c] = fmaxf(hi[c], x);
            }
        }
    }
    __shared__ float s_lo[4][kMaxBinDims], s_hi[4][kMaxBinDims];
#pragma unroll
    for (int c = 0; c < kMaxBinDims; ++c) {
        float a = lo[c], b = hi[c];
        for (int off = 32; off > 0; off >>= 1) {
            a = fminf(a, __shfl_xor(a, off, kWave));
            b = fmaxf(b, __shfl_xor(b, off, kWave));
        }
        if (lane_id() == 0) {
            s_lo[threadIdx.x >> 6][c] = a;
            s_hi[threadIdx.x >> 6][c] = b;
        }
    }
    __syncthreads();
    if (threadIdx.x < kMaxBinDims) {
        int c = threadIdx.x;
        float a = fminf(fminf(s_lo[0][c], s_lo[1][c]), fminf(s_lo[2][c], s_lo[3][c]));
        float b = fmaxf(fmaxf(s_hi[0][c], s_hi[1][c]), fmaxf(s_hi[2][c], s_hi[3][c]));
        partial[((size_t)blockIdx.x * 2 + 0) * kMaxBinDims + c] = a;
        partial[((size_t)blockIdx.x * 2 + 1) * kMaxBinDims + c] = b;
    }
}

// shift, common bin width and bins per dimension from the column minima / maxima:
// the fp32 operations of modules/bin_by_coordinates_op.py:50-65 in their order
__device__ inline void derive_grid(const float *lo, const float *hi, int n_dims, int pre_normalized,
                                   int n_bins_scalar, const float *bin_width_in, float *shift, float *bin_width,
                                   int *n_bins) {
    float extent[kMaxBinDims];
    float bw = 0.f;
    for (int c = 0; c < n_dims; ++c) {
        const float sh = pre_normalized ? 0.f : lo[c];
        // the extent is the largest shifted coordinate; subtraction is monotonic,
        // so that is (column max - shift)
        float e = hi[c] - sh;
        const float shifted_min = lo[c] - sh;
        if (shifted_min == e) e = e + 1.f;
        e = e + 1e-3f;
        if (!isfinite(e)) e = 1.f;
        extent[c] = e;
        shift[c] = sh;
        if (n_bins_scalar > 0) bw = fmaxf(bw, e / (float)n_bins_scalar);
    }
    if (n_bins_scalar <= 0) bw = bin_width_in[0];
    bin_width[0] = bw;
    for (int c = 0; c < n_dims; ++c) {
        float nb = extent[c] / bw;
        nb = nb + 1.f;
        n_bins[c] = (int)nb;
    }
}

// stage 2: one wave folds the partials and derives shift / bin width / bin counts
__global__ __launch_bounds__(64) void grid_params_kernel(const float *__restrict__ partial, int n_partial,
                                                         int n_dims, int pre_normalized, int n_bins_scalar,
                                                         const float *__restrict__ bin_width_in,
                                                         float *__restrict__ shift, float *__restrict__ bin_width,
                                                         int *__restrict__ n_bins) {
    float lo[kMaxBinDims], hi[kMaxBinDims];
#pragma unroll
    for (int c = 0; c < kMaxBinDims; ++c) {
        float a = FLT_MAX, b = -FLT_MAX;
        for (int i = threadIdx.x; i < n_partial; i += kWave) {
            a = fminf(a, partial[((size_t)i * 2 + 0) * kMaxBinDims + c]);
            b = fmaxf(b, partial[((size_t)i * 2 + 1) * kMaxBinDims + c]);
        }
        for (int off = 32; off > 0; off >>= 1) {
            a = fminf(a, __shfl_xor(a, off, kWave));
            b = fmaxf(b, __shfl_xor(b, off, kWave));
        }
        lo[c] = a;
        hi[c] = b;
    }
    if (threadIdx.x != 0) return;
    derive_grid(lo, hi, n_dims, pre_normalized, n_bins_scalar, bin_width_in, shift, bin_width, n_bins);
}

// ---- per-point assignment ---------------------------------------------------

__global__ __launch_bounds__(256) void bin_points_kernel(
    const float *__restrict__ coords, int stride, const float *__restrict__ shift,
    const int *__restrict__ row_splits, const float *__restrict__ bin_width, const int *__restrict__ n_bins,
    int *__restrict__ binass, int *__restrict__ flat, int *__restrict__ n_per_bin,
    int *__restrict__ n_out_of_range, int *__restrict__ status, int n_vert, int n_dims, int n_rs, int n_total_bins,
    int calc_n_per_bin) {
    const int p = blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= n_vert) return;
    const float bw = bin_width[0];
    int mul = 1, cell = 0, bad = 0, flags = 0;
    for (int c = n_dims - 1; c >= 0; --c) {
        float x = coords[(size_t)p * stride + c];
        if (!isfinite(x)) flags |= HGC_FLAG_COORDINATE_NOT_FINITE;
        if (shift) x = x - shift[c];
        int k = (int)(x / bw);
        const int nb = n_bins[c];
        if (k < 0 || k >= nb) {
            k = 0;
            ++bad;
        }
        binass[(size_t)p * (n_dims + 1) + c + 1] = k;
        cell += k * mul;
        mul *= nb;
    }
    // event = number of row splits (from the second on) that are <= p; the
    // splits are non decreasing, so a binary search gives the linear scan's answer
    int lo = 1, hi = n_rs;
    while (lo < hi) {
        int mid = (lo + hi) >> 1;
        if (row_splits[mid] > p)
            hi = mid;
        else
            lo = mid + 1;
    }
    const int ev = lo - 1;
    cell += ev * mul;
    if (bad && n_out_of_range) atomicAdd(n_out_of_range, bad);
    if (bad) flags |= HGC_FLAG_COORDINATE_OUT_OF_GRID;
    if (flags && status) atomicOr(status, flags);
    if (cell >= n_total_bins) return;
    binass[(size_t)p * (n_dims + 1)] = ev;
    flat[p] = cell;
    if (calc_n_per_bin) atomicAdd(&n_per_bin[cell], 1);
}

// The same assignment fused with the condensate wrapper's shift to the column minima: every
// block derives the grid from the column ranges itself (pre-normalised coordinates: shift 0,
// extent = largest shifted value = max - min, rounding is monotonic).
__device__ __forceinline__ float from_ordered_pattern(uint32_t u) {
    return __uint_as_float((u & 0x80000000u) ? (u & 0x7fffffffu) : ~u);
}

__global__ __launch_bounds__(256) void shift_and_bin_kernel(
    const float *__restrict__ coords, const uint32_t *__restrict__ min_bits, const uint32_t *__restrict__ max_bits_inv,
    const int *__restrict__ row_splits, int n_vert, int n_coords, int n_dims, int n_rs, int n_bins_scalar,
    int n_total_bins, float *__restrict__ shifted, float *__restrict__ bin_width_out, int *__restrict__ n_bins_out,
    int *__restrict__ binass, int *__restrict__ flat, int *__restrict__ status) {
    __shared__ float s_min[16], s_bw;
    __shared__ int s_nb[kMaxBinDims];
    if (threadIdx.x < n_coords) s_min[threadIdx.x] = from_ordered_pattern(min_bits[threadIdx.x]);
    __syncthreads();
    if (threadIdx.x == 0) {
        float lo[kMaxBinDims], hi[kMaxBinDims], unused_shift[kMaxBinDims];
        for (int c = 0; c < n_dims; ++c) {
            lo[c] = s_min[c] - s_min[c];
            hi[c] = from_ordered_pattern(~max_bits_inv[c]) - s_min[c];
        }
        derive_grid(lo, hi, n_dims, 1, n_bins_scalar, nullptr, unused_shift, &s_bw, s_nb);
        if (blockIdx.x == 0) {
            for (int c = 0; c < n_dims; ++c) n_bins_out[c] = s_nb[c];
            bin_width_out[0] = s_bw;
        }
    }
    __syncthreads();
    const int p = blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= n_vert) return;
    const float bw = s_bw;
    int mul = 1, cell = 0, flags = 0;
    for (int c = n_coords - 1; c >= 0; --c) {
        const float x = coords[(size_t)p * n_coords + c] - s_min[c];
        shifted[(size_t)p * n_coords + c] = x;
        if (c >= n_dims) continue;
        if (!isfinite(x)) flags |= HGC_FLAG_COORDINATE_NOT_FINITE;
        int k = (int)(x / bw);
        const int nb = s_nb[c];
        if (k < 0 || k >= nb) {
            k = 0;
            flags |= HGC_FLAG_COORDINATE_OUT_OF_GRID;
        }
        binass[(size_t)p * (n_dims + 1) + c + 1] = k;
        cell += k * mul;
        mul *= nb;
    }
    int lo = 1, hi = n_rs;  // event: number of row splits (from the second on) that are <= p
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (row_splits[mid] > p)
            hi = mid;
        else
            lo = mid + 1;
    }
    const int ev = lo - 1;
    cell += ev * mul;
    if (flags && status) atomicOr(status, flags);
    if (cell >= n_total_bins) return;
    binass[(size_t)p * (n_dims + 1)] = ev;
    flat[p] = cell;
}

// ---- boundaries from the sorted keys -----------------------------------------

__global__ __launch_bounds__(256) void bin_boundaries_kernel(const int *__restrict__ sorted_bins, int n_vert,
                                                             int *__restrict__ boundaries, int n_total_bins) {
    const int b = blockIdx.x * blockDim.x + threadIdx.x;
    if (b > n_total_bins) return;
    int lo = 0, hi = n_vert;  // first position whose key is >= b
    while (lo < hi) {
        int mid = (lo + hi) >> 1;
        if (sorted_bins[mid] < b)
            lo = mid + 1;
        else
            hi = mid;
    }
    boundaries[b] = lo;
}

template <int W>
__global__ __launch_bounds__(256) void gather_rows_kernel(const uint32_t *__restrict__ in, const int *__restrict__ rows,
                                                          uint32_t *__restrict__ out, int n_rows, int width) {
    const long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const int w = W > 0 ? W : width;
    if (t >= (long long)n_rows * w) return;
    const int r = (int)(t / w), c = (int)(t - (long long)r * w);
    out[t] = in[(size_t)rows[r] * w + c];
}

__global__ __launch_bounds__(256) void index_replacer_kernel(const int *__restrict__ tbr, const int *__restrict__ repl,
                                                             int *__restrict__ out, int *__restrict__ status, int n,
                                                             int n_repl) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int v = tbr[i];
    if (v < 0)
        out[i] = v;
    else if (v < n_repl)
        out[i] = repl[v];
    else if (status)
        atomicOr(status, HGC_FLAG_REPLACEMENT_OUT_OF_RANGE);
}

// ---- bin order by counting (no order guarantee inside a bin) -------------------
//
// For callers that only need the points grouped by bin: a counting sort whose
// rank inside the bin is the order in which the points' atomic increments
// arrive. The kernels below follow column_minmax_kernel (which also clears the
// counters): every block folds the column minima / maxima and derives the grid
// itself, so there is no separate launch for that.

__global__ __launch_bounds__(256) void bin_points_ranked_kernel(
    const float *__restrict__ coords, int stride, const float *__restrict__ partial, int n_partial,
    const int *__restrict__ row_splits, int n_vert, int n_dims, int n_rs, int n_bins_scalar,
    float *__restrict__ shift_out, float *__restrict__ bin_width_out, int *__restrict__ n_bins_out,
    int *__restrict__ binass, int *__restrict__ flat, int *__restrict__ rank, int *__restrict__ counts,
    int n_bins_bound, int sub_shift, int spatial, int *__restrict__ status) {
    __shared__ float s_lo[4][kMaxBinDims], s_hi[4][kMaxBinDims];
    __shared__ float s_shift[kMaxBinDims], s_bw;
    __shared__ int s_nb[kMaxBinDims];
#pragma unroll
    for (int c = 0; c < kMaxBinDims; ++c) {
        float a = FLT_MAX, b = -FLT_MAX;
        for (int i = threadIdx.x; i < n_partial; i += blockDim.x) {
            a = fminf(a, partial[((size_t)i * 2 + 0) * kMaxBinDims + c]);
            b = fmaxf(b, partial[((size_t)i * 2 + 1) * kMaxBinDims + c]);
        }
        for (int off = 32; off > 0; off >>= 1) {
            a = fminf(a, __shfl_xor(a, off, kWave));
            b = fmaxf(b, __shfl_xor(b, off, kWave));
        }
        if (lane_id() == 0) {
            s_lo[threadIdx.x >> 6][c] = a;
            s_hi[threadIdx.x >> 6][c] = b;
        }
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        float lo[kMaxBinDims], hi[kMaxBinDims];
        for (int c = 0; c < kMaxBinDims; ++c) {
            lo[c] = fminf(fminf(s_lo[0][c], s_lo[1][c]), fminf(s_lo[2][c], s_lo[3][c]));
            hi[c] = fmaxf(fmaxf(s_hi[0][c], s_hi[1][c]), fmaxf(s_hi[2][c], s_hi[3][c]));
        }
        derive_grid(lo, hi, n_dims, 0, n_bins_scalar, nullptr, s_shift, &s_bw, s_nb);
        if (blockIdx.x == 0) {
            for (int c = 0; c < n_dims; ++c) {
                shift_out[c] = s_shift[c];
                n_bins_out[c] = s_nb[c];
            }
            bin_width_out[0] = s_bw;
        }
    }
    __syncthreads();
    const float bw = s_bw;
    for (int p = blockIdx.x * blockDim.x + threadIdx.x; p < n_vert; p += gridDim.x * blockDim.x) {
        int mul = 1, cell = 0, flags = 0, half = 0;
        int ks[kMaxBinDims];
        for (int c = n_dims - 1; c >= 0; --c) {
            const float raw = coords[(size_t)p * stride + c];
            if (!isfinite(raw)) flags |= HGC_FLAG_COORDINATE_NOT_FINITE;
            const float x = raw - s_shift[c];
            const float in_bins = x / bw;
            int k = (int)in_bins;
            const int nb = s_nb[c];
            if (k < 0 || k >= nb) {
                k = 0;
                flags |= HGC_FLAG_COORDINATE_OUT_OF_GRID;
            } else if (in_bins - (float)k >= 0.5f) {
                half |= 1 << (n_dims - 1 - c);  // upper half of the bin in this dimension (last dimension: bit 0)
            }
            ks[c] = k;
            cell += k * mul;
            mul *= nb;
        }
        int lo = 1, hi = n_rs;  // event: number of row splits (from the second on) that are <= p
        while (lo < hi) {
            const int mid = (lo + hi) >> 1;
            if (row_splits[mid] > p)
                hi = mid;
            else
                lo = mid + 1;
        }
        const int ev = lo - 1;
        cell += ev * mul;
        if (flags && status) atomicOr(status, flags);
        cell = min(cell, n_bins_bound - 1);  // no effect for row splits that end at n_vert
        if (n_dims == 3) {  // one 16-byte row (the workspace is aligned)
            reinterpret_cast<int4 *>(binass)[p] = make_int4(ev, ks[0], ks[1], ks[2]);
        } else {
            binass[(size_t)p * (n_dims + 1)] = ev;
            for (int c = 0; c < n_dims; ++c) binass[(size_t)p * (n_dims + 1) + c + 1] = ks[c];
        }
        // Every bin has 2^sub_shift counters, so that the increments of a crowded bin queue up on
        // several addresses instead of one. spatial (sub_shift = n_dims): the counter is the half of
        // the bin the point lies in, per dimension -- the bin's points then come grouped by these
        // 2^n_dims sub-cells, a grid of half the bin width nested in the bins, and the flat index
        // names the sub-cell. Otherwise a point takes the counter its index names.
        const int counter = (cell << sub_shift) | (spatial ? half : (p & ((1 << sub_shift) - 1)));
        flat[p] = spatial ? counter : cell;
        rank[p] = atomicAdd(&counts[counter], 1);
    }
}

// position of every point in bin order, and its inputs moved there: row `at` of every
// output is row sorting[at] of its input
__global__ __launch_bounds__(256) void move_to_bin_order_kernel(
    const float *__restrict__ coords, const int *__restrict__ binass, const int *__restrict__ flat,
    const int *__restrict__ rank, const int *__restrict__ direction, const int *__restrict__ boundaries, int n_vert,
    int n_coords, int n_dims, int sub_shift, int spatial, int rows_aligned, int *__restrict__ sorting,
    float *__restrict__ scoords, int *__restrict__ sflat, int *__restrict__ sbinass, int *__restrict__ sdir) {
    const int p = blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= n_vert) return;
    const int cell = flat[p];  // spatial: the sub-cell, which is its own counter
    const int at = boundaries[spatial ? (size_t)cell : ((size_t)cell << sub_shift) | (p & ((1 << sub_shift) - 1))] + rank[p];
    sorting[at] = p;
    sflat[at] = cell;
    if (n_coords == 4 && rows_aligned) {
        reinterpret_cast<float4 *>(scoords)[at] = reinterpret_cast<const float4 *>(coords)[p];
    } else if (n_coords == 3) {  // one 12-byte store per row instead of three of 4 bytes to a scattered address
        struct __attribute__((packed, aligned(4))) Row3 { float v[3]; };
        reinterpret_cast<Row3 *>(scoords)[at] = reinterpret_cast<const Row3 *>(coords)[p];
    } else {
        for (int c = 0; c < n_coords; ++c) scoords[(size_t)at * n_coords + c] = coords[(size_t)p * n_coords + c];
    }
    if (n_dims == 3) {
        reinterpret_cast<int4 *>(sbinass)[at] = reinterpret_cast<const int4 *>(binass)[p];
    } else {
        for (int c = 0; c <= n_dims; ++c) sbinass[(size_t)at * (n_dims + 1) + c] = binass[(size_t)p * (n_dims + 1) + c];
    }
    if (direction) sdir[at] = direction[p];
}

// ---- exclusive scan of the counters = the boundary table ----
// Two plain passes (sums of chunks of kScanChunk counters; then every chunk adds up the sums in
// front of it and scans itself): a few thousand chunks at most, and no chunk waits for another
// as in a single-pass scan with look-back (2.5 M counters: 9 us against 19 us for the library scan).
constexpr int kScanChunk = 2048;  // 256 threads x 8 counters
constexpr int kMaxScanChunks = 16384;

__global__ __launch_bounds__(256) void strided_copy_kernel(const int *__restrict__ in, int *__restrict__ out, int n,
                                                           int shift) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = in[(size_t)i << shift];
}

__global__ __launch_bounds__(256) void counter_chunk_sums_kernel(const int *__restrict__ counts, long long n,
                                                                 int *__restrict__ chunk_sums) {
    __shared__ int s_wave[4];
    const long long base = (long long)blockIdx.x * kScanChunk + threadIdx.x * 8;
    int sum = 0;
    if (base + 8 <= n) {
        const int4 a = *reinterpret_cast<const int4 *>(counts + base), b = *reinterpret_cast<const int4 *>(counts + base + 4);
        sum = a.x + a.y + a.z + a.w + b.x + b.y + b.z + b.w;
    } else {
        for (int j = 0; j < 8; ++j)
            if (base + j < n) sum += counts[base + j];
    }
    sum = wave_inclusive_sum(sum);
    if (lane_id() == kWave - 1) s_wave[threadIdx.x >> 6] = sum;
    __syncthreads();
    if (threadIdx.x == 0) chunk_sums[blockIdx.x] = s_wave[0] + s_wave[1] + s_wave[2] + s_wave[3];
}

// boundaries[i] = sum of counts[0 .. i); bin_starts[b] = boundaries[b << sub_shift] (may be null)
__global__ __launch_bounds__(256) void counter_scan_kernel(const int *__restrict__ counts, long long n,
                                                           const int *__restrict__ chunk_sums,
                                                           int *__restrict__ boundaries, int *__restrict__ bin_starts,
                                                           int sub_shift) {
    __shared__ int s_wave[4], s_before;
    int before = 0;  // the chunks in front of this one
    for (int c = threadIdx.x; c < (int)blockIdx.x; c += blockDim.x) before += chunk_sums[c];
    before = wave_inclusive_sum(before);
    if (lane_id() == kWave - 1) s_wave[threadIdx.x >> 6] = before;
    __syncthreads();
    if (threadIdx.x == 0) s_before = s_wave[0] + s_wave[1] + s_wave[2] + s_wave[3];
    __syncthreads();
    const long long base = (long long)blockIdx.x * kScanChunk + threadIdx.x * 8;
    int v[8];
    if (base + 8 <= n) {
        const int4 a = *reinterpret_cast<const int4 *>(counts + base), b = *reinterpret_cast<const int4 *>(counts + base + 4);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    } else {
        for (int j = 0; j < 8; ++j) v[j] = base + j < n ? counts[base + j] : 0;
    }
    int own = 0;
    for (int j = 0; j < 8; ++j) own += v[j];
    const int upto = wave_inclusive_sum(own);  // this thread's counters included
    __syncthreads();                           // s_wave is reused
    if (lane_id() == kWave - 1) s_wave[threadIdx.x >> 6] = upto;
    __syncthreads();
    int at = s_before + upto - own;
    for (int w = 0; w < (int)(threadIdx.x >> 6); ++w) at += s_wave[w];
    int out[8];
    for (int j = 0; j < 8; ++j) {
        out[j] = at;
        at += v[j];
    }
    if (base + 8 <= n) {
        *reinterpret_cast<int4 *>(boundaries + base) = make_int4(out[0], out[1], out[2], out[3]);
        *reinterpret_cast<int4 *>(boundaries + base + 4) = make_int4(out[4], out[5], out[6], out[7]);
    } else {
        for (int j = 0; j < 8; ++j)
            if (base + j < n) boundaries[base + j] = out[j];
    }
    if (bin_starts) {
        const int step = 1 << sub_shift;
        for (int j = 0; j < 8; ++j)
            if (base + j < n && ((base + j) & (step - 1)) == 0) bin_starts[(base + j) >> sub_shift] = out[j];
    }
}

int key_bits(int n_total_bins) {
    int bits = 1;
    while (bits < 31 && (1ll << bits) < (long long)n_total_bins) ++bits;
    return bits;
}

}  // namespace

int shift_and_bin(const float *d_coords, const uint32_t *d_min_bits, const uint32_t *d_max_bits_inverted,
                  const int *d_row_splits, int n_vert, int n_coords, int n_bin_dims, int n_rs, int n_bins_scalar,
                  int n_total_bins, float *d_shifted, float *d_bin_width, int *d_n_bins, int *d_assigned_bin,
                  int *d_flat_bin, hipStream_t s) {
    HGC_REQUIRE(n_coords >= 1 && n_coords <= 16 && n_bin_dims >= 1 && n_bin_dims <= kMaxBinDims &&
                    n_bin_dims <= n_coords,
                "bad coordinate or binning dimensions");
    if (n_vert <= 0) return HGC_OK;
    shift_and_bin_kernel<<<ceil_div(n_vert, 256), 256, 0, s>>>(d_coords, d_min_bits, d_max_bits_inverted, d_row_splits,
                                                               n_vert, n_coords, n_bin_dims, n_rs, n_bins_scalar,
                                                               n_total_bins, d_shifted, d_bin_width, d_n_bins,
                                                               d_assigned_bin, d_flat_bin, status_word());
    return check_launch("shift_and_bin");
}

int launch_fill_i32(int *p, int value, long long n, hipStream_t s) {
    if (n <= 0) return HGC_OK;
    int blocks = (int)std::min<long long>((n + 255) / 256, 4096);
    fill_i32_kernel<<<blocks, 256, 0, s>>>(p, value, n);
    return check_launch("fill_i32");
}


// few blocks fold the bounding box (every binning block reads all their partial
// results again), many assign the bins
static int grouping_blocks(int n_vert) { return std::max(1, std::min(128, ceil_div(n_vert, 1024))); }

bool bin_grouping_spatial(int n_bins_bound, int n_bin_dims) {
    return n_bin_dims >= 2 && n_bin_dims <= 4 && (((size_t)n_bins_bound << n_bin_dims) + 1) <= ((size_t)1 << 22);
}

int bin_grouping_sub_shift(int n_bins_bound, int n_bin_dims, bool spatial) {
    if (spatial && bin_grouping_spatial(n_bins_bound, n_bin_dims)) return n_bin_dims;
    int shift = 0;
    while (shift < 5 && (((size_t)n_bins_bound << (shift + 1)) + 1) <= ((size_t)1 << 20)) ++shift;
    return shift;
}

static size_t grouping_counters(int n_bins_bound, int n_bin_dims, bool spatial) {
    return ((size_t)n_bins_bound << bin_grouping_sub_shift(n_bins_bound, n_bin_dims, spatial)) + 1;
}

// scratch of the boundary table's scan: the chunk sums, or the library scan's own for tables of more
// than kMaxScanChunks chunks
static size_t scan_scratch_bytes(size_t n_counters) {
    const size_t n_chunks = (n_counters + kScanChunk - 1) / kScanChunk;
    if (n_chunks <= (size_t)kMaxScanChunks) return n_chunks * sizeof(int);
    size_t temp = 0;
    (void)rocprim::exclusive_scan(nullptr, temp, (const int *)nullptr, (int *)nullptr, 0, n_counters,
                                  rocprim::plus<int>(), (hipStream_t) nullptr);
    return temp;
}

size_t bin_grouping_workspace_bytes(int n_vert, int n_bins_bound, int n_bin_dims, bool spatial) {
    const size_t n = std::max(n_vert, 1);
    const size_t n_counters = grouping_counters(n_bins_bound, n_bin_dims, spatial);
    return align_up(scan_scratch_bytes(n_counters)) +
           align_up((size_t)grouping_blocks(n_vert) * 2 * kMaxBinDims * sizeof(float)) +
           align_up(n_counters * sizeof(int)) + 2 * align_up(n * sizeof(int)) +
           align_up(n * (kMaxBinDims + 1) * sizeof(int));
}

int bin_grouping(const float *d_coords, const int *d_row_splits, const int *d_direction, int n_vert, int n_coords,
                 int n_bin_dims, int n_rs, int n_bins_scalar, int n_bins_bound, float *d_shift, float *d_bin_width,
                 int *d_n_bins, int *d_boundaries, int *d_sorting, float *d_scoords, int *d_sflat, int *d_sbinass,
                 int *d_sdir, bool spatial, int *d_bin_starts, void *workspace, size_t workspace_bytes,
                 hipStream_t s) {
    spatial = spatial && bin_grouping_spatial(n_bins_bound, n_bin_dims);
    if (!workspace || !aligned256(workspace) ||
        workspace_bytes < bin_grouping_workspace_bytes(n_vert, n_bins_bound, n_bin_dims, spatial))
        return fail(HGC_ERR_WORKSPACE, "bin grouping workspace missing, misaligned or too small");
    const int blocks = grouping_blocks(n_vert);
    Carver carve(workspace);
    float *partial = carve.take<float>((size_t)blocks * 2 * kMaxBinDims);
    const int sub_shift = bin_grouping_sub_shift(n_bins_bound, n_bin_dims, spatial);
    const size_t n_counters = grouping_counters(n_bins_bound, n_bin_dims, spatial);
    int *counts = carve.take<int>(n_counters);
    int *flat = carve.take<int>(n_vert);
    int *rank = carve.take<int>(n_vert);
    int *binass = carve.take<int>((size_t)n_vert * (kMaxBinDims + 1));
    const int n_chunks = (int)ceil_div(n_counters, (size_t)kScanChunk);
    size_t scan_temp_bytes = scan_scratch_bytes(n_counters);
    int *chunk_sums = reinterpret_cast<int *>(carve.take<char>(scan_temp_bytes));
    column_minmax_kernel<<<blocks, 256, 0, s>>>(d_coords, n_coords, n_vert, n_bin_dims, partial, counts,
                                                (long long)n_counters);
    int rc = check_launch("column_minmax");
    if (rc) return rc;
    bin_points_ranked_kernel<<<std::min(4096, ceil_div(n_vert, 256)), 256, 0, s>>>(d_coords, n_coords, partial, blocks, d_row_splits, n_vert,
                                                    n_bin_dims, n_rs, n_bins_scalar, d_shift, d_bin_width, d_n_bins,
                                                    binass, flat, rank, counts, n_bins_bound, sub_shift,
                                                    spatial ? 1 : 0, status_word());
    rc = check_launch("bin_points_ranked");
    if (rc) return rc;
    // boundaries[b << sub_shift] = number of points in bins below b
    if (n_chunks <= kMaxScanChunks) {
        counter_chunk_sums_kernel<<<n_chunks, 256, 0, s>>>(counts, (long long)n_counters, chunk_sums);
        counter_scan_kernel<<<n_chunks, 256, 0, s>>>(counts, (long long)n_counters, chunk_sums, d_boundaries,
                                                     d_bin_starts, sub_shift);
        rc = check_launch("counter_scan");
    } else {  // every chunk adds up the sums in front of it: quadratic in the chunks, so huge tables take the library scan
        HGC_HIP(rocprim::exclusive_scan(chunk_sums, scan_temp_bytes, counts, d_boundaries, 0, n_counters,
                                        rocprim::plus<int>(), s));
        if (d_bin_starts) {
            strided_copy_kernel<<<ceil_div((long long)n_bins_bound + 1, 256), 256, 0, s>>>(d_boundaries, d_bin_starts,
                                                                                          n_bins_bound + 1, sub_shift);
        }
        rc = check_launch("bin boundary table");
    }
    if (rc) return rc;
    const int rows_aligned =
        ((reinterpret_cast<uintptr_t>(d_coords) | reinterpret_cast<uintptr_t>(d_scoords)) & 15u) == 0;
    move_to_bin_order_kernel<<<ceil_div(n_vert, 256), 256, 0, s>>>(d_coords, binass, flat, rank, d_direction,
                                                                   d_boundaries, n_vert, n_coords, n_bin_dims,
                                                                   sub_shift, spatial ? 1 : 0, rows_aligned, d_sorting,
                                                                   d_scoords, d_sflat, d_sbinass, d_sdir);
    return check_launch("move_to_bin_order");
}

}  // namespace hgc

using namespace hgc;

extern "C" {

int hgc_version(void) { return 101; }

int hgc_set_status_word(int *d_word) {
    hgc::g_status_word = d_word;
    return HGC_OK;
}

int *hgc_get_status_word(void) { return hgc::g_status_word; }

const char *hgc_last_error(void) { return hgc::last_error_buffer(); }

int hgc_bin_by_coordinates_total_bins(const int *h_n_bins, int n_nbins, int n_rs, int *h_out_total_bins) {
    HGC_REQUIRE(h_n_bins && h_out_total_bins, "null pointer");
    HGC_REQUIRE(n_nbins >= 1 && n_rs >= 1, "need at least one dimension and one row split entry");
    long long n = 1;
    for (int i = 0; i < n_nbins; ++i) {
        HGC_REQUIRE(h_n_bins[i] > 0, "n_bins[%d] = %d must be positive", i, h_n_bins[i]);
        n *= h_n_bins[i];
        HGC_REQUIRE(n < (1ll << 31), "bin count overflows int32");
    }
    n *= (n_rs - 1);
    HGC_REQUIRE(n < (1ll << 31), "bin count overflows int32");
    *h_out_total_bins = (int)n;
    return HGC_OK;
}

int hgc_bin_by_coordinates_strided(const float *d_coords, int coord_stride, const float *d_shift,
                                   const int *d_rs, const float *d_binswidth, const int *d_n_bins,
                                   int *d_assigned_bin, int *d_flat_assigned_bin, int *d_n_per_bin,
                                   int *d_n_out_of_range, int n_vert, int n_bin_dims, int n_rs,
                                   int n_total_bins, int calc_n_per_bin, hgc_stream_t stream) {
    HGC_REQUIRE(n_vert >= 0 && n_total_bins >= 0, "negative size");
    HGC_REQUIRE(n_bin_dims >= 1 && n_bin_dims <= kMaxBinDims, "1 <= binning dimensions <= %d", kMaxBinDims);
    HGC_REQUIRE(coord_stride >= n_bin_dims, "coordinate stride smaller than the binning dimensions");
    HGC_REQUIRE(n_rs >= 2, "BinByCoordinatesOp expects at least two row splits entries");
    HGC_REQUIRE(d_rs && d_binswidth && d_n_bins, "null pointer");
    hipStream_t s = as_stream(stream);
    if (d_n_per_bin) {
        int rc = launch_fill_i32(d_n_per_bin, 0, n_total_bins, s);
        if (rc) return rc;
    }
    if (n_vert == 0) return HGC_OK;
    HGC_REQUIRE(d_coords && d_assigned_bin && d_flat_assigned_bin, "null pointer");
    HGC_REQUIRE(!calc_n_per_bin || d_n_per_bin, "calc_n_per_bin needs d_n_per_bin");
    bin_points_kernel<<<ceil_div(n_vert, 256), 256, 0, s>>>(d_coords, coord_stride, d_shift, d_rs, d_binswidth,
                                                            d_n_bins, d_assigned_bin, d_flat_assigned_bin,
                                                            d_n_per_bin, d_n_out_of_range, status_word(), n_vert,
                                                            n_bin_dims, n_rs, n_total_bins, calc_n_per_bin);
    return check_launch("bin_points");
}

int hgc_bin_by_coordinates(const float *d_coords, const int *d_rs, const float *d_binswidth,
                           const int *d_n_bins, int *d_assigned_bin, int *d_flat_assigned_bin,
                           int *d_n_per_bin, int n_vert, int n_coords, int n_rs, int n_total_bins,
                           int calc_n_per_bin, hgc_stream_t stream) {
    return hgc_bin_by_coordinates_strided(d_coords, n_coords, nullptr, d_rs, d_binswidth, d_n_bins,
                                          d_assigned_bin, d_flat_assigned_bin, d_n_per_bin, nullptr, n_vert,
                                          n_coords, n_rs, n_total_bins, calc_n_per_bin, stream);
}

static int setup_blocks(int n_vert) { return std::max(1, std::min(1024, ceil_div(n_vert, 256 * 4))); }

size_t hgc_bin_setup_workspace_bytes(int n_vert, int n_bin_dims) {
    (void)n_bin_dims;
    return align_up((size_t)setup_blocks(n_vert) * 2 * kMaxBinDims * sizeof(float));
}

int hgc_bin_setup(const float *d_coords, int coord_stride, int n_vert, int n_bin_dims, int pre_normalized,
                  int n_bins_scalar, const float *d_bin_width_in, float *d_shift, float *d_bin_width,
                  int *d_n_bins, void *workspace, size_t workspace_bytes, hgc_stream_t stream) {
    HGC_REQUIRE(n_vert >= 1, "binning needs at least one point");
    HGC_REQUIRE(n_bin_dims >= 1 && n_bin_dims <= kMaxBinDims, "1 <= binning dimensions <= %d", kMaxBinDims);
    HGC_REQUIRE(coord_stride >= n_bin_dims, "coordinate stride smaller than the binning dimensions");
    HGC_REQUIRE(d_coords && d_shift && d_bin_width && d_n_bins, "null pointer");
    HGC_REQUIRE(n_bins_scalar > 0 || d_bin_width_in, "either n_bins or bin_width must be given");
    if (!workspace || !aligned256(workspace) ||
        workspace_bytes < hgc_bin_setup_workspace_bytes(n_vert, n_bin_dims))
        return fail(HGC_ERR_WORKSPACE, "bin_setup workspace missing, misaligned or too small");
    hipStream_t s = as_stream(stream);
    const int blocks = setup_blocks(n_vert);
    float *partial = static_cast<float *>(workspace);
    column_minmax_kernel<<<blocks, 256, 0, s>>>(d_coords, coord_stride, n_vert, n_bin_dims, partial, nullptr, 0);
    int rc = check_launch("column_minmax");
    if (rc) return rc;
    grid_params_kernel<<<1, 64, 0, s>>>(partial, blocks, n_bin_dims, pre_normalized, n_bins_scalar, d_bin_width_in,
                                        d_shift, d_bin_width, d_n_bins);
    return check_launch("grid_params");
}

static int hits_per_bin(int n_vert, int n_total_bins) { return std::max(1, n_vert / std::max(n_total_bins, 1)); }

size_t hgc_sort_by_bin_workspace_bytes(int n_vert, int n_total_bins) {
    size_t temp = 0;
    const int n = std::max(n_vert, 1);
    if (stable_key_sort_supported(n, std::max(n_total_bins, 1), hits_per_bin(n, n_total_bins)))
        return stable_key_sort_workspace_bytes(n, std::max(n_total_bins, 1), hits_per_bin(n, n_total_bins));
    (void)rocprim::radix_sort_pairs(nullptr, temp, (const unsigned int *)nullptr, (unsigned int *)nullptr,
                                    (const int *)nullptr, (int *)nullptr, (size_t)n, 0,
                                    key_bits(std::max(n_total_bins, 2)), (hipStream_t) nullptr);
    return align_up(temp) + 2 * align_up((size_t)n * sizeof(int));
}

int hgc_sort_by_bin(const int *d_flat_bin, int n_vert, int n_total_bins, int *d_sorting,
                    int *d_bin_boundaries, void *workspace, size_t workspace_bytes, hgc_stream_t stream) {
    HGC_REQUIRE(n_vert >= 0 && n_total_bins >= 1, "bad sizes");
    HGC_REQUIRE(d_bin_boundaries, "null pointer");
    hipStream_t s = as_stream(stream);
    if (n_vert == 0) return launch_fill_i32(d_bin_boundaries, 0, (long long)n_total_bins + 1, s);
    HGC_REQUIRE(d_flat_bin && d_sorting, "null pointer");
    if (!workspace || !aligned256(workspace) ||
        workspace_bytes < hgc_sort_by_bin_workspace_bytes(n_vert, n_total_bins))
        return fail(HGC_ERR_WORKSPACE, "sort_by_bin workspace missing, misaligned or too small");
    // a stable counting sort by bin yields the order and the boundary table at once
    if (stable_key_sort_supported(n_vert, n_total_bins, hits_per_bin(n_vert, n_total_bins)))
        return stable_key_sort(d_flat_bin, nullptr, n_vert, n_total_bins, hits_per_bin(n_vert, n_total_bins),
                               d_bin_boundaries, d_sorting, workspace, workspace_bytes, s);
    Carver carve(workspace);
    int *iota = carve.take<int>(n_vert);
    unsigned int *keys_out = carve.take<unsigned int>(n_vert);
    void *temp = carve.base + carve.used;
    size_t temp_bytes = workspace_bytes - carve.used;
    iota_i32_kernel<<<ceil_div(n_vert, 256), 256, 0, s>>>(iota, n_vert);
    int rc = check_launch("iota");
    if (rc) return rc;
    // LSD radix sort: stable, so equal bins keep ascending original index
    HGC_HIP(rocprim::radix_sort_pairs(temp, temp_bytes, reinterpret_cast<const unsigned int *>(d_flat_bin),
                                      keys_out, iota, d_sorting, (size_t)n_vert, 0, key_bits(n_total_bins), s));
    bin_boundaries_kernel<<<ceil_div((long long)n_total_bins + 1, 256), 256, 0, s>>>(
        reinterpret_cast<const int *>(keys_out), n_vert, d_bin_boundaries, n_total_bins);
    return check_launch("bin_boundaries");
}

int hgc_gather_rows(const void *d_in, const int *d_rows, void *d_out, int n_rows, int width,
                    hgc_stream_t stream) {
    HGC_REQUIRE(n_rows >= 0 && width >= 1, "bad sizes");
    if (n_rows == 0) return HGC_OK;
    HGC_REQUIRE(d_in && d_rows && d_out, "null pointer");
    hipStream_t s = as_stream(stream);
    const long long total = (long long)n_rows * width;
    const int blocks = ceil_div(total, 256);
    const uint32_t *in = static_cast<const uint32_t *>(d_in);
    uint32_t *out = static_cast<uint32_t *>(d_out);
    switch (width) {
        case 1: gather_rows_kernel<1><<<blocks, 256, 0, s>>>(in, d_rows, out, n_rows, width); break;
        case 2: gather_rows_kernel<2><<<blocks, 256, 0, s>>>(in, d_rows, out, n_rows, width); break;
        case 3: gather_rows_kernel<3><<<blocks, 256, 0, s>>>(in, d_rows, out, n_rows, width); break;
        case 4: gather_rows_kernel<4><<<blocks, 256, 0, s>>>(in, d_rows, out, n_rows, width); break;
        default: gather_rows_kernel<0><<<blocks, 256, 0, s>>>(in, d_rows, out, n_rows, width); break;
    }
    return check_launch("gather_rows");
}

int hgc_index_replacer(const int *d_to_be_replaced, const int *d_replacements, int *d_replaced,
                       int n_to_be_replaced, int n_replacements, hgc_stream_t stream) {
    HGC_REQUIRE(n_to_be_replaced >= 0 && n_replacements >= 0, "negative size");
    if (n_to_be_replaced == 0) return HGC_OK;
    HGC_REQUIRE(d_to_be_replaced && d_replaced && (d_replacements || n_replacements == 0), "null pointer");
    index_replacer_kernel<<<ceil_div(n_to_be_replaced, 256), 256, 0, as_stream(stream)>>>(
        d_to_be_replaced, d_replacements, d_replaced, status_word(), n_to_be_replaced, n_replacements);
    return check_launch("index_replacer");
}

}  // extern "C"
