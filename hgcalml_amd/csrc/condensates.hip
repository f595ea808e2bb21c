// Object-condensation condensate assignment: greedy highest-beta-first
// selection of condensation points with radius claims, per event.
//
// Reference behaviour restated here:
//   modules/compiled/binned_assign_to_condensates_kernel.cc:23-125  (claim step)
//   modules/compiled/binned_assign_to_condensates_kernel.cc:128-241 (greedy loop)
//   modules/compiled/binstepper.h:100-165                           (box of bins)
//
// The reference picks, again and again, the unclaimed high-beta hit with the
// largest beta (first one in bin order on ties) by a linear scan, and lets it
// claim the hits of its box of bins that lie inside its sphere. Two facts turn
// that chain of claim steps into wide kernels:
//   * the order of the picks is static: the high-beta hits of every event are
//     sorted once by (event, beta descending, position ascending);
//   * a high-beta hit becomes a condensation point exactly if no condensation
//     point EARLIER in that order covers it, in both assignment modes (the
//     first condensation point that covers a hit always claims it), and only
//     a few hundred of tens of thousands do.
// So the condensation points are found first, from the sorted candidates alone:
// one workgroup per event walks the list in windows, one candidate per thread;
// a window is resolved wave after wave (inside a wave: the first open lane is
// a condensation point, the lanes it covers close), every later wave dropping
// what the new points cover. Between a few launches of that kernel, whose
// share of the list grows geometrically, a grid-wide kernel drops every
// remaining candidate that the points found so far cover, so that the event's
// workgroup only ever tests its candidates against the points of its own launch
// (kept in LDS). Finally every hit looks for the points of its event that cover
// it, in selection order: the first one (max-beta mode) or the reference's
// running comparison over all of them (min-distance mode).
//
// "Covers" is the reference's claim test: inside the sphere (serial fp32 over
// the coordinates, no FMA contraction), the hit's bin inside the point's box
// of bins (floor((c-r)/bw) .. ceil((c+r)/bw) per binned dimension), mask rules
// as in the reference. The reference checks only the flat index of a box cell,
// so a box that sticks out of the grid also walks cells of the neighbouring
// row; their hits lie outside the sphere, which makes the per-dimension test
// here equivalent. Only comparisons and order-independent writes are involved,
// so the result is the reference's bit for bit.
#include "hgc_common.hpp"

#include <climits>
#include <cstring>
#include <algorithm>

#include <rocprim/rocprim.hpp>

namespace hgc {

int launch_fill_i32(int *p, int value, long long n, hipStream_t s);

namespace {

constexpr int kMaxDims = 16;     // coordinate dimensions
constexpr int kMaxBinDims = 6;   // binned dimensions
constexpr int kBlock = 1024;     // threads of an event's workgroup
constexpr int kWavesPerBlock = kBlock / kWave;
constexpr int kFill = 4;         // windows of the sorted list looked at per refill of the queue
constexpr int kQueueCap = kBlock + kFill * kBlock;
constexpr int kScanBlock = 256;  // threads of the grid-wide kernels
constexpr int kTile = 256;       // condensation points staged in LDS at a time there (one per thread)
constexpr int kMaxLaunches = 3;  // launches of the event kernel (cfg5-like input: 0.47 ms with 3, 0.48 with 4, 0.55 with 2)

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
    int rows_aligned;  // ccoords and ccoords_h start on 16-byte boundaries
    // The *_h arrays may be the arrays of all hits themselves (n_vert_h == n_vert, identity
    // indices) instead of a filtered copy: then `high` [n_vert] says which hits belong to the
    // high-beta subset, and `quirk` = {index of the first of them, its no_condensation_mask,
    // that of the second one} stands for the first two entries of the filtered mask.
    const int *high;
    const int *quirk;
    // workspace
    const int *order_h;  // high-beta hits in selection order, grouped by event
    int *pos_h;          // [n_vert_h] position of a high-beta hit among all hits, -1 unknown
    int *hit_bin;        // [n_vert] bin of a hit inside its event's grid, INT_MIN unknown
    uint32_t *cand;      // [n_vert_h] candidate records in selection order
    unsigned long long *open_bits;  // one bit per selection position, 64 positions a word: still a
                                    // candidate (it can be picked at all, and no point found so far covers it)
    uint32_t *points;    // [n_vert_h] an event's condensation points in selection order, from
                         // row_splits_h[event] on
    int *walk_end;       // [num_rows] end of the event's candidates that can be picked at all
    int *cursor_at;      // [kMaxLaunches][num_rows] selection position an event's walk stopped at
    int *n_alpha_at;     // [kMaxLaunches][num_rows] points of the event after that launch
};

// A candidate record (CMAX = coordinate slots, unused ones hold 0 and add an
// exact 0 to every distance):
//   [0, CMAX)          coordinates of its hit
//   [CMAX, CMAX+6)     per-dimension bins of its hit, saturated to 16 bits (-32768: unknown)
//   CMAX+6             1: its hit is masked (or unknown), no sphere claims it
//   CMAX+7             unused
//   [CMAX+8, ...)      the condensation point it would be:
//     [0, CMAX) centre, CMAX radius^2, CMAX+1 q | solitary << 31, CMAX+2 original index,
//     CMAX+3 unused, [CMAX+4, CMAX+10) box of bins per dimension, lo | hi << 16 (saturated to 16
//     bits; dimensions that are not binned hold the full range); padded to 16 bytes
// The box test is exact up to 16383 bins per dimension (the sphere test is what decides beyond
// fp32 rounding at a bin boundary).
__host__ __device__ constexpr int alpha_words(int cmax) { return (cmax + 4 + kMaxBinDims + 3) / 4 * 4; }
__host__ __device__ constexpr int cand_words(int cmax) { return cmax + 8 + alpha_words(cmax); }

__device__ __forceinline__ int saturate16(int v) { return max(-32768, min(32767, v)); }

// the reference indexes the high-beta mask with the truth value of (q > 0)
__device__ __forceinline__ bool always_first(const CondParams &p, int q) {
    if (p.high) return (q == p.quirk[0] ? p.quirk[1] : p.quirk[2]) != 0;
    const int slot = q > 0 ? 1 : 0;
    return slot < p.n_vert_h && p.mask_h[slot] != 0;
}

// 0: picked as soon as it is the first unclaimed one, in position order; 1: picked by beta;
// 2: never picked
__device__ __forceinline__ int selection_class(const CondParams &p, int q) {
    if (p.high && !p.high[q]) return 2;
    if (always_first(p, q)) return 0;
    return p.beta_h[q] > -1.f ? 1 : 2;  // beta <= -1 (or NaN) is never picked
}

// r with splits[r] <= i < splits[r+1]
__device__ __forceinline__ int event_of(const int *__restrict__ splits, int num_rows, int i) {
    int lo = 1, hi = num_rows + 1;
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (splits[mid] > i)
            hi = mid;
        else
            lo = mid + 1;
    }
    return min(lo - 1, num_rows - 1);
}

// ascending sort key == selection order; clears the per-candidate outputs
// position_bits > 0: the position goes into the key's low bits (all keys differ, the sort need not be stable)
__global__ __launch_bounds__(256) void selection_keys_kernel(const CondParams p, uint64_t *__restrict__ keys,
                                                             int *__restrict__ values, int position_bits) {
    const int q = blockIdx.x * blockDim.x + threadIdx.x;
    if (q >= p.n_vert_h) return;
    const uint64_t ev = (uint64_t)event_of(p.row_splits_h, p.num_rows, q);
    const uint64_t cls = (uint64_t)selection_class(p, q);
    uint64_t low = 0;
    if (cls == 1) {
        uint32_t u = __float_as_uint(p.beta_h[q]);
        u = (u & 0x80000000u) ? ~u : (u | 0x80000000u);  // monotone map float -> uint
        low = (uint32_t)~u;                               // larger beta first
    }
    const uint64_t key = (ev << 34) | (cls << 32) | low;
    keys[q] = position_bits ? ((key << position_bits) | (uint64_t)q) : key;
    values[q] = q;
    p.is_alpha_h[q] = 0;
    p.taken_h[q] = 0;
    p.alpha_indices[q] = -1;
    if (!p.high) p.pos_h[q] = -1;
}

// bin of every hit inside its event's grid (from the bin boundaries), and the
// position of every high-beta hit among all hits
__global__ __launch_bounds__(256) void hit_prepare_kernel(const CondParams p) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < p.num_rows) p.walk_end[i] = p.row_splits_h[i + 1];  // unless candidate_records_kernel finds less
    if (i >= p.n_vert) return;
    const int r = event_of(p.row_splits, p.num_rows, i);
    int cells = 1;
    for (int d = 0; d < p.B; ++d) cells *= p.n_bins[d];
    const int *splits = p.bin_splits + (size_t)cells * r;
    int lo = 0, hi = cells;  // last bin whose first hit is <= i
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (splits[mid] <= i)
            lo = mid;
        else
            hi = mid;
    }
    p.hit_bin[i] = (cells > 0 && splits[lo] <= i && i < splits[lo + 1]) ? lo : INT_MIN;
    const int q = p.to_filtered[i];
    if (!p.high && q >= 0 && q < p.n_vert_h) p.pos_h[q] = i;
}

struct Grid {
    int nb[kMaxBinDims];
    float bw;
    __device__ __forceinline__ void load(const CondParams &p) {
#pragma unroll
        for (int d = 0; d < kMaxBinDims; ++d) nb[d] = d < p.B ? p.n_bins[d] : 1;
        bw = p.bin_widths[0];
    }
    // per-dimension bin indices of a bin of the event's grid, as the box test wants them
    __device__ __forceinline__ void split(int bin, int B, int (&k)[kMaxBinDims]) const {
        const bool known = bin != INT_MIN;
#pragma unroll
        for (int d = kMaxBinDims - 1; d >= 0; --d) {
            k[d] = d < B ? -32768 : 0;
            if (d < B && known) {
                k[d] = saturate16(bin % nb[d]);
                bin /= nb[d];
            }
        }
    }
};

// everything a candidate needs, gathered into selection order
template <int CMAX>
__global__ __launch_bounds__(256) void candidate_records_kernel(const CondParams p) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    const bool in_range = i < p.n_vert_h;
    const int q = in_range ? p.order_h[i] : 0;
    const bool selectable = in_range && selection_class(p, q) < 2;
    const uint64_t open = __ballot(selectable);  // a wave holds 64 consecutive positions of one word
    if ((threadIdx.x & (kWave - 1)) == 0 && in_range) p.open_bits[i >> 6] = open;
    if (!in_range) return;
    constexpr int cw = cand_words(CMAX);
    const int C = p.C, B = p.B;
    Grid g;
    g.load(p);
    if (!selectable) {
        // those that are never picked come last in an event's order: the walk ends at the first one
        const int ev = event_of(p.row_splits_h, p.num_rows, i);
        if (i == p.row_splits_h[ev] || selection_class(p, p.order_h[i - 1]) < 2) p.walk_end[ev] = i;
        return;  // nobody reads its record
    }
    const int at = p.high ? q : p.pos_h[q];  // hits as their own high-beta subset: same index
    uint32_t rec[cw];
    uint32_t *point = rec + CMAX + 8;
    float centre[CMAX];
    if (CMAX == 4 && C == 4 && p.rows_aligned) {  // one 16-byte load per row
        const float4 h = at >= 0 ? reinterpret_cast<const float4 *>(p.ccoords)[at] : float4{0.f, 0.f, 0.f, 0.f};
        const float4 a = reinterpret_cast<const float4 *>(p.ccoords_h)[q];
        rec[0] = __float_as_uint(h.x), rec[1] = __float_as_uint(h.y), rec[2] = __float_as_uint(h.z),
        rec[3] = __float_as_uint(h.w);
        centre[0] = a.x, centre[1] = a.y, centre[2] = a.z, centre[3] = a.w;
    } else {
#pragma unroll
        for (int c = 0; c < CMAX; ++c) {
            centre[c] = c < C ? p.ccoords_h[(size_t)q * C + c] : 0.f;
            rec[c] = (c < C && at >= 0) ? __float_as_uint(p.ccoords[(size_t)at * C + c]) : 0u;
        }
    }
#pragma unroll
    for (int c = 0; c < CMAX; ++c) point[c] = __float_as_uint(centre[c]);
    int k[kMaxBinDims];
    g.split(at >= 0 ? p.hit_bin[at] : INT_MIN, B, k);
#pragma unroll
    for (int d = 0; d < kMaxBinDims; ++d) rec[CMAX + d] = (uint32_t)k[d];
    rec[CMAX + 6] = (at < 0 || p.mask[at] != 0) ? 1u : 0u;
    rec[CMAX + 7] = 0u;
    float radius = p.dist_h[q];
    const bool solitary = p.mask_h[q] > 0;
    point[CMAX] = __float_as_uint(radius * radius);
    point[CMAX + 1] = (uint32_t)q | (solitary ? 0x80000000u : 0u);
    point[CMAX + 2] = (uint32_t)p.orig_h[q];
    point[CMAX + 3] = 0u;
    if (solitary) radius = 0.f;
#pragma unroll
    for (int d = 0; d < kMaxBinDims; ++d) {
        int lo = -32768, hi = 32767;
        if (d < B) {
            float fl = floorf((centre[d] - radius) / g.bw), fh = ceilf((centre[d] + radius) / g.bw);
            // keep the box finite for absurd radii; the clamped range still covers
            // every bin of the grid in this dimension
            fl = fminf(fmaxf(fl, (float)(-g.nb[d])), (float)(2 * g.nb[d]));
            fh = fminf(fmaxf(fh, (float)(-g.nb[d])), (float)(2 * g.nb[d]));
            lo = saturate16((int)fl);
            hi = saturate16((int)fh);
        }
        point[CMAX + 4 + d] = ((uint32_t)lo & 0xffffu) | ((uint32_t)hi << 16);
    }
#pragma unroll
    for (int w = CMAX + 4 + kMaxBinDims; w < alpha_words(CMAX); ++w) point[w] = 0u;
    uint4 *out = reinterpret_cast<uint4 *>(p.cand + (size_t)i * cw);
#pragma unroll
    for (int w = 0; w < cw; w += 4) out[w / 4] = uint4{rec[w], rec[w + 1], rec[w + 2], rec[w + 3]};
}

// The reference's claim test of one hit against one condensation point, in two
// parts: sphere and mask rules on the first CMAX+2 words of the point ...
template <int CMAX>
__device__ __forceinline__ bool in_sphere(const uint32_t (&a)[CMAX + 2], const float (&x)[CMAX], bool uncoverable,
                                          int self_q, float &dsq) {
    float acc = 0.f;
#pragma unroll
    for (int c = 0; c < CMAX; ++c) {
        const float t = __uint_as_float(a[c]) - x[c];
        acc = acc + t * t;
    }
    dsq = acc;
    if (a[CMAX + 1] >> 31) return self_q == (int)(a[CMAX + 1] & 0x7fffffffu);
    return !uncoverable && acc <= __uint_as_float(a[CMAX]);
}

// ... and the hit's bin against the point's box of bins
__device__ __forceinline__ bool in_box(const uint32_t (&box)[kMaxBinDims], const int (&k)[kMaxBinDims]) {
    int inside = 1;  // no short cuts: twelve compares cost less than a chain of branches
#pragma unroll
    for (int d = 0; d < kMaxBinDims; ++d)
        inside &= (int)(k[d] >= (int)(int16_t)(box[d] & 0xffffu)) & (int)(k[d] <= ((int)box[d] >> 16));
    return inside != 0;
}

// the whole test against a point in LDS (16-byte aligned); the box is only read for hits inside the sphere
template <int CMAX>
__device__ __forceinline__ bool covers(const uint32_t *a, const float (&x)[CMAX], bool uncoverable, int self_q,
                                       const int (&k)[kMaxBinDims], float &dsq) {
    uint32_t head[CMAX + 2];
#pragma unroll
    for (int c4 = 0; c4 < CMAX; c4 += 4) {
        const uint4 v = *reinterpret_cast<const uint4 *>(a + c4);
        head[c4] = v.x, head[c4 + 1] = v.y, head[c4 + 2] = v.z, head[c4 + 3] = v.w;
    }
    const uint2 rs = *reinterpret_cast<const uint2 *>(a + CMAX);
    head[CMAX] = rs.x, head[CMAX + 1] = rs.y;
    if (!in_sphere<CMAX>(head, x, uncoverable, self_q, dsq)) return false;
    const uint4 b0 = *reinterpret_cast<const uint4 *>(a + CMAX + 4);
    const uint2 b1 = *reinterpret_cast<const uint2 *>(a + CMAX + 8);
    const uint32_t box[kMaxBinDims] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y};
    return in_box(box, k);
}

__device__ __forceinline__ unsigned long long coherent_load(const unsigned long long *ptr) {
    return __hip_atomic_load(ptr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The event kernel's list of condensation points in LDS, by component: word w of
// point s sits at list[w * capacity + s] (capacity a multiple of 4, the list on a
// 16-byte boundary), so that four points are tested at a time. Word CMAX, the
// squared radius, holds -1 for a point that claims only its own hit (its radius
// sits in word CMAX + 3), so that it never passes the sphere test. True if one of
// the points [lo & ~3, hi) covers the candidate (never by the self rule; xs is the
// candidate's position). Points before lo in the first group are tested again: the
// candidate has been through them, none covers it. Slots from hi on are never
// looked at: another wave may be writing them.
template <int CMAX>
__device__ __forceinline__ bool covered_by_list(const uint32_t *list, int capacity, int lo, int hi,
                                                const float (&xs)[CMAX], const int (&k)[kMaxBinDims]) {
    for (int s4 = lo & ~3; s4 < hi; s4 += 4) {
        float d0 = 0.f, d1 = 0.f, d2 = 0.f, d3 = 0.f;
#pragma unroll
        for (int c = 0; c < CMAX; ++c) {
            const float4 cc = *reinterpret_cast<const float4 *>(list + (size_t)c * capacity + s4);
            float t = cc.x - xs[c];
            d0 = d0 + t * t;
            t = cc.y - xs[c];
            d1 = d1 + t * t;
            t = cc.z - xs[c];
            d2 = d2 + t * t;
            t = cc.w - xs[c];
            d3 = d3 + t * t;
        }
        float4 rr = *reinterpret_cast<const float4 *>(list + (size_t)CMAX * capacity + s4);
        if (s4 + 4 > hi) {  // slots behind the range may be in the middle of being written
            // Invariant: nothing read from a slot >= hi may reach `hits`. The distances d0..d3 of such
            // slots are sums of squares of whatever the slot held -- non-negative, infinite or NaN --
            // and their radius is forced to -1 here, so `d <= rr` is false for every one of them;
            // the box words of a slot are only read for a set bit of `hits`.
            const int real = hi - s4;
            rr.w = -1.f;
            if (real < 3) rr.z = -1.f;
            if (real < 2) rr.y = -1.f;
        }
        if (!((d0 <= rr.x) | (d1 <= rr.y) | (d2 <= rr.z) | (d3 <= rr.w))) continue;
        uint32_t hits = (d0 <= rr.x ? 1u : 0u) | (d1 <= rr.y ? 2u : 0u) | (d2 <= rr.z ? 4u : 0u) | (d3 <= rr.w ? 8u : 0u);
        while (hits) {
            const int s = s4 + __builtin_ctz(hits);
            hits &= hits - 1u;
            uint32_t box[kMaxBinDims];
#pragma unroll
            for (int d = 0; d < kMaxBinDims; ++d) box[d] = list[(size_t)(CMAX + 4 + d) * capacity + s];
            if (in_box(box, k)) return true;
        }
    }
    return false;
}

// Finds the condensation points among the next `budget` candidates (all that are
// left: budget < 0) of one event per workgroup. The walk over the sorted list
// collects the candidates that are still open in a queue; `window` of them are
// resolved at a time, one per thread; `capacity` points of this launch fit into
// the LDS list.
template <int CMAX>
__global__ __launch_bounds__(kBlock) void condensate_event_kernel(const CondParams p, int launch, int budget,
                                                                  int window, int capacity) {
    extern __shared__ __align__(16) uint32_t s_list[];
    __shared__ int s_queue[kQueueCap];
    __shared__ int s_fill[kFill][kWavesPerBlock];
    __shared__ int s_open[kWavesPerBlock], s_cnt[kWavesPerBlock];
    constexpr int aw = alpha_words(CMAX), cw = cand_words(CMAX);

    const int r = blockIdx.x;
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid >> 6;
    const int first_h = p.row_splits_h[r], last_h = p.walk_end[r];

    int cur = launch == 0 ? first_h : p.cursor_at[(launch - 1) * p.num_rows + r];
    int n_alpha = launch == 0 ? 0 : p.n_alpha_at[(launch - 1) * p.num_rows + r];
    const int end = budget < 0 ? last_h : (int)min((long long)last_h, (long long)cur + budget);
    int n_list = 0;  // points of this launch, all in s_list
    // The points go to global memory (for the grid-wide kernels) when the list is given
    // up, not as they are found: a store in a stage would be waited for at its barrier.
    auto flush_list = [&]() {
        const int rank0 = n_alpha - n_list;
        for (int i = tid; i < n_list; i += kBlock) {
            uint32_t word[aw];
#pragma unroll
            for (int t = 0; t < aw; ++t) word[t] = s_list[(size_t)t * capacity + i];
            if (word[CMAX + 1] >> 31) word[CMAX] = word[CMAX + 3], word[CMAX + 3] = 0u;
            uint32_t *out = p.points + (size_t)(first_h + rank0 + i) * aw;
#pragma unroll
            for (int t = 0; t < aw; t += 4)
                *reinterpret_cast<uint4 *>(out + t) = uint4{word[t], word[t + 1], word[t + 2], word[t + 3]};
            const int q = (int)(word[CMAX + 1] & 0x7fffffffu);
            p.alpha_indices[first_h + rank0 + i] = (int)word[CMAX + 2];
            p.is_alpha_h[q] = 1;
            p.taken_h[q] = 1;
        }
    };
    int n_queue = 0;
    int stopped_at = -1;

    for (;;) {
        // ---- refill the queue with the open candidates of the next windows, in order ----
        // One word of 64 positions per thread. If the open ones of all 1024 words fit
        // into the queue they are all taken (the rule once most candidates are covered),
        // else as many words as fit whatever they hold.
        while (n_queue < window && cur < end) {
            const int word0 = cur >> 6;
            const long long base = ((long long)word0 + tid) << 6;
            unsigned long long bits = base < end ? coherent_load(p.open_bits + word0 + tid) : 0ull;
            if (tid == 0) bits &= ~0ull << (cur & 63);
            if (base + 64 > end) bits = end > base ? bits & ((1ull << (end - base)) - 1ull) : 0ull;
            const int mine = __popcll(bits);
            const int upto = wave_inclusive_sum(mine);
            if (lane == kWave - 1) s_fill[0][wave] = upto;
            __syncthreads();
            int before = upto - mine, total = 0;
#pragma unroll
            for (int w = 0; w < kWavesPerBlock; ++w) {
                if (w < wave) before += s_fill[0][w];
                total += s_fill[0][w];
            }
            const int room = kQueueCap - n_queue;
            int words = kBlock, taken = total;
            if (total > room) {
                words = room >> 6;
                if (tid == words) s_fill[1][0] = before;
                __syncthreads();
                taken = s_fill[1][0];
            }
            if (tid < words) {
                int at = n_queue + before;
                while (bits) {
                    s_queue[at++] = (int)base + __builtin_ctzll(bits);
                    bits &= bits - 1ull;
                }
            }
            n_queue += taken;
            cur = (int)min((long long)end, ((long long)word0 + words) << 6);
            __syncthreads();
        }
        if (n_queue == 0) break;
        const int take = min(n_queue, window);
        if (n_list + take > capacity) {
            // the list may not hold what this window adds
            const int front = s_queue[0];
            if (budget >= 0) {  // the grid-wide kernel after this launch takes the list over
                stopped_at = front;
                break;
            }
            // last launch: this workgroup closes what the list covers among the rest of
            // its candidates itself, then starts a new list and walks on from the
            // front of the queue
            __syncthreads();
            for (int i = front + tid; i < last_h; i += kBlock) {
                if (!((coherent_load(p.open_bits + (i >> 6)) >> (i & 63)) & 1ull)) continue;
                const uint32_t *ri = p.cand + (size_t)i * cw;
                if (ri[CMAX + 6]) continue;
                float xi[CMAX];
                int ki[kMaxBinDims];
#pragma unroll
                for (int c = 0; c < CMAX; ++c) xi[c] = __uint_as_float(ri[c]);
#pragma unroll
                for (int d = 0; d < kMaxBinDims; ++d) ki[d] = (int)ri[CMAX + d];
                if (covered_by_list<CMAX>(s_list, capacity, 0, n_list, xi, ki))
                    atomicAnd(p.open_bits + (i >> 6), ~(1ull << (i & 63)));
            }
            flush_list();
            __threadfence();
            __syncthreads();
            n_list = 0;
            n_queue = 0;
            cur = front;
            continue;
        }

        // ---- this thread's candidate ----
        const bool valid = tid < take;
        const int pos = valid ? s_queue[tid] : first_h;
        float x[CMAX];
        int k[kMaxBinDims];
        uint32_t point[aw];
        bool uncoverable = false;
        {
            const uint32_t *rec = p.cand + (size_t)pos * cw;
#pragma unroll
            for (int c4 = 0; c4 < CMAX; c4 += 4) {
                const float4 v = valid ? *reinterpret_cast<const float4 *>(rec + c4) : float4{0.f, 0.f, 0.f, 0.f};
                x[c4] = v.x, x[c4 + 1] = v.y, x[c4 + 2] = v.z, x[c4 + 3] = v.w;
            }
#pragma unroll
            for (int d = 0; d < kMaxBinDims; ++d) k[d] = valid ? (int)rec[CMAX + d] : INT_MIN;
            uncoverable = valid && rec[CMAX + 6] != 0;
#pragma unroll
            for (int w4 = 0; w4 < aw; w4 += 4) {
                const uint4 v = valid ? *reinterpret_cast<const uint4 *>(rec + CMAX + 8 + w4) : uint4{0u, 0u, 0u, 0u};
                point[w4] = v.x, point[w4 + 1] = v.y, point[w4 + 2] = v.z, point[w4 + 3] = v.w;
            }
        }
        bool open = valid;

        // ---- points found earlier in this launch ----
        if (open && !uncoverable && covered_by_list<CMAX>(s_list, capacity, 0, n_list, x, k)) open = false;
        const uint64_t wave_open = __ballot(open);
        if (lane == 0) {
            s_open[wave] = wave_open != 0;
            s_cnt[wave] = 0;
        }
        __syncthreads();

        // ---- the window, wave after wave ----
        // Stage w: wave w picks its condensation points one after the other (the first
        // open lane is one, the lanes it covers close) and adds them to the list. The
        // waves behind it test their candidates against the points of the stage before
        // while it does so; wave w itself has done that first.
        const int n_waves = (take + kWave - 1) / kWave;
        const uint64_t coverable_lanes = __ballot(!uncoverable);
        int tested = n_list;  // the waves still waiting for their stage have seen the list up to here
        for (int w = 0; w < n_waves; ++w) {
            if (!s_open[w]) continue;  // uniform
            if (wave == w) __builtin_amdgcn_s_setprio(3);  // the others wait for this wave
            if (wave >= w && open && !uncoverable && covered_by_list<CMAX>(s_list, capacity, tested, n_list, x, k))
                open = false;
            if (wave == w) {
                uint64_t open_lanes = __ballot(open), chosen_lanes = 0;
                while (open_lanes) {
                    const int first = __builtin_ctzll(open_lanes);  // the next condensation point
                    open_lanes &= open_lanes - 1ull;
                    chosen_lanes |= 1ull << first;
                    // the other lanes get the point from that lane's registers
                    uint32_t head[CMAX + 2];
#pragma unroll
                    for (int t = 0; t < CMAX + 2; ++t) head[t] = (uint32_t)__builtin_amdgcn_readlane((int)point[t], first);
                    if (head[CMAX + 1] >> 31) continue;  // claims only its own hit
                    float acc = 0.f;  // every lane, whatever its state: the masks below are scalars
#pragma unroll
                    for (int c = 0; c < CMAX; ++c) {
                        const float t = __uint_as_float(head[c]) - x[c];
                        acc = acc + t * t;
                    }
                    uint64_t inside = __ballot(acc <= __uint_as_float(head[CMAX])) & open_lanes & coverable_lanes;
                    if (inside) {  // the box only matters for lanes inside the sphere
                        uint32_t box[kMaxBinDims];
#pragma unroll
                        for (int d = 0; d < kMaxBinDims; ++d)
                            box[d] = (uint32_t)__builtin_amdgcn_readlane((int)point[CMAX + 4 + d], first);
                        inside &= __ballot(in_box(box, k));
                        open_lanes &= ~inside;
                    }
                }
                open = false;  // every lane of the wave is a condensation point now, or covered by one
                if ((chosen_lanes >> lane) & 1ull) {
                    // for the waves behind
                    const int nth = __popcll(chosen_lanes & ((1ull << lane) - 1ull));
                    const bool solitary = point[CMAX + 1] >> 31;
#pragma unroll
                    for (int t = 0; t < aw; ++t) {
                        uint32_t word = point[t];
                        if (t == CMAX && solitary) word = __float_as_uint(-1.f);
                        if (t == CMAX + 3 && solitary) word = point[CMAX];
                        s_list[(size_t)t * capacity + n_list + nth] = word;
                    }
                }
                if (lane == 0) s_cnt[w] = __popcll(chosen_lanes);
                __builtin_amdgcn_s_setprio(0);
            }
            __syncthreads();
            const int added = s_cnt[w];
            tested = n_list;
            n_list += added;
            n_alpha += added;
        }

        // ---- the rest of the queue moves to its front ----
        const int rest = n_queue - take;
        int moved[kFill];
#pragma unroll
        for (int j = 0; j < kFill; ++j) moved[j] = j * kBlock + tid < rest ? s_queue[take + j * kBlock + tid] : 0;
        __syncthreads();
#pragma unroll
        for (int j = 0; j < kFill; ++j)
            if (j * kBlock + tid < rest) s_queue[j * kBlock + tid] = moved[j];
        n_queue = rest;
        __syncthreads();
    }
    flush_list();
    if (tid == 0) {
        p.cursor_at[launch * p.num_rows + r] = stopped_at >= 0 ? stopped_at : end;
        p.n_alpha_at[launch * p.num_rows + r] = n_alpha;
    }
}

// Grid-wide pass over items of all events against the condensation points of
// their event, a tile of points in LDS at a time.
//   MODE 0: items = candidates from the event's cursor on, points = those the last
//           launch of the event kernel added; closes what they cover
//   MODE 1: items = all hits, all points; first point that covers the hit (max-beta)
//   MODE 2: items = all hits, all points; the reference's running comparison (min-distance)
// The hits come in bin order, so the 256 of a workgroup share a narrow range of bins in the
// leading binned dimensions: only the points whose box of bins meets that range go into the
// tile (a point outside it covers none of these hits, whatever its sphere), in their order.
template <int CMAX, int MODE>
__global__ __launch_bounds__(kScanBlock) void cover_scan_kernel(const CondParams p, int launch) {
    constexpr int aw = alpha_words(CMAX), cw = cand_words(CMAX);
    __shared__ __align__(16) uint32_t s_tile[kTile * aw];
    // the same tile by component, for four sphere tests at a time: centres, radius^2 (-1 for
    // a point that claims only itself), and q | 1 << 31 of such points (0 for the others)
    __shared__ __align__(16) float s_centre[CMAX][kTile];
    __shared__ __align__(16) float s_rsq[kTile];
    __shared__ __align__(16) uint32_t s_self[kTile];
    __shared__ int s_rank[kTile];                // rank of a tile entry among the event's points
    __shared__ int s_kept[kTile / kWave];        // entries each wave adds to the tile
    __shared__ int s_bin_lo[kMaxBinDims], s_bin_hi[kMaxBinDims];
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1), wave = tid >> 6;
    const int C = p.C, B = p.B;
    const int n_items = MODE == 0 ? p.n_vert_h : p.n_vert;
    const int *splits = MODE == 0 ? p.row_splits_h : p.row_splits;
    const int i_first = blockIdx.x * kScanBlock;
    const int i = i_first + tid;
    const bool valid = i < n_items;
    const int ev_lo = event_of(splits, p.num_rows, i_first);
    const int ev_hi = event_of(splits, p.num_rows, min(i_first + kScanBlock, n_items) - 1);
    // the workgroup's items span few events: uniform loads instead of a search per thread
    int my_ev = valid ? ev_lo : -1;
    for (int ev = ev_lo + 1; ev <= ev_hi; ++ev)
        if (valid && splits[ev] <= i) my_ev = ev;

    // ---- this thread's item ----
    float x[CMAX];
    int k[kMaxBinDims];
    bool alive = valid, uncoverable = false;
    int self_q = -1;
#pragma unroll
    for (int c = 0; c < CMAX; ++c) x[c] = 0.f;
#pragma unroll
    for (int d = 0; d < kMaxBinDims; ++d) k[d] = INT_MIN;
    bool was_open = false;
    if (MODE == 0) {
        // a wave's 64 positions are one word of the bit array
        const unsigned long long word = i_first + (tid & ~(kWave - 1)) < n_items ? p.open_bits[i >> 6] : 0ull;
        was_open = valid && ((word >> (tid & (kWave - 1))) & 1ull);
        alive = false;
        if (was_open) {
            const uint32_t *rec = p.cand + (size_t)i * cw;
            alive = i >= p.cursor_at[launch * p.num_rows + my_ev] && rec[CMAX + 6] == 0;
            if (alive) {
#pragma unroll
                for (int c = 0; c < CMAX; ++c) x[c] = __uint_as_float(rec[c]);
#pragma unroll
                for (int d = 0; d < kMaxBinDims; ++d) k[d] = (int)rec[CMAX + d];
            }
        }
    } else if (valid) {
        Grid g;
        g.load(p);
        if (CMAX == 4 && C == 4 && p.rows_aligned) {
            const float4 v = reinterpret_cast<const float4 *>(p.ccoords)[i];
            x[0] = v.x, x[1] = v.y, x[2] = v.z, x[3] = v.w;
        } else {
#pragma unroll
            for (int c = 0; c < CMAX; ++c)
                if (c < C) x[c] = p.ccoords[(size_t)i * C + c];
        }
        uncoverable = p.mask[i] != 0;
        self_q = p.to_filtered[i];
        g.split(p.hit_bin[i], B, k);
    }

    // sphere tests run on a copy whose first coordinate is NaN for a masked hit: no sphere claims it
    float xs[CMAX];
#pragma unroll
    for (int c = 0; c < CMAX; ++c) xs[c] = x[c];
    if (uncoverable) xs[0] = __uint_as_float(0x7fc00000u);
    const uint32_t self_key = self_q >= 0 ? ((uint32_t)self_q | 0x80000000u) : 0xffffffffu;

    int shower = -1, asso = -1;
    float best = 10e20f;

    for (int ev = ev_lo; ev <= ev_hi; ++ev) {
        const int first_h = p.row_splits_h[ev];
        const int rank_lo = (MODE == 0 && launch > 0) ? p.n_alpha_at[(launch - 1) * p.num_rows + ev] : 0;
        const int rank_hi = p.n_alpha_at[launch * p.num_rows + ev];
        bool mine = alive && my_ev == ev;
        // the bins of this workgroup's items of the event, per dimension
        int bin_lo[kMaxBinDims], bin_hi[kMaxBinDims];
#pragma unroll
        for (int d = 0; d < kMaxBinDims; ++d) bin_lo[d] = INT_MIN, bin_hi[d] = INT_MAX;
        if (MODE != 0 && rank_lo < rank_hi) {
            __syncthreads();  // everyone is done with the previous event's range
            if (tid < kMaxBinDims) s_bin_lo[tid] = INT_MAX, s_bin_hi[tid] = INT_MIN;
            __syncthreads();
#pragma unroll
            for (int d = 0; d < kMaxBinDims; ++d) {
                if (d >= B) continue;
                int lo = mine ? k[d] : INT_MAX, hi = mine ? k[d] : INT_MIN;
#pragma unroll
                for (int m = 1; m < kWave; m <<= 1) {
                    lo = min(lo, __shfl_xor(lo, m));
                    hi = max(hi, __shfl_xor(hi, m));
                }
                if (lane == 0) {
                    atomicMin(&s_bin_lo[d], lo);
                    atomicMax(&s_bin_hi[d], hi);
                }
            }
            __syncthreads();
#pragma unroll
            for (int d = 0; d < kMaxBinDims; ++d)
                if (d < B) bin_lo[d] = s_bin_lo[d], bin_hi[d] = s_bin_hi[d];
        }
        for (int base = rank_lo; base < rank_hi; base += kTile) {
            if (!__syncthreads_or(mine)) break;  // also: everyone is done with the previous tile
            int n_tile;
            bool solitary_here = false;
            if (MODE == 0) {
                // the candidates come in selection order, their bins are anywhere: every point goes in
                n_tile = min(kTile, rank_hi - base);
                const uint4 *src = reinterpret_cast<const uint4 *>(p.points + (size_t)(first_h + base) * aw);
                for (int e = tid; e < n_tile * (aw / 4); e += kScanBlock) reinterpret_cast<uint4 *>(s_tile)[e] = src[e];
                __syncthreads();
                if (tid < kTile) {
                    const uint32_t *a = s_tile + (size_t)tid * aw;
                    const bool real = tid < n_tile;
                    const uint32_t solq = real ? a[CMAX + 1] : 0u;
                    solitary_here = solq >> 31;
#pragma unroll
                    for (int c = 0; c < CMAX; ++c) s_centre[c][tid] = real ? __uint_as_float(a[c]) : 0.f;
                    s_rsq[tid] = (real && !solitary_here) ? __uint_as_float(a[CMAX]) : -1.f;
                    s_self[tid] = solitary_here ? solq : 0u;
                    s_rank[tid] = base + tid;
                }
            } else {
                // one point per thread; it stays if its box meets the items' bins
                const int n_chunk = min(kTile, rank_hi - base);
                const uint32_t *src = p.points + (size_t)(first_h + base + tid) * aw;
                uint32_t w[aw];
                bool keep = false;
                if (tid < n_chunk) {
#pragma unroll
                    for (int e = 0; e < aw / 4; ++e) {
                        const uint4 v = reinterpret_cast<const uint4 *>(src)[e];
                        w[4 * e] = v.x, w[4 * e + 1] = v.y, w[4 * e + 2] = v.z, w[4 * e + 3] = v.w;
                    }
                    keep = true;
#pragma unroll
                    for (int d = 0; d < kMaxBinDims; ++d) {
                        const uint32_t box = w[CMAX + 4 + d];
                        keep = keep && (int)(int16_t)(box & 0xffffu) <= bin_hi[d] && ((int)box >> 16) >= bin_lo[d];
                    }
                }
                const uint64_t kept = __ballot(keep);
                if (lane == 0) s_kept[wave] = __popcll(kept);
                __syncthreads();
                int at = 0;
                n_tile = 0;
#pragma unroll
                for (int w = 0; w < kTile / kWave; ++w) {
                    if (w == wave) at = n_tile;
                    n_tile += s_kept[w];
                }
                if (keep) {
                    const int t = at + __popcll(kept & ((1ull << lane) - 1ull));
#pragma unroll
                    for (int e = 0; e < aw / 4; ++e)
                        reinterpret_cast<uint4 *>(s_tile + (size_t)t * aw)[e] =
                            uint4{w[4 * e], w[4 * e + 1], w[4 * e + 2], w[4 * e + 3]};
                    const uint32_t solq = w[CMAX + 1];
                    solitary_here = solq >> 31;
#pragma unroll
                    for (int c = 0; c < CMAX; ++c) s_centre[c][t] = __uint_as_float(w[c]);
                    s_rsq[t] = solitary_here ? -1.f : __uint_as_float(w[CMAX]);
                    s_self[t] = solitary_here ? solq : 0u;
                    s_rank[t] = base + tid;
                }
                if (tid >= n_tile && tid < ((n_tile + 3) & ~3)) {  // the four-wide test reads up to here
#pragma unroll
                    for (int c = 0; c < CMAX; ++c) s_centre[c][tid] = 0.f;
                    s_rsq[tid] = -1.f;
                    s_self[tid] = 0u;
                }
            }
            const bool any_solitary = __syncthreads_or(solitary_here);
            if (mine) {
                int next_t = 0;
                while (next_t < n_tile) {
                    // the first point from next_t on whose sphere (or self test) takes the hit: four
                    // tests per step, each the reference's serial sum over the coordinates. The lanes
                    // of a wave leave this loop one by one; the complete test below then runs once
                    // for all of them.
                    int found = n_tile;
                    for (int t4 = next_t & ~3; t4 < n_tile; t4 += 4) {
                        float d0 = 0.f, d1 = 0.f, d2 = 0.f, d3 = 0.f;
#pragma unroll
                        for (int c = 0; c < CMAX; ++c) {
                            const float4 cc = *reinterpret_cast<const float4 *>(&s_centre[c][t4]);
                            float t = cc.x - xs[c];
                            d0 = d0 + t * t;
                            t = cc.y - xs[c];
                            d1 = d1 + t * t;
                            t = cc.z - xs[c];
                            d2 = d2 + t * t;
                            t = cc.w - xs[c];
                            d3 = d3 + t * t;
                        }
                        const float4 rr = *reinterpret_cast<const float4 *>(&s_rsq[t4]);
                        uint32_t hits = (d0 <= rr.x ? 1u : 0u) | (d1 <= rr.y ? 2u : 0u) | (d2 <= rr.z ? 4u : 0u) |
                                        (d3 <= rr.w ? 8u : 0u);
                        if (any_solitary) {
                            const uint4 sk = *reinterpret_cast<const uint4 *>(&s_self[t4]);
                            hits |= (sk.x == self_key ? 1u : 0u) | (sk.y == self_key ? 2u : 0u) |
                                    (sk.z == self_key ? 4u : 0u) | (sk.w == self_key ? 8u : 0u);
                        }
                        if (MODE == 2) {
                            // every point that covers the hit takes part in the running comparison
                            for (int j = 0; j < 4; ++j) {
                                if (!((hits >> j) & 1u)) continue;
                                const uint32_t *a = s_tile + (size_t)(t4 + j) * aw;
                                float dsq;
                                if (!covers<CMAX>(a, x, uncoverable, self_q, k, dsq)) continue;
                                const float lhs = best * __uint_as_float(a[CMAX]);
                                if (!(lhs >= dsq)) continue;
                                best = dsq;
                                shower = s_rank[t4 + j];
                                asso = (int)a[CMAX + 2];
                            }
                            continue;
                        }
                        if (t4 < next_t) hits &= ~((1u << (next_t - t4)) - 1u);
                        if (hits) {
                            found = t4 + __builtin_ctz(hits);
                            break;
                        }
                    }
                    if (found >= n_tile) break;
                    next_t = found + 1;
                    // the complete test for that one
                    const uint32_t *a = s_tile + (size_t)found * aw;
                    float dsq;
                    if (!covers<CMAX>(a, x, uncoverable, self_q, k, dsq)) continue;
                    shower = s_rank[found];
                    asso = (int)a[CMAX + 2];
                    mine = alive = false;
                    break;
                }
            }
        }
    }
    if (MODE == 0) {
        const unsigned long long still_open = __ballot(was_open && shower < 0);
        if ((tid & (kWave - 1)) == 0 && valid) p.open_bits[i >> 6] = still_open;
        return;
    }
    if (!valid) return;
    {
        p.assignment[i] = shower;
        p.association[i] = asso;
        if (MODE == 2) p.best_dsq[i] = best;
        if (shower >= 0 && self_q >= 0 && self_q < p.n_vert_h) p.taken_h[self_q] = 1;
    }
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

struct Workspace {
    uint64_t *keys, *keys_sorted;
    int *values, *order, *pos_h, *hit_bin, *walk_end, *cursor_at, *n_alpha_at;
    unsigned long long *open_bits;
    uint32_t *cand, *points;
    size_t used;
};

int coordinate_slots(int dimensions) { return dimensions <= 4 ? 4 : dimensions <= 8 ? 8 : kMaxDims; }

Workspace carve_workspace(void *base, int n_vert, int n_vert_h, int num_rows, int dimensions) {
    const int cmax = coordinate_slots(dimensions);
    const size_t nh = std::max(n_vert_h, 1), n = std::max(n_vert, 1), rows = std::max(num_rows, 1);
    Carver carve(base);
    Workspace w;
    w.keys = carve.take<uint64_t>(nh);
    w.keys_sorted = carve.take<uint64_t>(nh);
    w.values = carve.take<int>(nh);
    w.order = carve.take<int>(nh);
    w.pos_h = carve.take<int>(nh);
    w.hit_bin = carve.take<int>(n);
    w.open_bits = carve.take<unsigned long long>(nh / 64 + 2);
    w.points = carve.take<uint32_t>(nh * (size_t)alpha_words(cmax));
    w.walk_end = carve.take<int>(rows);
    w.cursor_at = carve.take<int>(kMaxLaunches * rows);
    w.n_alpha_at = carve.take<int>(kMaxLaunches * rows);
    w.cand = carve.take<uint32_t>(nh * (size_t)cand_words(cmax));
    w.used = carve.used;
    return w;
}

// returns through `last_launch` which launch of the event kernel holds the final counts
template <int CMAX>
int run(const CondParams &p, hipStream_t s, int &last_launch) {
    int rc;
    hit_prepare_kernel<<<ceil_div(std::max(p.n_vert, p.num_rows), 256), 256, 0, s>>>(p);
    if ((rc = check_launch("hit_prepare"))) return rc;
    if (p.n_vert_h > 0) {
        candidate_records_kernel<CMAX><<<ceil_div(p.n_vert_h, 256), 256, 0, s>>>(p);
        if ((rc = check_launch("candidate_records"))) return rc;
    }
    // the event kernel's list of condensation points lives in dynamic LDS; more than
    // the default has to be granted per kernel
    const size_t point_bytes = (size_t)alpha_words(CMAX) * sizeof(uint32_t);
    size_t list_bytes = 40 * 1024;
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(&condensate_event_kernel<CMAX>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024) == hipSuccess)
        list_bytes = 128 * 1024;
    (void)hipGetLastError();  // a refused grant is not an error of this call
    const int capacity = (int)(list_bytes / point_bytes) & ~3;  // the list is read four points at a time
    const int window = std::min(kBlock, capacity / 2 / kWave * kWave);
    // geometric shares of the sorted candidates, the last launch takes what is left;
    // n_vert_h bounds every event
    int budgets[kMaxLaunches];
    int n_launches = 0;
    long long reach = 0;
    for (int share = 1024; n_launches < kMaxLaunches - 1 && reach + share < p.n_vert_h; share *= 4) {
        budgets[n_launches++] = share;
        reach += share;
    }
    budgets[n_launches++] = -1;
    for (int l = 0; l < n_launches; ++l) {
        condensate_event_kernel<CMAX><<<p.num_rows, kBlock, list_bytes, s>>>(p, l, budgets[l], window, capacity);
        if ((rc = check_launch("condensate_event_kernel"))) return rc;
        if (l + 1 < n_launches && p.n_vert_h > 0) {
            cover_scan_kernel<CMAX, 0><<<ceil_div(p.n_vert_h, kScanBlock), kScanBlock, 0, s>>>(p, l);
            if ((rc = check_launch("cover_scan_kernel (candidates)"))) return rc;
        }
    }
    if (p.n_vert > 0) {
        if (p.by_max_beta)
            cover_scan_kernel<CMAX, 1><<<ceil_div(p.n_vert, kScanBlock), kScanBlock, 0, s>>>(p, n_launches - 1);
        else
            cover_scan_kernel<CMAX, 2><<<ceil_div(p.n_vert, kScanBlock), kScanBlock, 0, s>>>(p, n_launches - 1);
        if ((rc = check_launch("cover_scan_kernel (hits)"))) return rc;
    }
    last_launch = n_launches - 1;
    return HGC_OK;
}

}  // namespace

size_t condensates_workspace_bytes(int n_vert, int n_vert_h, int num_rows, int dimensions) {
    const size_t nh = std::max(n_vert_h, 1);
    size_t temp = 0;
    (void)rocprim::radix_sort_pairs(nullptr, temp, (const uint64_t *)nullptr, (uint64_t *)nullptr,
                                    (const int *)nullptr, (int *)nullptr, nh, 0,
                                    selection_key_bits(std::max(num_rows, 1)), (hipStream_t) nullptr);
    temp = std::max(temp, sample_sort_workspace_bytes());
    return align_up(temp) + carve_workspace(nullptr, n_vert, n_vert_h, num_rows, dimensions).used;
}

int condensates_assign(int dimensions, int dimensions_binning, int *d_condensates_assigned_h,
                       const float *d_ccoords_h, const float *d_dist_h, const float *d_beta_h,
                       const int *d_no_condensation_mask_h, int *d_high_assigned_status_h,
                       const int *d_original_indices_h, const int *d_row_splits_h, const float *d_ccoords,
                       const int *d_no_condensation_mask, const int *d_indices_to_filtered,
                       float *d_assignment_min_distance, int *d_assignment, int *d_association,
                       int *d_n_condensates, int *d_alpha_indices, const int *d_bin_splits, const int *d_n_bins,
                       const float *d_bin_widths, const int *d_row_splits, int num_rows, int assign_by_max_beta,
                       int n_vert, int n_vert_h, int *d_error, const int *d_high, const int *d_quirk,
                       void *workspace, size_t workspace_bytes, hipStream_t s) {
    HGC_REQUIRE(dimensions >= 1 && dimensions <= kMaxDims, "1 <= coordinate dimensions <= %d", kMaxDims);
    HGC_REQUIRE(dimensions_binning >= 1 && dimensions_binning <= kMaxBinDims && dimensions_binning <= dimensions,
                "1 <= binning dimensions <= min(%d, coordinate dimensions)", kMaxBinDims);
    HGC_REQUIRE(num_rows >= 0 && n_vert >= 0 && n_vert_h >= 0 && n_vert_h <= n_vert, "bad sizes");
    HGC_REQUIRE(d_n_condensates && d_row_splits && d_row_splits_h, "null pointer");
    HGC_REQUIRE(!d_high || (d_quirk && n_vert_h == n_vert), "hits as their own high-beta subset: sizes differ");
    if (!workspace || !aligned256(workspace) ||
        workspace_bytes < condensates_workspace_bytes(n_vert, n_vert_h, num_rows, dimensions))
        return fail(HGC_ERR_WORKSPACE, "condensates workspace missing, misaligned or too small");
    if (n_vert > 0)
        HGC_REQUIRE(d_ccoords && d_no_condensation_mask && d_indices_to_filtered && d_assignment && d_association &&
                        d_bin_splits && d_n_bins && d_bin_widths && (assign_by_max_beta || d_assignment_min_distance),
                    "null pointer");
    if (n_vert_h > 0)
        HGC_REQUIRE(d_condensates_assigned_h && d_ccoords_h && d_dist_h && d_beta_h && d_no_condensation_mask_h &&
                        d_high_assigned_status_h && d_original_indices_h && d_alpha_indices,
                    "null pointer");

    const Workspace w = carve_workspace(workspace, n_vert, n_vert_h, num_rows, dimensions);
    void *temp = static_cast<char *>(workspace) + w.used;
    size_t temp_bytes = workspace_bytes - w.used;

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
    p.rows_aligned = ((reinterpret_cast<uintptr_t>(d_ccoords) | reinterpret_cast<uintptr_t>(d_ccoords_h)) & 15u) == 0;
    p.high = d_high;
    p.quirk = d_quirk;
    p.order_h = w.order;
    p.pos_h = w.pos_h;
    p.hit_bin = w.hit_bin;
    p.cand = w.cand;
    p.open_bits = w.open_bits;
    p.points = w.points;
    p.walk_end = w.walk_end;
    p.cursor_at = w.cursor_at;
    p.n_alpha_at = w.n_alpha_at;

    int last_launch = 0;
    if (num_rows > 0) {
        if (n_vert_h > 0) {
            // The position of a hit completes its key where both fit into 64 bits: then the
            // keys differ pairwise and the sample sort orders them; a stable library radix
            // sort otherwise.
            int position_bits = 1;
            while ((1ll << position_bits) < (long long)n_vert_h) ++position_bits;
            const bool own_sort =
                sample_sort_supported(n_vert_h) && selection_key_bits(num_rows) + position_bits <= 64;
            selection_keys_kernel<<<ceil_div(n_vert_h, 256), 256, 0, s>>>(p, w.keys, w.values,
                                                                          own_sort ? position_bits : 0);
            int rc = check_launch("selection_keys");
            if (rc) return rc;
            if (own_sort) {
                rc = sample_sort_values(w.keys, w.keys_sorted, n_vert_h, position_bits, w.order, temp, temp_bytes, 0, s);
                if (rc) return rc;
            } else {
                HGC_HIP(rocprim::radix_sort_pairs(temp, temp_bytes, w.keys, w.keys_sorted, w.values, w.order,
                                                  (size_t)n_vert_h, 0, selection_key_bits(num_rows), s));
            }
        }
        const int slots = coordinate_slots(dimensions);
        const int rc = slots == 4   ? run<4>(p, s, last_launch)
                       : slots == 8 ? run<8>(p, s, last_launch)
                                    : run<kMaxDims>(p, s, last_launch);
        if (rc) return rc;
    }
    cumulative_counts_kernel<<<1, 64, 0, s>>>(w.n_alpha_at + (size_t)last_launch * num_rows, num_rows,
                                              d_n_condensates, d_error);
    return check_launch("cumulative_counts");
}

}  // namespace hgc

using namespace hgc;

extern "C" {

size_t hgc_binned_assign_to_condensates_workspace_bytes(int n_vert, int n_vert_h, int num_rows) {
    return condensates_workspace_bytes(n_vert, n_vert_h, num_rows, kMaxDims);  // the dimensions come with the call
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
    return condensates_assign(dimensions, dimensions_binning, d_condensates_assigned_h, d_ccoords_h, d_dist_h,
                              d_beta_h, d_no_condensation_mask_h, d_high_assigned_status_h, d_original_indices_h,
                              d_row_splits_h, d_ccoords, d_no_condensation_mask, d_indices_to_filtered,
                              d_assignment_min_distance, d_assignment, d_association, d_n_condensates,
                              d_alpha_indices, d_bin_splits, d_n_bins, d_bin_widths, d_row_splits, num_rows,
                              assign_by_max_beta, n_vert, n_vert_h, d_error, nullptr, nullptr, workspace,
                              workspace_bytes, as_stream(stream));
}

}  // extern "C"
