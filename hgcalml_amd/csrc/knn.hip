// Exact binned k-nearest-neighbour search, one wave64 per query point.
//
// Reference behaviour restated here:
//   modules/compiled/binned_select_knn_kernel.cc:19-196 (search, defaults, stop rule)
//   modules/compiled/binstepper.h:11-97                 (shell of bins at distance d)
//   modules/binned_select_knn_op.py:92-95               (un-sort, fused when a sorting is given)
//   modules/compiled/select_knn_kernel.cc:158,244-245   (radius rule)
//
// Design (gfx950, wave64):
//   * Points arrive grouped by bin, so the bins of one row of the grid (last
//     binned dimension running) are one contiguous range of points. A shell of
//     half-width d is cut into such ranges ("segments"); the 64 lanes look up 64
//     segments at once (cutting each against the current K-th distance) and
//     prefix-sum their lengths. Every non-empty segment marks the position of
//     its first candidate in a strip of LDS; the wave then walks the
//     concatenated candidate list 64 points per step, fully coalesced, and finds
//     the segment of a position as the prefix maximum of the marks.
//   * Each lane evaluates one candidate: serial fp32 sum of squared coordinate
//     differences in coordinate order (no FMA contraction), packed with the
//     candidate's index into a 64-bit key (distance bits high, index low), so a
//     single unsigned compare orders by (distance, index).
//   * The K-1 best keys live in registers, sorted across the lanes (rank r in
//     lane r%64, register r/64). A ballot finds the candidates that beat the
//     current K-th key; each is inserted with one DPP wave shift and two
//     compares, and the new K-th key is read back with a readlane. When 20 or
//     more of a step's 64 candidates enter (the first steps of every query), the
//     step is sorted across the lanes by a bitonic network and merged into the
//     list in one go instead.
//   * The shell loop stops exactly as the reference does: list full and
//     ((bw*d)*bw)*d > K-th distance, or no bin of the shell inside the grid.
//   * Only the rows of a shell that lie inside the grid and within reach of the
//     search get a slot: one per row on a face of the shell (its run), one or
//     two per inner row (its end caps).
//   * Optionally (callers that group the points by half-bin cells) the queries of
//     crowded bins walk a nested grid of half the bin width: walk_shells<FINE>.
//   * The kernel is bound by vector ALU issue; LDS holds only the marks. No
//     atomics, no barriers; every wave is its own workgroup and exits on its own.
#include "hgc_common.hpp"

namespace hgc {
namespace {

constexpr int kMaxBinDims = 5;
constexpr uint64_t kEmptyKey = ~0ull;

struct KnnParams {
    const float *coord;
    const int *bin_idx;
    const int *direction;
    const int *dim_bin_idx;
    const int *bin_boundaries;
    const int *cell_boundaries;  // NESTED kernels: one entry per half-bin cell
    const int *n_bins;
    const float *bin_width;
    const int *sorting;  // may be null
    const float *shift;  // may be null: what the binning subtracted from the binned coordinates
    int *out_idx;
    float *out_dist;
    int *status;      // may be null: device status word for data errors
    float radius_sq;  // < 0: no radius
    int n_vert, K, n_coords, n_bin_dim, n_bboundaries, tf_compat, use_direction;
    int boundary_shift;  // the boundary of bin b sits at bin_boundaries[b << boundary_shift]
    int rank_base;       // WINDOW kernels: the neighbour ranks below this one are in the output already
    // fine_bits = n_bin_dim: bin_idx is that of the spatial grouping, bin_idx[q] = bin << fine_bits |
    // half-bin bits, and the points of a bin are grouped by these cells. NESTED kernels: a query
    // whose bin holds more than fine_min_population points walks the nested grid of half the bin
    // width over cell_boundaries.
    int fine_bits, fine_min_population;
};

template <int C>
__device__ __forceinline__ float dist_sq(const float (&q)[C > 0 ? C : 1], const float *__restrict__ coord, int j,
                                         int n_coords, const float *__restrict__ qrow) {
    float acc = 0.f;
    if constexpr (C > 0) {
        // uniform base + 32-bit byte offset: the load takes its base from scalar registers
        const float *r = reinterpret_cast<const float *>(reinterpret_cast<const char *>(coord) +
                                                         (uint32_t)j * (uint32_t)(C * sizeof(float)));
        float x[C];
        if constexpr (C == 4 || C == 8) {  // rows are 16-byte aligned (checked on the host)
#pragma unroll
            for (int c = 0; c < C; c += 4) {
                const float4 v = *reinterpret_cast<const float4 *>(r + c);
                x[c] = v.x; x[c + 1] = v.y; x[c + 2] = v.z; x[c + 3] = v.w;
            }
        } else if constexpr (C == 6) {     // 8-byte aligned
#pragma unroll
            for (int c = 0; c < C; c += 2) {
                const float2 v = *reinterpret_cast<const float2 *>(r + c);
                x[c] = v.x; x[c + 1] = v.y;
            }
        } else if constexpr (C == 2) {
            const float2 v = *reinterpret_cast<const float2 *>(r);
            x[0] = v.x; x[1] = v.y;
        } else {
#pragma unroll
            for (int c = 0; c < C; ++c) x[c] = r[c];
        }
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const float d = q[c] - x[c];
            acc = acc + d * d;
        }
    } else {
        const float *r = coord + (size_t)j * n_coords;
        for (int c = 0; c < n_coords; ++c) {
            const float d = qrow[c] - r[c];
            acc = acc + d * d;
        }
    }
    return acc;
}

// A value that is the same in every lane, told to the compiler: what is computed from it
// then sits in scalar registers. (Loads through pointers the compiler cannot prove read-only
// are vector loads even at a wave-uniform address.) Not everything gains by it: a vector
// instruction takes one scalar operand only, so values that meet in one instruction, like
// the two edge distances of a dimension, are better left in vector registers.
__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ float uniform(float v) {
    return __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(v)));
}

extern "C" __device__ int __llvm_amdgcn_writelane(int, int, int) __asm("llvm.amdgcn.writelane");

// `into` with lane `lane` (wave-uniform) replaced by the wave-uniform `value`
__device__ __forceinline__ uint64_t writelane_u64(uint64_t value, int lane, uint64_t into) {
    const uint32_t lo = (uint32_t)__llvm_amdgcn_writelane((int)(uint32_t)value, lane, (int)(uint32_t)into);
    const uint32_t hi = (uint32_t)__llvm_amdgcn_writelane((int)(uint32_t)(value >> 32), lane, (int)(uint32_t)(into >> 32));
    return ((uint64_t)hi << 32) | lo;
}

// lane i receives v from lane i-1; lane 0 (and lanes whose source is masked off) read 0
__device__ __forceinline__ uint64_t wave_shift_up1_zero(uint64_t v) {
    const uint32_t lo = (uint32_t)__builtin_amdgcn_mov_dpp((int)(uint32_t)v, 0x138, 0xf, 0xf, true);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_mov_dpp((int)(uint32_t)(v >> 32), 0x138, 0xf, 0xf, true);
    return ((uint64_t)hi << 32) | lo;
}

// Sorted insert of the wave-uniform key c into the ascending list held across
// the lanes (and register levels); the largest key falls off the end. Lanes
// holding a larger key take their left neighbour's key (DPP wave shift under the
// execution mask of exactly those lanes), then c is written into the first of
// them. A key that is larger than everything in the list changes nothing.
template <int S>
__device__ __forceinline__ void sorted_insert(uint64_t (&key)[S], uint64_t c) {
    if constexpr (S == 1) {
        const uint64_t old = key[0];
        const bool larger = old > c;
        const uint64_t run = __builtin_amdgcn_ballot_w64(larger);  // contiguous upper lanes, the list is sorted
        if (run) {
            if (larger) key[0] = wave_shift_up1_zero(old);
            key[0] = writelane_u64(c, __ffsll((long long)run) - 1, key[0]);
        }
    } else {
        uint64_t carry = 0;   // what enters lane 0 of the next register level
        bool placed = false;  // wave-uniform
#pragma unroll
        for (int s = 0; s < S; ++s) {
            const uint64_t old = key[s];
            const uint64_t last = readlane_u64(old, kWave - 1);
            const bool larger = placed || old > c;
            const uint64_t run = __builtin_amdgcn_ballot_w64(larger);
            if (run) {
                if (larger) key[s] = wave_shift_up1_u64(old, carry);
                if (!placed) {
                    key[s] = writelane_u64(c, __ffsll((long long)run) - 1, key[s]);
                    placed = true;
                }
            }
            carry = last;
        }
    }
}

// value of lane `src` (taken modulo 64); one LDS crossbar pass, no bounds logic
__device__ __forceinline__ int from_lane_i32(int v, int src) { return __builtin_amdgcn_ds_bpermute(src << 2, v); }

__device__ __forceinline__ uint64_t from_lane_u64(uint64_t v, int src) {
    const uint32_t lo = (uint32_t)__builtin_amdgcn_ds_bpermute(src << 2, (int)(uint32_t)v);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_ds_bpermute(src << 2, (int)(uint32_t)(v >> 32));
    return ((uint64_t)hi << 32) | lo;
}

// ---- bulk insert: sort a batch of 64 keys across the lanes and merge it into the list ----
//
// A compare-exchange step of the bitonic network between lanes i and i^J. Which
// of the two lanes keeps the smaller key is a compile-time lane pattern, so it
// sits in scalar registers as a constant and the swap decision is one 64-bit
// compare plus a scalar xor; keys are unique apart from the empty key, for which
// a swap changes nothing.
constexpr uint64_t keeps_min_mask(int k, int j) {
    uint64_t m = 0;
    for (int i = 0; i < 64; ++i)
        if (((i & j) == 0) == ((i & k) == 0)) m |= 1ull << i;
    return m;
}

template <int K, int J>
__device__ __forceinline__ uint64_t compare_exchange(uint64_t key) {
    constexpr uint64_t kMin = keeps_min_mask(K, J);
    const uint64_t other = from_lane_u64(key, lane_id() ^ J);
    const uint64_t lt = __builtin_amdgcn_ballot_w64(other < key);
    // the lane that keeps the smaller key swaps when the other one is smaller, its partner when not
    const bool swap = __builtin_amdgcn_inverse_ballot_w64(lt ^ ~kMin);
    return swap ? other : key;
}

template <int K>
__device__ __forceinline__ uint64_t bitonic_merge_steps(uint64_t key) {
    if constexpr (K >= 64) key = compare_exchange<K, 32>(key);
    if constexpr (K >= 32) key = compare_exchange<K, 16>(key);
    if constexpr (K >= 16) key = compare_exchange<K, 8>(key);
    if constexpr (K >= 8) key = compare_exchange<K, 4>(key);
    if constexpr (K >= 4) key = compare_exchange<K, 2>(key);
    return compare_exchange<K, 1>(key);
}

// ascending sort of one key per lane
__device__ __forceinline__ uint64_t wave_sort_u64(uint64_t key) {
    key = bitonic_merge_steps<2>(key);
    key = bitonic_merge_steps<4>(key);
    key = bitonic_merge_steps<8>(key);
    key = bitonic_merge_steps<16>(key);
    key = bitonic_merge_steps<32>(key);
    return bitonic_merge_steps<64>(key);
}

// the 64 smallest of an ascending list and an ascending batch, ascending:
// min(list[i], batch[63-i]) is a bitonic sequence, six more steps sort it
__device__ __forceinline__ uint64_t merge_lowest_64(uint64_t list, uint64_t batch) {
    const uint64_t rev = from_lane_u64(batch, (kWave - 1) - lane_id());
    return bitonic_merge_steps<128>(rev < list ? rev : list);
}

// Merges an ascending batch of 64 keys into the list of S ascending runs of 64
// (run s holds ranks 64 s .. 64 s + 63): run by run, min(run[i], carry[63-i])
// and max(run[i], carry[63-i]) are bitonic sequences that hold the 64 smallest
// and the 64 largest of the two; six steps sort each, the smaller half stays,
// the larger one is carried to the next run. What falls off the last run is dropped.
template <int S>
__device__ __forceinline__ void merge_batch(uint64_t (&key)[S], uint64_t batch) {
#pragma unroll
    for (int s = 0; s < S; ++s) {
        if (s + 1 == S) {
            key[s] = merge_lowest_64(key[s], batch);
        } else {
            const uint64_t rev = from_lane_u64(batch, (kWave - 1) - lane_id());
            const bool take = rev < key[s];
            const uint64_t low = take ? rev : key[s], high = take ? key[s] : rev;
            key[s] = bitonic_merge_steps<128>(low);
            batch = bitonic_merge_steps<128>(high);
        }
    }
}

// below this many entering candidates in a step of 64 the one-by-one insert is cheaper
// (150k points in 4-D, K = 64, clusters / Gaussian blob: 0.519 / 0.924 ms at 12, 0.508 / 0.881 at 16,
// 0.504 / 0.864 at 20 and 24, 0.517 / 0.899 at 32)
constexpr int kBulkInsertMin = 20;
// lists of more runs than this would insert one by one (a merge costs 12 more steps per run)
constexpr int kBulkInsertMaxRuns = 8;

// NEAR_FIRST (the kernels of the nested grid, i.e. 48 neighbours and more: 16 events of 3-D points
// with K = 32 and a radius ran 4 % slower with it): segments of a batch whose bins are at least
// sqrt(kNearFirst) * d bin widths away (shell d) are walked after the nearer ones
// (150,000 points in 4-D, K = 64, kernel: Gaussian blob 508 us without,
// 455 / 464 / 464 / 473 us at 0.3 / 0.45 / 0.6 / 0.75; clusters + noise 409, 407 / 405 / 413 / 418;
// uniform 347, 359 / 352 / 347 / 354)
constexpr float kNearFirst = 0.45f;

// Candidates of one batch of segments that are walked per refill of a wave's
// strip of segment marks (one byte of LDS each); a multiple of 512.
constexpr int kMarkCap = 2048;

// Waves (= queries) per workgroup. Queries differ a lot in cost, and a wave slot
// of a workgroup is handed on only when the whole workgroup has ended: one wave
// per workgroup measured fastest (150k clustered points in 4-D, K = 64: 0.75 ms
// against 0.78 ms with 4 and 0.95 ms with 8).
constexpr int kQueriesPerBlock = 1;

// q = x / w, r = x % w for 0 <= x < 2^22 and w < 2^13, without an integer divide: with inv_w
// within an ulp of 1 / w (the hardware's approximate reciprocal will do) the float quotient is
// off by at most one, the remainder says which way
__device__ __forceinline__ void divmod_small(int x, int w, float inv_w, int &q, int &r) {
    q = (int)((float)x * inv_w);
    r = x - q * w;
    const int fix = (r >= w ? 1 : 0) - (r < 0 ? 1 : 0);
    q += fix;
    r -= fix * w;
}

// The walk over the shells of bins around query q (one wave), which leaves the Kn smallest keys
// in `key`. FINE: the walk runs on the nested grid of half the bin width (see KnnParams::fine_bits).
// Its cells are numbered 2 k + h per dimension (bin k, half h); the points of a bin come grouped
// by half-bin cell with the LAST dimension's half as the lowest bit, so a run of cells along the
// last dimension is contiguous inside a bin and falls into one piece per bin it touches: a row of
// the shell at distance d takes up to d + 1 segments instead of one. Any grid gives the same
// result, the K smallest keys: the choice is one of cost only.
//
// A walk on the nested grid gives up (returns false, the list is to be discarded) when it has not
// ended after shell kFineMaxShell: its shells have 2^(B-1) times the rows of the bins' shells
// and more segments per row, which pays only while few of them are needed. All coordinates
// being binned, that is the rule where the bin's neighbourhood is about as crowded as the bin.
constexpr int kFineMaxShell = 3;

template <int C, int NB, int S, bool MAPPED, bool WINDOW, bool FINE, bool NEAR_FIRST>
__device__ __forceinline__ bool walk_shells(const KnnParams &p, const int q, const int lane, uint8_t *const marks,
                                            const int Kn, const uint64_t floor_key, uint64_t (&key)[S]) {
    constexpr int kDims = NB > 0 ? NB : kMaxBinDims;  // array extents
    {
        // query coordinates (wave-uniform)
        float qc[C > 0 ? C : 1];
        const float *qrow = p.coord + (size_t)q * p.n_coords;
        if constexpr (C > 0) {
#pragma unroll
            for (int c = 0; c < C; ++c) qc[c] = qrow[c];
        }

        const int B = NB > 0 ? NB : p.n_bin_dim;
        const int own_cell = uniform(p.bin_idx[q]);   // with fine_bits: bin and half-bin bits
        const int own_bin = own_cell >> p.fine_bits;
        int nb[kDims], qb[kDims];
        int cells_per_event = 1;
        int reach_max = 0;  // beyond this shell distance no bin is inside the grid
#pragma unroll
        for (int i = 0; i < kDims; ++i) {
            nb[i] = 1;
            qb[i] = 0;
            if (i < B) {
                nb[i] = uniform(p.n_bins[i]);
                qb[i] = uniform(p.dim_bin_idx[(size_t)q * (B + 1) + 1 + i]);
                cells_per_event *= nb[i];
                if (FINE) {
                    nb[i] *= 2;
                    qb[i] = 2 * qb[i] + ((own_cell >> (B - 1 - i)) & 1);
                }
                reach_max = max(reach_max, max(qb[i], nb[i] - 1 - qb[i]));
            }
        }
        const int event_base = cells_per_event * (own_bin / cells_per_event);
        const int nb_last = nb[B - 1], qb_last = qb[B - 1];
        const int bins_last = FINE ? nb_last >> 1 : nb_last;  // bins (not cells) along the last dimension
        const float bw = FINE ? 0.5f * p.bin_width[0] : p.bin_width[0];
        const float inv_bw = 1.f / bw;
        const float bins_per_unit = 1.001f * inv_bw;  // generous by 0.1 %, for the pruning bound only

        // Position of the query inside its own bin, in bin widths: to_lower[i] is a
        // lower bound of its distance to the bin's lower edge, to_upper[i] to the
        // upper edge (both 0 when the binning shift is unknown). They tighten the
        // lower bound of the distance to neighbouring bins used for pruning.
        float to_lower[kDims], to_upper[kDims];
#pragma unroll
        for (int i = 0; i < kDims; ++i) {
            to_lower[i] = 0.f;
            to_upper[i] = 0.f;
            if (i < B && p.shift) {
                const float frac = (qrow[i] - p.shift[i]) * inv_bw - (float)qb[i];
                if (frac >= 0.f && frac <= 1.f) {
                    to_lower[i] = fmaxf(frac - 1e-3f, 0.f);
                    to_upper[i] = fmaxf(1.f - frac - 1e-3f, 0.f);
                }
            }
        }
        const float tl_last = to_lower[B - 1], tu_last = to_upper[B - 1];

        const bool has_radius = p.radius_sq >= 0.f;
        const int kth_lane = (Kn - 1) & (kWave - 1);
        const int kth_level = (Kn - 1) >> 6;
        // The K-th key is re-read once per step of 64 candidates, not per insert.
        uint64_t thr = kEmptyKey;  // current K-th key: candidates at or above it cannot enter
        // first key beyond the radius: d² <= r² <=> key < (bits(r²) + 1) << 32 for the non-negative r²
        const uint64_t radius_limit = has_radius ? (uint64_t)(__float_as_uint(p.radius_sq) + 1u) << 32 : kEmptyKey;
        uint64_t cut = radius_limit;  // min(thr, radius_limit): what a candidate's key has to stay below

        // Row and slot numbers of a shell are divided as floats (divmod_small), which is exact below
        // 2^22 for divisors below 2^13: no shell has more rows than the grid, times the pieces of
        // a row on the nested grid.
        {
            long long grid_rows = FINE ? nb_last / 2 + 2 : 2;
            bool rows_fit = true;
            for (int i = 0; i < B - 1; ++i) {
                grid_rows = min(grid_rows * nb[i], 1ll << 40);
                rows_fit = rows_fit && nb[i] < (1 << 13);
            }
            if (!rows_fit || grid_rows >= (1ll << 22)) {
                if (FINE) return false;  // the grid of bins may do
                if (p.status && lane == 0) atomicOr(p.status, HGC_FLAG_SHELL_TOO_WIDE);
                return true;  // the list stays empty
            }
        }
        // the first shell whose slots need more than one batch of 64 (walked whole: (2d+1)^(B-1)
        // rows and (2d-1)^(B-1) inner rows; on the nested grid d + 1 pieces per row)
        const int first_cut_shell = FINE ? (B == 2 ? 5 : B == 3 ? 2 : B == 4 ? 2 : 1) : (B == 2 ? 17 : B == 3 ? 3 : B == 4 ? 2 : 1);

        // Shell 0 (the query's own bin) never ends the search. When it cannot fill
        // the list either (so that it cannot prune shell 1), it is walked together
        // with shell 1: every row of that shell then takes its whole run of the last
        // dimension, and the run of the centre row contains the own bin.
        bool with_own_bin = false;
        if (reach_max > 0 && own_bin + 1 < p.n_bboundaries) {
            if (FINE)
                with_own_bin = p.cell_boundaries[own_cell + 1] - p.cell_boundaries[own_cell] <= Kn;
            else
                with_own_bin = p.bin_boundaries[(size_t)(own_bin + 1) << p.boundary_shift] -
                                   p.bin_boundaries[(size_t)own_bin << p.boundary_shift] <= Kn;
        }
        for (int d = uniform(with_own_bin ? 1 : 0); d <= reach_max; ++d) {
            if (FINE && d > kFineMaxShell) return false;
            // The shell is walked as rows of bins (cells) along the last dimension. Only rows inside
            // the grid and within reach of the search are numbered: per leading dimension the
            // offsets -below[i] .. -below[i] + width[i] - 1, where an offset o is within reach when
            // (|o| - 1 + distance to the facing edge of the own bin) bin widths do not exceed the
            // K-th distance (the radius) as it is when the shell begins, generously rounded.
            // (A shell whose slots fit one batch anyway is cut to the grid only.)
            const bool cut_to_reach = d >= first_cut_shell;
            float reach_bins = 3.0e9f;
            if (cut_to_reach) {
                float reach2_shell = thr == kEmptyKey ? 3.0e38f : __uint_as_float((uint32_t)(thr >> 32));
                if (has_radius) reach2_shell = fminf(reach2_shell, p.radius_sq);
                if (reach2_shell < 1.0e37f) reach_bins = __builtin_amdgcn_sqrtf(reach2_shell) * bins_per_unit + 1.001f;
            }
            int below[kDims], width[kDims], below_in[kDims], width_in[kDims];
            float inv_width[kDims], inv_width_in[kDims];
            int n_rows = 1;
            int n_inner = 1;  // rows with every leading offset inside +-(d - 1): they contribute end caps only
#pragma unroll
            for (int i = 0; i < kDims - 1; ++i) {
                below[i] = below_in[i] = 0;
                width[i] = width_in[i] = 1;
                inv_width[i] = inv_width_in[i] = 1.f;
                if (i < B - 1) {
                    int lo_i = min(d, qb[i]), hi_i = min(d, nb[i] - 1 - qb[i]);
                    if (cut_to_reach) {
                        lo_i = min(lo_i, uniform((int)fminf(reach_bins - to_lower[i], 1.0e9f)));
                        hi_i = min(hi_i, uniform((int)fminf(reach_bins - to_upper[i], 1.0e9f)));
                    }
                    below[i] = lo_i;
                    width[i] = lo_i + hi_i + 1;
                    below_in[i] = min(lo_i, max(d - 1, 0));
                    width_in[i] = below_in[i] + min(hi_i, max(d - 1, 0)) + 1;
                    if (i > 0) {  // the leading digit of a row number is what the divisions leave
                        inv_width[i] = __builtin_amdgcn_rcpf((float)width[i]);
                        inv_width_in[i] = __builtin_amdgcn_rcpf((float)width_in[i]);
                    }
                    n_rows *= width[i];  // at most the rows of the grid: see rows_fit
                    n_inner *= width_in[i];
                }
            }
            // the last dimension: are the end caps (offsets -d and +d) inside the grid and within reach?
            int lo_last = min(d, qb_last), hi_last = min(d, nb_last - 1 - qb_last);
            if (cut_to_reach) {
                lo_last = min(lo_last, uniform((int)fminf(reach_bins - tl_last, 1.0e9f)));
                hi_last = min(hi_last, uniform((int)fminf(reach_bins - tu_last, 1.0e9f)));
            }
            const bool low_caps = lo_last == d, high_caps = hi_last == d;
            // Segments per row on the nested grid: a run falls into one piece per bin it touches
            // (an inner row uses two of them for its end caps).
            const int P = FINE ? max(2, ((qb_last + hi_last) >> 1) - ((qb_last - lo_last) >> 1) + 1) : 1;
            const float inv_P = __builtin_amdgcn_rcpf((float)P);
            const float near2 = kNearFirst * (bw * (float)d) * (bw * (float)d);
            // Slots of the shell. Grid of bins: one per row (the run of a row on a face of the
            // shell, one end cap of an inner row) and, when both end caps are in reach, one more per
            // inner row. When the own bin is walked with shell 1 every row is a run. Nested grid:
            // P per row.
            const bool runs_only = d == 0 || (d == 1 && with_own_bin);
            const int n_slots = d == 0 ? 1 : FINE ? n_rows * P : (!runs_only && low_caps && high_caps) ? n_rows + n_inner : n_rows;

            // batches of 64 slots; NEAR_FIRST: from the middle of the numbering outwards, so that the rows
            // with small leading offsets, the nearer ones, come first (1 to 2 % of the kernel time)
            const int n_batches = (n_slots + kWave - 1) / kWave;
            for (int slot_lin = 0, turn = 0; slot_lin < n_slots; slot_lin += kWave, ++turn) {
                int slot0 = slot_lin;
                if constexpr (NEAR_FIRST) {
                    const int mid = (n_batches - 1) >> 1;
                    slot0 = kWave * ((turn & 1) ? mid + ((turn + 1) >> 1) : mid - (turn >> 1));
                }
                // ---- each lane resolves one segment of the shell ----
                int seg_start = 0, seg_len = 0;
                [[maybe_unused]] bool far_segment = false;  // NEAR_FIRST: walked after the near ones of its batch
                const int slot = slot0 + lane;
                // Nothing farther than `reach2` can still enter the list (K-th distance
                // once the list is full, the radius cut otherwise). A bin at offset o
                // from the query's bin is at least (|o|-1) bin widths, plus the
                // distance to the facing edge of the own bin, away in that dimension.
                float reach2 = thr == kEmptyKey ? 3.0e38f : __uint_as_float((uint32_t)(thr >> 32));
                if (has_radius) reach2 = fminf(reach2, p.radius_sq);
                if (slot < n_slots) {
                    int row, piece;
                    bool inner = false;  // numbered among the inner rows
                    if (FINE) {
                        divmod_small(slot, P, inv_P, row, piece);
                    } else {
                        inner = slot >= n_rows;
                        row = inner ? slot - n_rows : slot;
                        piece = (inner || !low_caps) ? 1 : 0;  // the end cap an inner row takes in this slot
                    }
                    const bool second = piece == 1;
                    bool on_face = runs_only;
                    int cell = 0, halves = 0;
                    float gap2 = 0.f;  // squared lower bound of the distance to this row of bins
                    int off[kDims];
#pragma unroll
                    for (int i = kDims - 2; i >= 0; --i) {
                        off[i] = 0;
                        if (i < B - 1) {
                            // digits of the row number: offsets of the leading dimensions
                            const int below_i = inner ? below_in[i] : below[i];
                            if (i > 0) {
                                int digit;
                                divmod_small(row, inner ? width_in[i] : width[i], inner ? inv_width_in[i] : inv_width[i],
                                             row, digit);
                                off[i] = digit - below_i;
                            } else {
                                off[i] = row - below_i;  // what is left is the leading digit
                            }
                        }
                    }
#pragma unroll
                    for (int i = 0; i < kDims - 1; ++i) {
                        if (i < B - 1) {
                            const int o = off[i];
                            const int k = qb[i] + o;  // inside the grid: the numbered rows all are
                            on_face = on_face || o == d || o == -d;
                            if (FINE) {
                                cell = cell * (nb[i] >> 1) + (k >> 1);
                                halves = (halves << 1) | (k & 1);
                            } else {
                                cell = cell * nb[i] + k;
                            }
                            const float edge = o > 0 ? to_upper[i] : to_lower[i];
                            const float g = o == 0 ? 0.f : ((float)(abs(o) - 1) + edge) * bw;
                            gap2 += g * g;
                        }
                    }
                    // a whole run of the last dimension (rows on a face of the shell), or one of the
                    // two end caps
                    const float cap_gap = ((float)(d - 1) + (second ? tu_last : tl_last)) * bw;
                    const float cap2 = gap2 + cap_gap * cap_gap;
                    // bins of a run that are provably too far are cut off (bound
                    // generous by 0.1 % and a thousandth of a bin)
                    const float rest = fmaxf(reach2 - 0.999f * gap2, 0.f);
                    const float span = rest < 1.0e37f ? __builtin_amdgcn_sqrtf(rest) * bins_per_unit + 1.001f : 3.0e9f;
                    const int run_lo = max(qb_last - d, qb_last - (int)fminf(span - tl_last, 1.0e9f));
                    const int run_hi = min(qb_last + d, qb_last + (int)fminf(span - tu_last, 1.0e9f));
                    const int cap = second ? qb_last + d : qb_last - d;
                    int lo = on_face ? run_lo : cap;
                    int hi = on_face ? run_hi : cap;
                    bool too_far = on_face ? 0.999f * gap2 > reach2 : (piece > 1 || 0.999f * cap2 > reach2);
                    if constexpr (NEAR_FIRST) far_segment = (on_face ? gap2 : cap2) > near2;
                    lo = max(lo, 0);
                    hi = min(hi, nb_last - 1);
                    if (FINE) {
                        if (on_face) {
                            // piece number `piece` of the run: the part inside one bin, counted from the
                            // first bin any run of this shell can touch (not from this row's own first
                            // bin: the run shrinks with the K-th distance while the row's slots may lie
                            // in two batches)
                            const int bin = ((qb_last - lo_last) >> 1) + piece;
                            lo = max(lo, 2 * bin);
                            hi = min(hi, 2 * bin + 1);
                        }
                    }
                    if (!too_far && lo <= hi) {
                        if (FINE) {
                            const int bin = event_base + cell * bins_last + (lo >> 1);
                            if (bin + 1 < p.n_bboundaries) {
                                const int first = (((bin << (B - 1)) | halves) << 1) | (lo & 1);
                                const int last = ((((bin << (B - 1)) | halves) << 1) | (hi & 1)) + 1;
                                seg_start = p.cell_boundaries[first];
                                seg_len = p.cell_boundaries[last] - seg_start;
                            } else if (p.status) {
                                atomicOr(p.status, HGC_FLAG_BIN_BEYOND_TABLE);
                            }
                        } else {
                            const int first = event_base + cell * nb_last + lo;
                            const int last = event_base + cell * nb_last + hi + 1;
                            if (last < p.n_bboundaries) {
                                seg_start = p.bin_boundaries[(size_t)first << p.boundary_shift];
                                seg_len = p.bin_boundaries[(size_t)last << p.boundary_shift] - seg_start;
                            } else if (p.status) {  // the reference prints "idx out of range" and skips the bin
                                atomicOr(p.status, HGC_FLAG_BIN_BEYOND_TABLE);
                            }
                        }
                    }
                }
                // The segments whose lower bound of the distance is within near2 come first in the
                // candidate list, the others behind them (marks 65..128, so that the prefix maximum
                // keeps the two apart): fewer candidates enter the list only to be pushed out again.
                int seg_off, total;
                uint8_t mark;
                if constexpr (NEAR_FIRST) {
                    const int end_near = wave_inclusive_sum(far_segment ? 0 : seg_len);
                    const int end_far = wave_inclusive_sum(far_segment ? seg_len : 0);
                    const int total_near = readlane_i32(end_near, kWave - 1);
                    seg_off = (far_segment ? total_near + end_far : end_near) - seg_len;
                    total = total_near + readlane_i32(end_far, kWave - 1);
                    mark = (uint8_t)(lane + (far_segment ? kWave + 1 : 1));
                } else {
                    const int seg_end_off = wave_inclusive_sum(seg_len);
                    seg_off = seg_end_off - seg_len;
                    total = readlane_i32(seg_end_off, kWave - 1);
                    mark = (uint8_t)(lane + 1);
                }
                // candidate position -> point index for the owning segment; kept one lane up,
                // so that the mark (lane number + 1) is the lane to read it from
                // (DPP wave_ror:1; lane 63's value goes to lane 0, which is where mark 64 reads)
                const int seg_delta = __builtin_amdgcn_update_dpp(0, seg_start - seg_off, 0x13c, 0xf, 0xf, false);

                // ---- walk the concatenated candidates, 64 per step ----
                // Every non-empty segment marks its first position of the list with its
                // lane number + 1 (+ 64 for the far ones) in this wave's strip of LDS; the owner of a
                // position is then the prefix maximum of the marks (offsets rise with the lane).
                uint32_t owner_carry = 0;
                for (int c0 = 0; c0 < total; c0 += kMarkCap) {
                    const int chunk = min(kMarkCap, total - c0);
                    for (int base = 0; base < chunk; base += kWave * 8)
                        *reinterpret_cast<uint64_t *>(marks + base + lane * 8) = 0;
                    wave_lds_fence();
                    const int rel = seg_off - c0;
                    if (seg_len > 0 && rel >= 0 && rel < chunk) marks[rel] = mark;
                    wave_lds_fence();
                    for (int t = 0; t < chunk; t += kWave) {
                        const int c = c0 + t + lane;
                        uint32_t owner = wave_inclusive_max(marks[t + lane]);
                        owner = max(owner, owner_carry);
                        owner_carry = (uint32_t)readlane_i32((int)owner, kWave - 1);
                        const int j = c + from_lane_i32(seg_delta, (int)owner);
                        // lane masks are combined as integers on the scalar side
                        const bool in_list = c < total;
                        uint64_t valid = __builtin_amdgcn_ballot_w64(in_list) & __builtin_amdgcn_ballot_w64(j != q);
                        const int jj = in_list ? j : q;
                        const uint32_t id = MAPPED ? *reinterpret_cast<const uint32_t *>(
                                                         reinterpret_cast<const char *>(p.sorting) + ((uint32_t)jj << 2))
                                                   : (uint32_t)jj;
                        const float dsq = dist_sq<C>(qc, p.coord, jj, p.n_coords, qrow);
                        if (p.use_direction) {
                            const int dj = p.direction[jj];
                            valid &= ~__builtin_amdgcn_ballot_w64(dj == 1 || dj == 2);  // may not be a neighbour
                        }
                        const uint64_t ck = ((uint64_t)__float_as_uint(dsq) << 32) | id;
                        if (WINDOW) valid &= __builtin_amdgcn_ballot_w64(ck > floor_key);
                        // below the K-th key and (keys compare like distances) within the radius
                        uint64_t beats = valid & __builtin_amdgcn_ballot_w64(ck < cut);
                        if (beats) {
                            if (S <= kBulkInsertMaxRuns && (int)__popcll(beats) >= kBulkInsertMin) {
                                const bool enters = __builtin_amdgcn_inverse_ballot_w64(beats);
                                const uint64_t batch = wave_sort_u64(enters ? ck : kEmptyKey);
                                // an empty list (its smallest key is the empty key) is replaced
                                if (readlane_u64(key[0], 0) == kEmptyKey) key[0] = batch;
                                else merge_batch<S>(key, batch);
                                beats = 0;
                            }
                            while (beats) {
                                const int src = __ffsll((long long)beats) - 1;
                                beats &= beats - 1;
                                const uint64_t cand = readlane_u64(ck, src);
                                // a candidate that an earlier insert of this step has pushed beyond the
                                // K-th rank lands in a spare rank behind it or, in a list without one,
                                // is larger than every key and changes nothing
                                sorted_insert<S>(key, cand);
                            }
#pragma unroll
                            for (int s = 0; s < S; ++s)
                                if (s == kth_level) thr = readlane_u64(key[s], kth_lane);
                            // the low word of radius_limit is 0: the high words decide
                            cut = (uint32_t)(thr >> 32) < (uint32_t)(radius_limit >> 32) ? thr : radius_limit;
                        }
                    }
                }
            }

            // stop rule (fp32, evaluated left to right); on the nested grid, which the reference does
            // not have, with a margin for points that rounding has put into the neighbouring cell
            float reach = bw * (float)d;
            reach = reach * bw;
            reach = reach * (float)d;
            if (FINE) reach *= 0.998f;
            uint64_t kth = kEmptyKey;
#pragma unroll
            for (int s = 0; s < S; ++s)
                if (s == kth_level) kth = readlane_u64(key[s], kth_lane);
            if (kth != kEmptyKey && reach > __uint_as_float((uint32_t)(kth >> 32))) break;
            if (has_radius && reach > p.radius_sq) break;
        }
    }
    return true;
}

// C: coordinates per point, NB: binned dimensions (0 for either: taken from the
// arguments), S: registers of the sorted list per lane, MAPPED: results in the
// index space and at the positions of `sorting`.
// WINDOW: more neighbours are asked for than the registers hold (64 S). The search then runs
// once per window of 64 S ranks: launch t finds the 64 S smallest keys ABOVE the last key of
// launch t-1 (read back from the output row) and writes them behind it. Every launch walks
// the shells from the query's bin again and stops by the same rule on its own list, so each
// window is exact; slow (the walk is repeated) but without a bound on K.
// NESTED: the search runs over a nested grid (see KnnParams::fine_bits): a query whose bin holds more
// than fine_min_population points walks the nested grid (and the grid of bins after all when that
// walk gives up), the others the grid of bins.
template <int C, int NB, int S, bool MAPPED, bool WINDOW = false, bool NESTED = false>
__global__ __launch_bounds__(kQueriesPerBlock * kWave)
__attribute__((amdgpu_waves_per_eu(S <= 2 ? 8 : 1, 8)))
void knn_wave_kernel(const KnnParams p) {
    __shared__ __attribute__((aligned(8))) uint8_t mark_strips[kQueriesPerBlock][kMarkCap];
    const int lane = lane_id();
    // queries come in bin order and differ a lot in cost from region to region:
    // chunks of 512 of them are dealt to the XCDs in turn
    const int tile = xcd_chunked_block<512>(blockIdx.x, gridDim.x);
    const int q = tile * kQueriesPerBlock + (threadIdx.x >> 6);  // one query per wave
    uint8_t *const marks = mark_strips[threadIdx.x >> 6];
    if (q >= p.n_vert) return;
    bool crowded = false;
    if constexpr (NESTED) {
        const int own_bin = uniform(p.bin_idx[q]) >> p.fine_bits;
        if (own_bin + 1 < p.n_bboundaries)
            crowded = p.bin_boundaries[(size_t)(own_bin + 1) << p.boundary_shift] -
                          p.bin_boundaries[(size_t)own_bin << p.boundary_shift] > p.fine_min_population;
    }

    const int K = p.K;
    const int rank_base = WINDOW ? p.rank_base : 0;
    const int Kn = WINDOW ? min(K - 1 - rank_base, S * kWave) : K - 1;  // neighbours (besides the point itself) to find
    const int self_id = MAPPED ? p.sorting[q] : q;
    const size_t out_row = (size_t)self_id * K;
    const int pad_idx = p.tf_compat ? self_id : -1;

    bool searching = Kn > 0;
    uint64_t floor_key = 0;  // WINDOW: only keys above this one are candidates
    if (WINDOW && rank_base > 0) {
        const int last_idx = p.out_idx[out_row + rank_base];
        const float last_dist = p.out_dist[out_row + rank_base];
        if (last_idx == pad_idx) searching = false;  // the windows before found fewer points than they had room for
        floor_key = ((uint64_t)__float_as_uint(last_dist) << 32) | (uint32_t)last_idx;
    }
    if (p.use_direction) {
        const int dq = p.direction[q];
        if (dq == 0 || dq == 2) searching = false;  // may not have neighbours
    }

    uint64_t key[S];
#pragma unroll
    for (int s = 0; s < S; ++s) key[s] = kEmptyKey;

    if (searching) {
        if constexpr (NESTED) {
            if (!crowded) {
                walk_shells<C, NB, S, MAPPED, WINDOW, false, NESTED>(p, q, lane, marks, Kn, floor_key, key);
            } else if (!walk_shells<C, NB, S, MAPPED, WINDOW, true, NESTED>(p, q, lane, marks, Kn, floor_key, key)) {
#pragma unroll
                for (int s = 0; s < S; ++s) key[s] = kEmptyKey;
                walk_shells<C, NB, S, MAPPED, WINDOW, false, NESTED>(p, q, lane, marks, Kn, floor_key, key);
            }
        } else {
            walk_shells<C, NB, S, MAPPED, WINDOW, false, NESTED>(p, q, lane, marks, Kn, floor_key, key);
        }
    }

    // ---- write the row: slot 0 = self, then ascending (distance, index) ----
    if (lane == 0 && rank_base == 0) {
        p.out_idx[out_row] = self_id;
        p.out_dist[out_row] = 0.f;
    }
#pragma unroll
    for (int s = 0; s < S; ++s) {
        const int rank = s * kWave + lane;
        if (rank < Kn) {
            const bool filled = key[s] != kEmptyKey;
            p.out_idx[out_row + 1 + rank_base + rank] = filled ? (int)(uint32_t)key[s] : pad_idx;
            p.out_dist[out_row + 1 + rank_base + rank] = filled ? __uint_as_float((uint32_t)(key[s] >> 32)) : 0.f;
        }
    }
}

template <int C, int NB, bool MAPPED>
int launch_levels(const KnnParams &p, hipStream_t s) {
    const int levels = std::max(1, ceil_div(p.K - 1, kWave));
    const dim3 grid(ceil_div(p.n_vert, kQueriesPerBlock)), block(kQueriesPerBlock * kWave);
    if (levels > kBulkInsertMaxRuns) {  // more neighbours than the registers hold: one launch per window of ranks
        KnnParams window = p;
        for (window.rank_base = 0; window.rank_base < p.K - 1; window.rank_base += kBulkInsertMaxRuns * kWave) {
            knn_wave_kernel<C, NB, kBulkInsertMaxRuns, MAPPED, true><<<grid, block, 0, s>>>(window);
            const int rc = check_launch("knn_wave_kernel (window of ranks)");
            if (rc) return rc;
        }
        return HGC_OK;
    }
    if constexpr (MAPPED && C == NB && NB >= 3 && NB <= 4) {  // all coordinates binned: a crowded bin has its neighbours close by
        if (p.fine_bits > 0 && p.cell_boundaries) {
            switch (levels) {
                case 1: knn_wave_kernel<C, NB, 1, MAPPED, false, true><<<grid, block, 0, s>>>(p); break;
                case 2: knn_wave_kernel<C, NB, 2, MAPPED, false, true><<<grid, block, 0, s>>>(p); break;
                case 3:
                case 4: knn_wave_kernel<C, NB, 4, MAPPED, false, true><<<grid, block, 0, s>>>(p); break;
                default: knn_wave_kernel<C, NB, 8, MAPPED, false, true><<<grid, block, 0, s>>>(p); break;
            }
            return check_launch("knn_wave_kernel (nested grid)");
        }
    }
    switch (levels) {
        case 1: knn_wave_kernel<C, NB, 1, MAPPED><<<grid, block, 0, s>>>(p); break;
        case 2: knn_wave_kernel<C, NB, 2, MAPPED><<<grid, block, 0, s>>>(p); break;
        case 3:
        case 4: knn_wave_kernel<C, NB, 4, MAPPED><<<grid, block, 0, s>>>(p); break;
        default: knn_wave_kernel<C, NB, 8, MAPPED><<<grid, block, 0, s>>>(p); break;
    }
    return check_launch("knn_wave_kernel");
}

// The usual shapes (up to 8 coordinates; binned dimensions = min(3, coordinates), the reference
// wrapper's default, or min(4, coordinates), the pipeline's own grid) get kernels with both
// numbers fixed at compile time, anything else the one that reads them.
template <bool MAPPED>
int launch_coords(const KnnParams &p, hipStream_t s) {
    if (p.n_coords == 2 && p.n_bin_dim == 2) return launch_levels<2, 2, MAPPED>(p, s);
    if (p.n_coords == 3 && p.n_bin_dim == 3) return launch_levels<3, 3, MAPPED>(p, s);
    if (p.n_coords == 4 && p.n_bin_dim == 3) return launch_levels<4, 3, MAPPED>(p, s);
    if (p.n_coords == 4 && p.n_bin_dim == 4) return launch_levels<4, 4, MAPPED>(p, s);
    if (p.n_coords == 5 && p.n_bin_dim == 4) return launch_levels<5, 4, MAPPED>(p, s);
    if (p.n_coords == 6 && p.n_bin_dim == 4) return launch_levels<6, 4, MAPPED>(p, s);
    if (p.n_coords == 7 && p.n_bin_dim == 4) return launch_levels<7, 4, MAPPED>(p, s);
    if (p.n_coords == 8 && p.n_bin_dim == 4) return launch_levels<8, 4, MAPPED>(p, s);
    if (p.n_coords == 5 && p.n_bin_dim == 3) return launch_levels<5, 3, MAPPED>(p, s);
    if (p.n_coords == 6 && p.n_bin_dim == 3) return launch_levels<6, 3, MAPPED>(p, s);
    if (p.n_coords == 7 && p.n_bin_dim == 3) return launch_levels<7, 3, MAPPED>(p, s);
    if (p.n_coords == 8 && p.n_bin_dim == 3) return launch_levels<8, 3, MAPPED>(p, s);
    return launch_levels<0, 0, MAPPED>(p, s);
}

}  // namespace

int binned_select_knn_strided(const float *d_coord, const int *d_bin_idx, const int *d_direction,
                              const int *d_dim_bin_idx, const int *d_bin_boundaries, int boundary_shift,
                              const int *d_n_bins, const float *d_bin_width, const int *d_sorting,
                              const float *d_shift, float max_radius, int *d_indices, float *d_dist, int n_vert,
                              int n_neigh, int n_coords, int n_bin_dim, int n_bboundaries, int tf_compat,
                              int use_direction, const int *d_cell_boundaries, int fine_bits,
                              int fine_min_population, hipStream_t s) {
    // same conditions as the reference op (binned_select_knn_kernel.cc:336-352)
    HGC_REQUIRE(n_bin_dim > 1, "BinnedSelectKnnOp expects at least 2 binning dimensions.");
    HGC_REQUIRE(n_bin_dim < 6, "BinnedSelectKnnOp expects maximum 5 binning dimensions.");
    HGC_REQUIRE(n_coords > 1, "BinnedSelectKnnOp expects at least 2 dimensions.");
    HGC_REQUIRE(n_coords >= n_bin_dim, "fewer coordinates than binning dimensions");
    HGC_REQUIRE(n_vert >= 0, "negative number of points");
    HGC_REQUIRE(n_neigh >= 1, "n_neighbours must be positive");
    HGC_REQUIRE((long long)n_vert * n_neigh < (1ll << 31), "n_vert * n_neighbours overflows int32");
    // candidate rows are addressed by 32-bit byte offsets
    HGC_REQUIRE((unsigned long long)n_vert * (unsigned long long)n_coords * sizeof(float) < (1ull << 32),
                "coordinate matrix must stay below 4 GiB");
    HGC_REQUIRE(n_bboundaries >= 2, "bin boundary table too short");
    HGC_REQUIRE(boundary_shift >= 0 && boundary_shift < 8, "bad boundary stride");
    HGC_REQUIRE(fine_bits == 0 || (fine_bits == n_bin_dim && fine_bits <= 4),
                "a nested grid has one bit per binned dimension, four at most");
    if (n_vert == 0) return HGC_OK;
    HGC_REQUIRE(d_coord && d_bin_idx && d_dim_bin_idx && d_bin_boundaries && d_n_bins && d_bin_width &&
                    d_indices && d_dist,
                "null pointer");
    HGC_REQUIRE(!use_direction || d_direction,
                "BinnedSelectKnnOp needs a direction tensor (0,1,2,other) with length nvert if use_direction=True.");
    HGC_REQUIRE((n_coords != 4 && n_coords != 2 && n_coords != 6 && n_coords != 8) ||
                    (reinterpret_cast<uintptr_t>(d_coord) & 15u) == 0,
                "coordinate matrix must be 16-byte aligned");

    KnnParams p;
    p.coord = d_coord;
    p.bin_idx = d_bin_idx;
    p.direction = d_direction;
    p.dim_bin_idx = d_dim_bin_idx;
    p.bin_boundaries = d_bin_boundaries;
    p.n_bins = d_n_bins;
    p.bin_width = d_bin_width;
    p.sorting = d_sorting;
    p.shift = d_shift;
    p.out_idx = d_indices;
    p.out_dist = d_dist;
    p.status = status_word();
    p.radius_sq = max_radius > 0.f ? max_radius * max_radius : -1.f;
    p.n_vert = n_vert;
    p.K = n_neigh;
    p.n_coords = n_coords;
    p.n_bin_dim = n_bin_dim;
    p.n_bboundaries = n_bboundaries;
    p.tf_compat = tf_compat;
    p.use_direction = use_direction;
    p.boundary_shift = boundary_shift;
    p.rank_base = 0;
    p.cell_boundaries = d_cell_boundaries;
    p.fine_bits = fine_bits;
    p.fine_min_population = fine_min_population;
    return d_sorting ? launch_coords<true>(p, s) : launch_coords<false>(p, s);
}

}  // namespace hgc

using namespace hgc;

extern "C" {

int hgc_binned_select_knn_fused(const float *d_coord, const int *d_bin_idx, const int *d_direction,
                                const int *d_dim_bin_idx, const int *d_bin_boundaries,
                                const int *d_n_bins, const float *d_bin_width, const int *d_sorting,
                                const float *d_shift, float max_radius, int *d_indices, float *d_dist, int n_vert, int n_neigh,
                                int n_coords, int n_bin_dim, int n_bboundaries, int tf_compat,
                                int use_direction, hgc_stream_t stream) {
    return binned_select_knn_strided(d_coord, d_bin_idx, d_direction, d_dim_bin_idx, d_bin_boundaries, 0, d_n_bins,
                                     d_bin_width, d_sorting, d_shift, max_radius, d_indices, d_dist, n_vert, n_neigh,
                                     n_coords, n_bin_dim, n_bboundaries, tf_compat, use_direction, nullptr, 0, 0,
                                     as_stream(stream));
}

int hgc_binned_select_knn(const float *d_coord, const int *d_bin_idx, const int *d_direction,
                          const int *d_dim_bin_idx, const int *d_bin_boundaries, const int *d_n_bins,
                          const float *d_bin_width, int *d_indices, float *d_dist, int n_vert, int n_neigh,
                          int n_coords, int n_bin_dim, int n_bboundaries, int tf_compat, int use_direction,
                          hgc_stream_t stream) {
    return hgc_binned_select_knn_fused(d_coord, d_bin_idx, d_direction, d_dim_bin_idx, d_bin_boundaries,
                                       d_n_bins, d_bin_width, nullptr, nullptr, -1.f, d_indices, d_dist, n_vert,
                                       n_neigh, n_coords, n_bin_dim, n_bboundaries, tf_compat, use_direction,
                                       stream);
}

}  // extern "C"
