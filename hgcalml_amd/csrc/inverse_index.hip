// Inverse neighbour index: for every vertex m the flat slots v*K+n of the
// neighbour table that name m, ascending. Every gather-instead-of-atomics kernel
// of the library reads it (gradient of the accumulation,
// modules/compiled/accumulate_knn_grad_kernel.cc:36-97; push_knn_kernel.cc:40-62;
// select_knn_grad_kernel.cu.cc:124-164 scatter with atomicAdd where this library
// gathers in a fixed order).
//
// It is a stable sort of the N*K slots by their target. Built here as a two-level
// split written for this problem (HBM-bound integer work, ~30 bytes per slot):
//
//   level 1  targets are cut into tiles of 2^lo_bits consecutive vertices. Every
//            workgroup counts the slots of its stretch of the table per tile
//            (LDS atomics), a scan over (tile, workgroup) turns the counts into
//            positions, and the workgroups move their slots, as (target, slot)
//            records, into tile order -- each wave walks its stretch in order and
//            ranks the 64 slots of a step among the equal tiles of that step with
//            one ballot per tile bit, so the move is stable.
//   level 2  one workgroup per tile sorts the tile's records by target in the same
//            way (count per wave, scan over the tile's targets, ordered walk) into a
//            stage in LDS, from where the tile's slots leave in whole lines.
//
// Slots without a neighbour (index < 0 or >= N) carry the key N and end up
// behind the last vertex's list. Tables with more tiles than the counters of a
// workgroup hold (2^22 vertices and more) take a library radix sort instead.
#include "hgc_common.hpp"

#include <algorithm>
#include <cstring>

#include <rocprim/rocprim.hpp>

namespace hgc {
int launch_fill_i32(int *p, int value, long long n, hipStream_t s);

namespace {

constexpr int kSplitWaves = 4;      // waves per workgroup, level 1
constexpr int kMaxTiles = 4096;     // level 1 counters: 4 waves x 4096 tiles x 4 B = 64 KB of LDS
constexpr int kMinLoBits = 5;
constexpr int kMaxLoBits = 10;      // level 2 counters: (waves + 1) x 2^lo_bits targets x 4 B <= 20 KB of LDS
constexpr int kStage = 32768;       // slots of one tile staged in LDS (128 KB) before they leave in whole lines
constexpr int kTileSlots = 16384;   // slots per tile aimed at: half of what the staging holds
constexpr int kSlotsPerGroup = 32768;
constexpr int kMaxGroups = 512;

struct Plan {
    int lo_bits, tile_bits, n_tiles, n_groups, per_wave;
    bool ok;
};

Plan make_plan(int n_vert, int n_neigh, long long total) {
    Plan p{};
    p.lo_bits = kMinLoBits;
    while (p.lo_bits < kMaxLoBits && ((long long)n_neigh << (p.lo_bits + 1)) <= kTileSlots) ++p.lo_bits;
    while (p.lo_bits < kMaxLoBits && (n_vert >> p.lo_bits) + 1 > kMaxTiles) ++p.lo_bits;
    p.n_tiles = (n_vert >> p.lo_bits) + 1;  // keys run from 0 to n_vert inclusive
    p.ok = p.n_tiles <= kMaxTiles;
    p.tile_bits = 1;
    while ((1 << p.tile_bits) < p.n_tiles) ++p.tile_bits;
    p.n_groups = (int)std::max<long long>(1, std::min<long long>(kMaxGroups, (total + kSlotsPerGroup - 1) / kSlotsPerGroup));
    const long long per = (total + (long long)p.n_groups * kSplitWaves - 1) / ((long long)p.n_groups * kSplitWaves);
    p.per_wave = (int)((per + kWave - 1) / kWave * kWave);
    return p;
}

__device__ __forceinline__ uint32_t slot_key(int j, uint32_t n_vert) { return (uint32_t)j < n_vert ? (uint32_t)j : n_vert; }

// the lanes among `active` whose `digit` agrees with this lane's in its low `bits` bits
__device__ __forceinline__ uint64_t same_digit_lanes(uint32_t digit, int bits, uint64_t active) {
    uint64_t peers = active;
    for (int b = 0; b < bits; ++b) {
        const bool set = (digit >> b) & 1u;
        const uint64_t with = __ballot(set);
        peers &= set ? with : ~with;
    }
    return peers;
}

// LDS accesses of one wave execute in program order; this only keeps the compiler from
// moving them across the point where lanes hand a counter to each other. (A memory fence
// would also wait for the global stores in flight and serialise the walk.)
__device__ __forceinline__ void lds_order_point() { __builtin_amdgcn_wave_barrier(); }

__device__ __forceinline__ int lanes_below(uint64_t mask) {
    return (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
}

// ---- level 1 ---------------------------------------------------------------

constexpr int kAhead = 8;  // steps of 64 slots whose loads are issued together (memory-level parallelism)

// counts[tile * n_groups + group]: slots of the group's stretch that fall into the tile
__global__ __launch_bounds__(kSplitWaves *kWave) void tile_count_kernel(const int *__restrict__ idx, int total,
                                                                        uint32_t n_vert, int lo_bits, int n_tiles,
                                                                        int n_groups, int per_wave,
                                                                        int *__restrict__ counts) {
    extern __shared__ int s_count[];  // [n_tiles]
    for (int t = threadIdx.x; t < n_tiles; t += blockDim.x) s_count[t] = 0;
    __syncthreads();
    const long long first = ((long long)blockIdx.x * kSplitWaves + (threadIdx.x >> 6)) * per_wave;
    const int begin = (int)min(first, (long long)total), end = (int)min(first + per_wave, (long long)total);
    for (int e0 = begin + lane_id(); e0 < end; e0 += kWave * kAhead) {
        int raw[kAhead];  // loads past the end re-read the last slot: no branch, all of them in flight together
#pragma unroll
        for (int a = 0; a < kAhead; ++a) raw[a] = idx[min(e0 + a * kWave, end - 1)];
#pragma unroll
        for (int a = 0; a < kAhead; ++a)
            if (e0 + a * kWave < end) atomicAdd(&s_count[slot_key(raw[a], n_vert) >> lo_bits], 1);
    }
    __syncthreads();
    for (int t = threadIdx.x; t < n_tiles; t += blockDim.x) counts[(size_t)t * n_groups + blockIdx.x] = s_count[t];
    if (blockIdx.x == 0 && threadIdx.x == 0) counts[(size_t)n_tiles * n_groups] = 0;  // the scan's last element
}

// records[position] = (target, flat slot), grouped by tile, flat slots ascending inside a tile
__global__ __launch_bounds__(kSplitWaves *kWave) void tile_move_kernel(const int *__restrict__ idx, int total,
                                                                       uint32_t n_vert, int lo_bits, int tile_bits,
                                                                       int n_tiles, int n_groups, int per_wave,
                                                                       const int *__restrict__ starts,
                                                                       uint2 *__restrict__ records) {
    extern __shared__ int s_cursor[];  // [kSplitWaves][n_tiles]
    const int wave = threadIdx.x >> 6, lane = lane_id();
    for (int t = threadIdx.x; t < n_tiles * kSplitWaves; t += blockDim.x) s_cursor[t] = 0;
    __syncthreads();
    int *const mine = s_cursor + wave * n_tiles;
    const long long first = ((long long)blockIdx.x * kSplitWaves + wave) * per_wave;
    const int begin = (int)min(first, (long long)total), end = (int)min(first + per_wave, (long long)total);
    for (int e0 = begin + lane; e0 < end; e0 += kWave * kAhead) {
        int raw[kAhead];
#pragma unroll
        for (int a = 0; a < kAhead; ++a) raw[a] = idx[min(e0 + a * kWave, end - 1)];
#pragma unroll
        for (int a = 0; a < kAhead; ++a)
            if (e0 + a * kWave < end) atomicAdd(&mine[slot_key(raw[a], n_vert) >> lo_bits], 1);
    }
    __syncthreads();
    // first position of every (wave, tile): the group's start in the tile, then wave after wave
    for (int t = threadIdx.x; t < n_tiles; t += blockDim.x) {
        int at = starts[(size_t)t * n_groups + blockIdx.x];
#pragma unroll
        for (int w = 0; w < kSplitWaves; ++w) {
            const int c = s_cursor[w * n_tiles + t];
            s_cursor[w * n_tiles + t] = at;
            at += c;
        }
    }
    __syncthreads();
    for (int c0 = begin; c0 < end; c0 += kWave * kAhead) {  // wave-uniform
        int raw[kAhead];
#pragma unroll
        for (int a = 0; a < kAhead; ++a) raw[a] = idx[min(c0 + a * kWave + lane, end - 1)];
#pragma unroll
        for (int a = 0; a < kAhead; ++a) {
            if (c0 + a * kWave >= end) break;  // wave-uniform
            const int e = c0 + a * kWave + lane;
            const bool valid = e < end;
            const uint32_t key = slot_key(raw[a], n_vert);
            const uint32_t tile = valid ? key >> lo_bits : 0u;
            const uint64_t peers = same_digit_lanes(tile, tile_bits, __ballot(valid));
            const int rank = lanes_below(peers);
            int at = 0;
            if (valid) at = mine[tile];
            lds_order_point();
            if (valid && rank == 0) mine[tile] = at + (int)__popcll(peers);
            lds_order_point();
            if (valid) records[(size_t)at + rank] = make_uint2(key, (uint32_t)e);
        }
    }
}

// ---- level 2 ---------------------------------------------------------------

// One workgroup per tile. The tile's slots leave through a stage in LDS, so that global memory
// sees whole lines instead of one 4-byte write per slot; a tile with more slots than the stage
// holds writes them one by one.
// waves per workgroup of level 2: as many as the counters leave room for next to the stage
constexpr int sort_waves(int lo_bits) { return lo_bits <= 8 ? 16 : lo_bits == 9 ? 8 : 4; }

template <int LO_BITS>
__global__ __launch_bounds__(sort_waves(LO_BITS) * kWave) void tile_sort_kernel(const uint2 *__restrict__ records,
                                                                      const int *__restrict__ starts, int n_groups,
                                                                      uint32_t n_vert, int *__restrict__ inv_offsets,
                                                                      int *__restrict__ inv_slots) {
    constexpr int T = 1 << LO_BITS;
    constexpr int kSortWaves = sort_waves(LO_BITS);
    __shared__ int s_cursor[kSortWaves][T];
    __shared__ int s_total[T];
    __shared__ int s_stage[kStage];
    const int wave = threadIdx.x >> 6, lane = lane_id();
    const int tile = blockIdx.x;
    const int begin_tile = starts[(size_t)tile * n_groups], end_tile = starts[(size_t)(tile + 1) * n_groups];
    const bool staged = end_tile - begin_tile <= kStage;
    for (int t = threadIdx.x; t < T * kSortWaves; t += blockDim.x) (&s_cursor[0][0])[t] = 0;
    __syncthreads();
    const int per_wave = ((end_tile - begin_tile + kSortWaves - 1) / kSortWaves + kWave - 1) / kWave * kWave;
    const int begin = min(begin_tile + wave * per_wave, end_tile), end = min(begin + per_wave, end_tile);
    for (int e0 = begin + lane; e0 < end; e0 += kWave * kAhead) {
        uint32_t key[kAhead];
#pragma unroll
        for (int a = 0; a < kAhead; ++a) key[a] = records[min(e0 + a * kWave, end - 1)].x;
#pragma unroll
        for (int a = 0; a < kAhead; ++a)
            if (e0 + a * kWave < end) atomicAdd(&s_cursor[wave][key[a] & (T - 1)], 1);
    }
    __syncthreads();
    // per target: the waves' counts become their first positions inside the target's list
    for (int t = threadIdx.x; t < T; t += blockDim.x) {
        int at = 0;
#pragma unroll
        for (int w = 0; w < kSortWaves; ++w) {
            const int c = s_cursor[w][t];
            s_cursor[w][t] = at;
            at += c;
        }
        s_total[t] = at;
    }
    __syncthreads();
    if (wave == 0) {  // exclusive scan of the list lengths over the tile's targets
        int carry = 0;
        for (int t0 = 0; t0 < T; t0 += kWave) {
            const int len = s_total[t0 + lane];
            const int incl = wave_inclusive_sum(len);
            s_total[t0 + lane] = carry + incl - len;
            carry += readlane_i32(incl, kWave - 1);
        }
    }
    __syncthreads();
    const uint32_t first_target = (uint32_t)tile << LO_BITS;
    for (int t = threadIdx.x; t < T; t += blockDim.x) {
        const int at = s_total[t];  // relative to the tile's first slot
        if (first_target + t <= n_vert) inv_offsets[first_target + t] = begin_tile + at;  // entry n_vert: the slots without a neighbour
#pragma unroll
        for (int w = 0; w < kSortWaves; ++w) s_cursor[w][t] += at;
    }
    __syncthreads();
    for (int c0 = begin; c0 < end; c0 += kWave * kAhead) {  // wave-uniform
        uint2 rec[kAhead];
#pragma unroll
        for (int a = 0; a < kAhead; ++a) rec[a] = records[min(c0 + a * kWave + lane, end - 1)];
#pragma unroll
        for (int a = 0; a < kAhead; ++a) {
            if (c0 + a * kWave >= end) break;  // wave-uniform
            const bool valid = c0 + a * kWave + lane < end;
            const uint32_t t = rec[a].x & (T - 1);
            const uint64_t peers = same_digit_lanes(t, LO_BITS, __ballot(valid));
            const int rank = lanes_below(peers);
            int at = 0;
            if (valid) at = s_cursor[wave][t];
            lds_order_point();
            if (valid && rank == 0) s_cursor[wave][t] = at + (int)__popcll(peers);
            lds_order_point();
            if (valid) {
                if (staged) s_stage[at + rank] = (int)rec[a].y;
                else inv_slots[(size_t)begin_tile + at + rank] = (int)rec[a].y;
            }
        }
    }
    if (!staged) return;
    __syncthreads();
    for (int i = threadIdx.x; i < end_tile - begin_tile; i += blockDim.x) inv_slots[(size_t)begin_tile + i] = s_stage[i];
}

// ---- library sort, for tables beyond the two-level split ---------------------

struct InverseKey {
    unsigned n_vert;
    __host__ __device__ unsigned operator()(int j) const { return (unsigned)j < n_vert ? (unsigned)j : n_vert; }
};

__global__ __launch_bounds__(256) void inverse_offsets_kernel(const unsigned int *__restrict__ sorted_keys,
                                                              long long total, int *__restrict__ offsets, int n_vert) {
    const int m = blockIdx.x * blockDim.x + threadIdx.x;
    if (m > n_vert) return;
    long long lo = 0, hi = total;  // first position whose key is >= m
    while (lo < hi) {
        long long mid = (lo + hi) >> 1;
        if (sorted_keys[mid] < (unsigned)m)
            lo = mid + 1;
        else
            hi = mid;
    }
    offsets[m] = (int)lo;
}

int inverse_key_bits(int n_vert) {
    int bits = 1;
    while (bits < 32 && (1ll << bits) <= (long long)n_vert) ++bits;  // keys go up to n_vert inclusive
    return bits;
}

size_t library_sort_bytes(size_t total, int n_vert) {
    size_t temp = 0;
    (void)rocprim::radix_sort_pairs(nullptr, temp, rocprim::make_transform_iterator((const int *)nullptr, InverseKey{1u}),
                                    (unsigned int *)nullptr, rocprim::counting_iterator<int>(0), (int *)nullptr, total, 0,
                                    inverse_key_bits(std::max(n_vert, 1)), (hipStream_t) nullptr);
    return align_up(temp) + align_up(total * sizeof(int));
}

size_t scan_bytes(size_t n) {
    size_t temp = 0;
    (void)rocprim::exclusive_scan(nullptr, temp, (const int *)nullptr, (int *)nullptr, 0, n, rocprim::plus<int>(),
                                  (hipStream_t) nullptr);
    return align_up(temp);
}

size_t split_bytes(const Plan &p, size_t total) {
    const size_t cells = (size_t)p.n_tiles * p.n_groups + 1;
    return align_up(total * sizeof(uint2)) + 2 * align_up(cells * sizeof(int)) + scan_bytes(cells);
}

}  // namespace
}  // namespace hgc

using namespace hgc;

extern "C" {

size_t hgc_inverse_neighbour_index_workspace_bytes(int n_vert, int n_neigh) {
    const size_t total = std::max<size_t>((size_t)std::max(n_vert, 0) * std::max(n_neigh, 0), 1);
    const Plan plan = make_plan(std::max(n_vert, 1), std::max(n_neigh, 1), (long long)total);
    return plan.ok ? split_bytes(plan, total) : library_sort_bytes(total, n_vert);
}

int hgc_inverse_neighbour_index(const int *d_idxs, int n_vert, int n_neigh, int *d_inv_offsets, int *d_inv_slots,
                                void *workspace, size_t workspace_bytes, hgc_stream_t stream) {
    HGC_REQUIRE(n_vert >= 0 && n_neigh >= 1, "bad sizes");
    HGC_REQUIRE((long long)n_vert * n_neigh < (1ll << 31), "n_vert * n_neigh overflows int32");
    HGC_REQUIRE(d_inv_offsets, "null pointer");
    hipStream_t s = as_stream(stream);
    if (n_vert == 0) return launch_fill_i32(d_inv_offsets, 0, 1, s);
    HGC_REQUIRE(d_idxs && d_inv_slots, "null pointer");
    if (!workspace || !aligned256(workspace) ||
        workspace_bytes < hgc_inverse_neighbour_index_workspace_bytes(n_vert, n_neigh))
        return fail(HGC_ERR_WORKSPACE, "inverse_neighbour_index workspace missing, misaligned or too small");
    const long long total = (long long)n_vert * n_neigh;
    const Plan plan = make_plan(n_vert, n_neigh, total);
    Carver carve(workspace);

    if (!plan.ok) {
        // Keys and values are generated on the fly: key = the slot's target (invalid
        // ones sort last), value = the flat slot itself. Stable: inside one target the
        // flat slots stay ascending, i.e. (vertex, slot) order.
        unsigned int *keys_sorted = carve.take<unsigned int>(total);
        void *temp = carve.base + carve.used;
        size_t temp_bytes = workspace_bytes - carve.used;
        const auto keys_in = rocprim::make_transform_iterator(d_idxs, InverseKey{(unsigned)n_vert});
        const rocprim::counting_iterator<int> slots_in(0);
        HGC_HIP(rocprim::radix_sort_pairs(temp, temp_bytes, keys_in, keys_sorted, slots_in, d_inv_slots, (size_t)total,
                                          0, inverse_key_bits(n_vert), s));
        inverse_offsets_kernel<<<ceil_div((long long)n_vert + 1, 256), 256, 0, s>>>(keys_sorted, total, d_inv_offsets,
                                                                                    n_vert);
        return check_launch("inverse_offsets");
    }

    const size_t cells = (size_t)plan.n_tiles * plan.n_groups + 1;
    uint2 *records = carve.take<uint2>(total);
    int *counts = carve.take<int>(cells);
    int *starts = carve.take<int>(cells);
    void *temp = carve.base + carve.used;
    size_t temp_bytes = workspace_bytes - carve.used;
    const dim3 split_block(kSplitWaves * kWave);
    tile_count_kernel<<<plan.n_groups, split_block, plan.n_tiles * sizeof(int), s>>>(
        d_idxs, (int)total, (uint32_t)n_vert, plan.lo_bits, plan.n_tiles, plan.n_groups, plan.per_wave, counts);
    int rc = check_launch("tile_count");
    if (rc) return rc;
    HGC_HIP(rocprim::exclusive_scan(temp, temp_bytes, counts, starts, 0, cells, rocprim::plus<int>(), s));
    tile_move_kernel<<<plan.n_groups, split_block, (size_t)plan.n_tiles * kSplitWaves * sizeof(int), s>>>(
        d_idxs, (int)total, (uint32_t)n_vert, plan.lo_bits, plan.tile_bits, plan.n_tiles, plan.n_groups, plan.per_wave, starts,
        records);
    if ((rc = check_launch("tile_move"))) return rc;
#define HGC_TILE_SORT(B)                                                                                       \
    case B:                                                                                                    \
        tile_sort_kernel<B><<<plan.n_tiles, sort_waves(B) * kWave, 0, s>>>(records, starts, plan.n_groups,    \
                                                                           (uint32_t)n_vert, d_inv_offsets,    \
                                                                           d_inv_slots);                       \
        break
    switch (plan.lo_bits) {
        HGC_TILE_SORT(5);
        HGC_TILE_SORT(6);
        HGC_TILE_SORT(7);
        HGC_TILE_SORT(8);
        HGC_TILE_SORT(9);
        HGC_TILE_SORT(10);
    }
#undef HGC_TILE_SORT
    return check_launch("tile_sort");
}

}  // extern "C"
