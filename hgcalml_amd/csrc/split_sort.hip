// Stable sort of integer keys from a known range -- a counting sort in two
// levels, written for the index tables of this library (HBM-bound integer work):
// the inverse neighbour index (keys: the target of every slot of the neighbour
// table), the hits in bin order (keys: flat bin index) and the condensates'
// selection order (keys: pieces of the beta ordering).
//
//   level 1  keys are cut into tiles of 2^lo_bits consecutive values. Every
//            workgroup counts the items of its stretch of the input per tile (LDS
//            atomics), a scan over (tile, workgroup) turns the counts into
//            positions, and the workgroups move their items, as (key, value)
//            records, into tile order -- each wave walks its stretch in order and
//            ranks the 64 items of a step among the equal tiles of that step with
//            one ballot per tile bit, so the move is stable.
//   level 2  one workgroup per tile sorts the tile's records by key in the same
//            way (count per wave, scan over the tile's keys, ordered walk) into a
//            stage in LDS, from where the tile's values leave in whole lines,
//            together with the first position of every key.
//
// Items whose key lies outside [0, n_keys) carry the key n_keys and end up last.
#include "hgc_common.hpp"

#include <algorithm>
#include <cstring>

#include <rocprim/rocprim.hpp>

namespace hgc {
namespace {

constexpr int kSplitWaves = 4;      // waves per workgroup, level 1
constexpr int kMaxTiles = 8192;     // level 1 counters: 4 waves x 8192 tiles x 4 B = 128 KB of LDS
constexpr int kMinLoBits = 5;
constexpr int kMaxLoBits = 10;      // level 2 counters: (waves + 1) x 2^lo_bits keys x 4 B <= 20 KB of LDS
constexpr int kStage = 32768;       // values of one tile staged in LDS (128 KB) before they leave in whole lines
constexpr int kTileItems = 16384;   // items per tile aimed at: half of what the staging holds
constexpr int kMinItemsPerGroup = 4096;
constexpr int kMaxGroups = 512;
constexpr int kWantedTiles = 512;   // small key ranges are cut finer, so that level 2 has workgroups to spread

struct Plan {
    int lo_bits, tile_bits, n_tiles, n_groups, per_wave;
    bool ok;
};

Plan make_plan(long long total, int n_keys, int per_key) {
    Plan p{};
    p.lo_bits = kMinLoBits;
    while (p.lo_bits < kMaxLoBits && ((long long)std::max(per_key, 1) << (p.lo_bits + 1)) <= kTileItems &&
           (n_keys >> (p.lo_bits + 1)) >= kWantedTiles)
        ++p.lo_bits;
    while (p.lo_bits < kMaxLoBits && (n_keys >> p.lo_bits) + 1 > kMaxTiles) ++p.lo_bits;
    p.n_tiles = (n_keys >> p.lo_bits) + 1;  // keys run from 0 to n_keys inclusive
    p.ok = p.n_tiles <= kMaxTiles && total < (1ll << 31);
    p.tile_bits = 1;
    while ((1 << p.tile_bits) < p.n_tiles) ++p.tile_bits;
    const long long per_group = std::max<long long>(kMinItemsPerGroup, (total + kMaxGroups - 1) / kMaxGroups);
    p.n_groups = (int)std::max<long long>(1, (total + per_group - 1) / per_group);
    const long long per = (total + (long long)p.n_groups * kSplitWaves - 1) / ((long long)p.n_groups * kSplitWaves);
    p.per_wave = (int)((per + kWave - 1) / kWave * kWave);
    return p;
}

__device__ __forceinline__ uint32_t clamp_key(int k, uint32_t n_keys) { return (uint32_t)k < n_keys ? (uint32_t)k : n_keys; }

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

constexpr int kAhead = 8;  // steps of 64 items whose loads are issued together (memory-level parallelism)

// item i has the key keys[values ? values[i] : i] and the value values ? values[i] : i
template <bool INDIRECT>
__device__ __forceinline__ void load_items(const int *__restrict__ keys, const int *__restrict__ values, int first,
                                           int last, int (&key)[kAhead], int (&value)[kAhead]) {
    // loads past the end re-read the last item: no branch, all of them in flight together
#pragma unroll
    for (int a = 0; a < kAhead; ++a) {
        const int i = min(first + a * kWave, last);
        value[a] = INDIRECT ? values[i] : i;
    }
#pragma unroll
    for (int a = 0; a < kAhead; ++a) key[a] = keys[value[a]];
}

// counts[tile * n_groups + group]: items of the group's stretch that fall into the tile
template <bool INDIRECT>
__global__ __launch_bounds__(kSplitWaves *kWave) void tile_count_kernel(const int *__restrict__ keys,
                                                                        const int *__restrict__ values, int total,
                                                                        uint32_t n_keys, int lo_bits, int n_tiles,
                                                                        int n_groups, int per_wave,
                                                                        int *__restrict__ counts) {
    extern __shared__ int s_count[];  // [n_tiles]
    for (int t = threadIdx.x; t < n_tiles; t += blockDim.x) s_count[t] = 0;
    __syncthreads();
    const long long first = ((long long)blockIdx.x * kSplitWaves + (threadIdx.x >> 6)) * per_wave;
    const int begin = (int)min(first, (long long)total), end = (int)min(first + per_wave, (long long)total);
    for (int e0 = begin + lane_id(); e0 < end; e0 += kWave * kAhead) {
        int raw[kAhead], val[kAhead];
        load_items<INDIRECT>(keys, values, e0, end - 1, raw, val);
#pragma unroll
        for (int a = 0; a < kAhead; ++a)
            if (e0 + a * kWave < end) atomicAdd(&s_count[clamp_key(raw[a], n_keys) >> lo_bits], 1);
    }
    __syncthreads();
    for (int t = threadIdx.x; t < n_tiles; t += blockDim.x) counts[(size_t)t * n_groups + blockIdx.x] = s_count[t];
    if (blockIdx.x == 0 && threadIdx.x == 0) counts[(size_t)n_tiles * n_groups] = 0;  // the scan's last element
}

// records[position] = (key, value), grouped by tile, in input order inside a tile
template <bool INDIRECT>
__global__ __launch_bounds__(kSplitWaves *kWave) void tile_move_kernel(const int *__restrict__ keys,
                                                                       const int *__restrict__ values, int total,
                                                                       uint32_t n_keys, int lo_bits, int tile_bits,
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
        int raw[kAhead], val[kAhead];
        load_items<INDIRECT>(keys, values, e0, end - 1, raw, val);
#pragma unroll
        for (int a = 0; a < kAhead; ++a)
            if (e0 + a * kWave < end) atomicAdd(&mine[clamp_key(raw[a], n_keys) >> lo_bits], 1);
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
        int raw[kAhead], val[kAhead];
        load_items<INDIRECT>(keys, values, c0 + lane, end - 1, raw, val);
#pragma unroll
        for (int a = 0; a < kAhead; ++a) {
            if (c0 + a * kWave >= end) break;  // wave-uniform
            const int e = c0 + a * kWave + lane;
            const bool valid = e < end;
            const uint32_t key = clamp_key(raw[a], n_keys);
            const uint32_t tile = valid ? key >> lo_bits : 0u;
            const uint64_t peers = same_digit_lanes(tile, tile_bits, __ballot(valid));
            const int rank = lanes_below(peers);
            int at = 0;
            if (valid) at = mine[tile];
            lds_order_point();
            if (valid && rank == 0) mine[tile] = at + (int)__popcll(peers);
            lds_order_point();
            if (valid) records[(size_t)at + rank] = make_uint2(key, (uint32_t)val[a]);
        }
    }
}

// ---- level 2 ---------------------------------------------------------------

// One workgroup per tile. The tile's values leave through a stage in LDS, so that global memory
// sees whole lines instead of one 4-byte write per slot; a tile with more items than the stage
// holds writes them one by one.
// waves per workgroup of level 2: as many as the counters leave room for next to the stage
constexpr int sort_waves(int lo_bits) { return lo_bits <= 8 ? 16 : lo_bits == 9 ? 8 : 4; }

template <int LO_BITS>
__global__ __launch_bounds__(sort_waves(LO_BITS) * kWave) void tile_sort_kernel(const uint2 *__restrict__ records,
                                                                      const int *__restrict__ starts, int n_groups,
                                                                      uint32_t n_keys, int *__restrict__ offsets,
                                                                      int *__restrict__ order) {
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
    // per key: the waves' counts become their first positions inside the key's run
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
    if (wave == 0) {  // exclusive scan of the run lengths over the tile's keys
        int carry = 0;
        for (int t0 = 0; t0 < T; t0 += kWave) {
            // a tile of fewer keys than the wave has lanes (T = 32): the lanes beyond it stay out of the table
            const bool in_table = t0 + lane < T;
            const int len = in_table ? s_total[t0 + lane] : 0;
            const int incl = wave_inclusive_sum(len);
            if (in_table) s_total[t0 + lane] = carry + incl - len;
            carry += readlane_i32(incl, kWave - 1);
        }
    }
    __syncthreads();
    const uint32_t first_target = (uint32_t)tile << LO_BITS;
    for (int t = threadIdx.x; t < T; t += blockDim.x) {
        const int at = s_total[t];  // relative to the tile's first item
        // entry n_keys: where the items without a valid key begin
        if (offsets && first_target + t <= n_keys) offsets[first_target + t] = begin_tile + at;
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
                else order[(size_t)begin_tile + at + rank] = (int)rec[a].y;
            }
        }
    }
    if (!staged) return;
    __syncthreads();
    for (int i = threadIdx.x; i < end_tile - begin_tile; i += blockDim.x) order[(size_t)begin_tile + i] = s_stage[i];
}


size_t scan_bytes(size_t n) {
    size_t temp = 0;
    (void)rocprim::exclusive_scan(nullptr, temp, (const int *)nullptr, (int *)nullptr, 0, n, rocprim::plus<int>(),
                                  (hipStream_t) nullptr);
    return align_up(temp);
}

}  // namespace

bool stable_key_sort_supported(long long total, int n_keys, int per_key_hint) {
    return n_keys >= 1 && make_plan(std::max<long long>(total, 1), n_keys, per_key_hint).ok;
}

size_t stable_key_sort_workspace_bytes(long long total, int n_keys, int per_key_hint) {
    total = std::max<long long>(total, 1);
    const Plan p = make_plan(total, std::max(n_keys, 1), per_key_hint);
    const size_t cells = (size_t)p.n_tiles * p.n_groups + 1;
    return align_up((size_t)total * sizeof(uint2)) + 2 * align_up(cells * sizeof(int)) + scan_bytes(cells);
}

int stable_key_sort(const int *d_keys, const int *d_values, long long total, int n_keys, int per_key_hint,
                    int *d_offsets, int *d_order, void *workspace, size_t workspace_bytes, hipStream_t s) {
    if (total <= 0) return d_offsets ? launch_fill_i32(d_offsets, 0, (long long)n_keys + 1, s) : HGC_OK;
    const Plan plan = make_plan(total, n_keys, per_key_hint);
    if (!plan.ok) return fail(HGC_ERR_UNSUPPORTED, "key range too wide for the two-level sort");
    if (!workspace || !aligned256(workspace) ||
        workspace_bytes < stable_key_sort_workspace_bytes(total, n_keys, per_key_hint))
        return fail(HGC_ERR_WORKSPACE, "sort workspace missing, misaligned or too small");
    Carver carve(workspace);
    const size_t cells = (size_t)plan.n_tiles * plan.n_groups + 1;
    uint2 *records = carve.take<uint2>(total);
    int *counts = carve.take<int>(cells);
    int *starts = carve.take<int>(cells);
    void *temp = carve.base + carve.used;
    size_t temp_bytes = workspace_bytes - carve.used;
    const dim3 split_block(kSplitWaves * kWave);
    if (d_values)
        tile_count_kernel<true><<<plan.n_groups, split_block, plan.n_tiles * sizeof(int), s>>>(
            d_keys, d_values, (int)total, (uint32_t)n_keys, plan.lo_bits, plan.n_tiles, plan.n_groups, plan.per_wave,
            counts);
    else
        tile_count_kernel<false><<<plan.n_groups, split_block, plan.n_tiles * sizeof(int), s>>>(
            d_keys, d_values, (int)total, (uint32_t)n_keys, plan.lo_bits, plan.n_tiles, plan.n_groups, plan.per_wave,
            counts);
    int rc = check_launch("tile_count");
    if (rc) return rc;
    HGC_HIP(rocprim::exclusive_scan(temp, temp_bytes, counts, starts, 0, cells, rocprim::plus<int>(), s));
    const size_t move_lds = (size_t)plan.n_tiles * kSplitWaves * sizeof(int);
    if (d_values)
        tile_move_kernel<true><<<plan.n_groups, split_block, move_lds, s>>>(
            d_keys, d_values, (int)total, (uint32_t)n_keys, plan.lo_bits, plan.tile_bits, plan.n_tiles, plan.n_groups,
            plan.per_wave, starts, records);
    else
        tile_move_kernel<false><<<plan.n_groups, split_block, move_lds, s>>>(
            d_keys, d_values, (int)total, (uint32_t)n_keys, plan.lo_bits, plan.tile_bits, plan.n_tiles, plan.n_groups,
            plan.per_wave, starts, records);
    if ((rc = check_launch("tile_move"))) return rc;
#define HGC_TILE_SORT(B)                                                                                          \
    case B:                                                                                                       \
        tile_sort_kernel<B><<<plan.n_tiles, sort_waves(B) * kWave, 0, s>>>(records, starts, plan.n_groups,       \
                                                                           (uint32_t)n_keys, d_offsets, d_order); \
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

}  // namespace hgc
