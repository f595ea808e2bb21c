// Gradient of the GravNet neighbour accumulation (mean and max) from ONE gather
// pass over the inverse neighbour index, with the max part delivered as one
// 32-byte record per (vertex, slot).
//
// Reference behaviour restated here:
//   modules/compiled/accumulate_knn_grad_kernel.cc:36-97   (feature gradient)
//   modules/compiled/accumulate_knn_grad_kernel.cc:99-165  (weight gradient)
//
// Of the N*K*F addends of the feature gradient only N*F carry a max part: feature
// f of vertex v has its maximum at exactly one slot. A first, streaming pass over
// the vertices (hit_records_kernel) turns the arg-max slot table and the max half
// of the upstream gradient into a record per (v, n): the weight w[v,n] and
//   - up to five "hits" (features whose maximum sits at slot n) with their
//     upstream gradients g[v, F+f], or
//   - for a slot with more hits, one bit per feature saying whether it is one.
// The gather pass (one wave per target m, entries (v, n) of m's inverse list in
// ascending order) then needs ONE 32-byte request per entry for everything that
// is specific to the entry, next to the 4*F bytes of the mean half of g[v, :].
// The 64 lanes decode the records of 64 entries at once into a table in LDS; the
// entry loop reads an entry's row of that table with wave-uniform addresses, so
// the few hits of an entry cost one compare and one masked add each instead of
// per-lane slot compares, selects and scattered loads for every entry. The max
// part of an entry's weight gradient is formed by the lane that decodes its
// record, from the target's own feature row in LDS. An entry of the second kind
// fetches the max half of its gradient row in the lanes its bits name.
//
// The addends of the feature gradient and their order are the reference CPU
// kernel's: ((g/K)*w + g_max*w) per entry, entries ascending in (v, n).
#include "accumulate_rows.hpp"

#include <algorithm>

namespace hgc {

namespace {

using namespace acc;

constexpr int kRecordWords = 8;  // 32 bytes
constexpr int kRecordHits = 5;   // hits a record lists
constexpr uint32_t kDense = 0x80;  // header flag: more hits than that, the record holds one bit per feature
constexpr int kRows = 4;    // gathered rows in flight per load batch
constexpr int kGroup = 8;   // entries per cross-lane reduction
constexpr uint32_t kOutOfRange = 0xfffffff0u;  // buffer offset no matrix reaches: the load returns 0
constexpr uint32_t kNoLane = 0xffu;  // key of a hit place that is empty

// Which lane of the gather pass owns feature f, and in which of its registers
// (VEC consecutive features per lane in blocks of 64 * VEC features).
// (vec is 1 or 2: written with shifts, the pass that builds the records gets it at run time)
__host__ __device__ __forceinline__ uint32_t owner_lane(uint32_t f, int vec) { return (f >> (vec - 1)) & (kWave - 1); }
__host__ __device__ __forceinline__ uint32_t owner_reg(uint32_t f, int vec) {
    return ((f >> (5 + vec)) << (vec - 1)) + (f & (uint32_t)(vec - 1));
}

// record of flat slot s at records[2*s], records[2*s+1]:
//   word 0      weight
//   word 1      number of hits (0..5) or kDense | f0 << 8 | f1 << 16 | f2 << 24   (features ascending)
//   listed:     word 2 = f3 | f4 << 8, words 3..7 = g[v, F + f0..f4] (0 where there is no hit)
//   kDense:     words 3..6 = 128 bits, bit 2 * owner_lane(f) + owner_reg(f) set for every hit f

// ---- pass 1: records ---------------------------------------------------------

// the lanes among `active` whose `digit` agrees with this lane's in its low `n_bits` bits
__device__ __forceinline__ uint64_t same_byte_lanes(uint32_t digit, uint64_t active, int n_bits) {
    uint64_t peers = active;
    for (int b = 0; b < n_bits; ++b) {
        const bool set = (digit >> b) & 1u;
        const uint64_t with = __ballot(set);
        peers &= set ? with : ~with;
    }
    return peers;
}

__device__ __forceinline__ int lanes_below(uint64_t mask) {
    return (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
}

// One wave per vertex. Every feature is ranked among the features that share its
// arg-max slot, in feature order (64 features per step: one ballot per slot bit finds
// the lanes with the same slot, a counter per slot in LDS carries the rank from step
// to step), so a slot's hits are listed ascending and nothing depends on the order in
// which lanes or LDS atomics execute. BLOCKS = ceil(F / 64); `vec`: features per
// lane of the gather pass (it fixes the bit positions of a kDense record).
template <int BLOCKS>
__global__ __launch_bounds__(256) void hit_records_kernel(const float *__restrict__ g, const float *__restrict__ w,
                                                          const unsigned char *__restrict__ maxslot,
                                                          uint4 *__restrict__ records, int n_vert, int K, int F,
                                                          int vec) {
    extern __shared__ int s_lists[];  // per wave: count[K], feature[K*5], value[K*5], bits[K*4]
    const int wave = threadIdx.x >> 6, lane = lane_id();
    const int v = blockIdx.x * 4 + wave;
    if (v >= n_vert) return;  // wave-uniform; the kernel has no workgroup barrier
    int *count = s_lists + wave * K * (5 + 2 * kRecordHits);
    int *feature = count + K;
    float *value = reinterpret_cast<float *>(feature + K * kRecordHits);
    unsigned int *bits = reinterpret_cast<unsigned int *>(feature + 2 * K * kRecordHits);
    for (int n = lane; n < K; n += kWave) {
        count[n] = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) bits[4 * n + j] = 0u;
    }
    wave_lds_fence();
    const unsigned char *srow = maxslot + (size_t)v * F;
    const float *grow = g + (size_t)v * 2 * F + F;
    const int slot_bits = 32 - __builtin_clz((unsigned)max(K - 1, 1));
    int slot[BLOCKS], rank[BLOCKS];
    float gv[BLOCKS];
#pragma unroll
    for (int b = 0; b < BLOCKS; ++b) {
        const int f = b * kWave + lane;
        slot[b] = f < F ? (int)srow[f] : 255;
        gv[b] = f < F ? grow[f] : 0.f;
    }
#pragma unroll
    for (int b = 0; b < BLOCKS; ++b) {
        const bool valid = slot[b] < K;  // 255: the feature has no arg-max slot
        const uint64_t peers = same_byte_lanes((uint32_t)slot[b], __ballot(valid), slot_bits);  // valid slots are below K
        const int among = lanes_below(peers);
        const int before = valid ? count[slot[b]] : 0;
        __builtin_amdgcn_wave_barrier();
        if (valid && among == 0) count[slot[b]] = before + (int)__popcll(peers);
        __builtin_amdgcn_wave_barrier();
        rank[b] = valid ? before + among : -1;
    }
    wave_lds_fence();
#pragma unroll
    for (int b = 0; b < BLOCKS; ++b) {
        const uint32_t f = (uint32_t)(b * kWave + lane);
        if (rank[b] >= 0) {
            if (count[slot[b]] > kRecordHits) {
                const uint32_t bit = 2u * owner_lane(f, vec) + owner_reg(f, vec);
                atomicOr(&bits[4 * slot[b] + (bit >> 5)], 1u << (bit & 31u));
            } else {
                feature[slot[b] * kRecordHits + rank[b]] = (int)f;
                value[slot[b] * kRecordHits + rank[b]] = gv[b];
            }
        }
    }
    wave_lds_fence();
    for (int n = lane; n < K; n += kWave) {
        const int c = count[n];
        const bool dense = c > kRecordHits;
        uint32_t ff[kRecordHits];
        float vv[kRecordHits];
#pragma unroll
        for (int j = 0; j < kRecordHits; ++j) {
            const bool live = !dense && j < c;
            ff[j] = live ? (uint32_t)feature[n * kRecordHits + j] : 0u;
            vv[j] = live ? value[n * kRecordHits + j] : 0.f;
        }
        const size_t s = (size_t)v * K + n;
        uint4 r0, r1;
        r0.x = __float_as_uint(w[s]);
        r0.y = (dense ? kDense : (uint32_t)c) | ff[0] << 8 | ff[1] << 16 | ff[2] << 24;
        r0.z = ff[3] | ff[4] << 8;
        r0.w = dense ? bits[4 * n + 0] : __float_as_uint(vv[0]);
        r1.x = dense ? bits[4 * n + 1] : __float_as_uint(vv[1]);
        r1.y = dense ? bits[4 * n + 2] : __float_as_uint(vv[2]);
        r1.z = dense ? bits[4 * n + 3] : __float_as_uint(vv[3]);
        r1.w = __float_as_uint(vv[4]);
        // (2 KB per 64 slots, read back much later by the gather)
        if (n - lane + kWave <= K) {  // wave-uniform: 64 records, written as whole lines --
            // lane i holds bytes [16 i, 16 i + 16) of either half of the 2 KB
            uint4 *block = records + 2 * (s - lane);
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int src = 32 * h + (lane >> 1);
                const bool odd = lane & 1;
                uint4 o;
                const uint32_t a0 = __shfl(r0.x, src, kWave), b0 = __shfl(r1.x, src, kWave);
                const uint32_t a1 = __shfl(r0.y, src, kWave), b1 = __shfl(r1.y, src, kWave);
                const uint32_t a2 = __shfl(r0.z, src, kWave), b2 = __shfl(r1.z, src, kWave);
                const uint32_t a3 = __shfl(r0.w, src, kWave), b3 = __shfl(r1.w, src, kWave);
                o.x = odd ? b0 : a0;
                o.y = odd ? b1 : a1;
                o.z = odd ? b2 : a2;
                o.w = odd ? b3 : a3;
                store_once(block + kWave * h + lane, o);
            }
        } else {
            store_once(records + 2 * s, r0);
            store_once(records + 2 * s + 1, r1);
        }
    }
}

// ---- pass 2: the gather ------------------------------------------------------

// DPP controls (gfx9 encoding)
constexpr int kDppQuadXor1 = 0xb1;    // quad_perm:[1,0,3,2]
constexpr int kDppQuadXor2 = 0x4e;    // quad_perm:[2,3,0,1]
constexpr int kDppRowRor8 = 0x128;    // row_ror:8: lane i of a row of 16 reads lane i ^ 8

template <int CTRL>
__device__ __forceinline__ float dpp_move(float x) {
    return __uint_as_float((uint32_t)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(x), CTRL, 0xf, 0xf, false));
}

// Eight partial sums per lane in; afterwards lane L holds the sum over all 64 lanes of
// value index (L & 7) -- in a fixed order, so the result is deterministic. The values
// are transposed while they are reduced: in the step for index bit h a lane whose bit h
// is clear keeps the values with that bit clear and adds its partner's, the partner does
// the same for the other half. Partners: the mirror image inside 8 lanes (bit 2 differs;
// the bank masks pick the halves, so the step takes two adds per pair of values and no
// select), then lane ^ 2 and lane ^ 1 (quad permutes), then the rows of 16 are summed
// over lane ^ 8 (row rotate), ^ 16 (swizzle) and ^ 32 (permute).
__device__ __forceinline__ float transpose_reduce_group(float (&val)[kGroup]) {
    static_assert(kGroup == 8, "the DPP steps are written for eight values");
    const int lane = lane_id();
    float s4[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
        // s_nop: a DPP operand must not be read within two instructions of the write that made it,
        // and the compiler does not look inside
        asm("s_nop 1\n\t"
            "v_add_f32_dpp %0, %1, %1 row_half_mirror row_mask:0xf bank_mask:0x5\n\t"
            "v_add_f32_dpp %0, %2, %2 row_half_mirror row_mask:0xf bank_mask:0xa"
            : "=&v"(s4[i])
            : "v"(val[i]), "v"(val[i + 4]));
    float s2[2];
    const bool up2 = (lane & 2) != 0, up1 = (lane & 1) != 0;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const float lo = s4[i] + dpp_move<kDppQuadXor2>(s4[i]);
        const float hi = s4[i + 2] + dpp_move<kDppQuadXor2>(s4[i + 2]);
        s2[i] = up2 ? hi : lo;
    }
    const float lo = s2[0] + dpp_move<kDppQuadXor1>(s2[0]);
    const float hi = s2[1] + dpp_move<kDppQuadXor1>(s2[1]);
    float r = up1 ? hi : lo;  // the sum over the lane's 8 lanes of value index (lane & 7)
    r = r + dpp_move<kDppRowRor8>(r);
    r = r + __uint_as_float((uint32_t)__builtin_amdgcn_ds_swizzle((int)__float_as_uint(r), 0x401f));  // lane ^ 16
    r = r + __shfl_xor(r, 32, kWave);
    return r;
}

// The table of a batch of 64 entries in LDS, one wave's share. A row is read with
// a wave-uniform address (every lane receives the same words).
//   head[e]  = { wk or w, owner lanes of hits 0..3 (one byte each, kNoLane: none),
//                owner lane of hit 4, a[4] }
//   pair[e]  = { a[0], b[0], a[1], b[1] }   listed: (a, b)[j] = hit j's addend of the feature gradient
//                                           in the owner's first / second register (one of them is 0)
//              { 128 feature bits }         kDense
//   more[e]  = { a[2], b[2], a[3], b[3] }   listed
//              { weight for the max part }  kDense (0 for a repeated self reference)
//   tail[e]  = b[4], offs[e] = byte offset of the entry's gradient row
template <int Q>
struct BatchTable {
    uint4 head[kWave];
    uint4 pair[kWave];
    uint4 more[kWave];
    uint32_t offs[kWave];
    float tail[kWave];
    float own[Q * kWave];  // the target's own feature row, zero beyond F
};

// part += (a, b) in the lane whose number is byte J of `keys` (wave-uniform): one SDWA compare
// straight into the execution mask, the adds under it. (Written out because the compiler turns
// the same thing into adds in all lanes followed by selects.)
#define HGC_HIT_ASM(BYTE)                                                                              \
    if constexpr (Q == 2)                                                                              \
        asm("v_cmp_eq_u32_sdwa vcc, %3, %4 src0_sel:" BYTE " src1_sel:DWORD\n\t"                       \
            "s_and_saveexec_b64 %2, vcc\n\t"                                                           \
            "v_add_f32 %0, %0, %5\n\t"                                                                 \
            "v_add_f32 %1, %1, %6\n\t"                                                                 \
            "s_mov_b64 exec, %2"                                                                       \
            : "+v"(part[0]), "+v"(part[Q - 1]), "=&s"(saved)                                           \
            : "v"(keys), "v"(lane), "v"(a), "v"(b)                                                     \
            : "vcc", "scc");                                                                                \
    else                                                                                               \
        asm("v_cmp_eq_u32_sdwa vcc, %2, %3 src0_sel:" BYTE " src1_sel:DWORD\n\t"                       \
            "s_and_saveexec_b64 %1, vcc\n\t"                                                           \
            "v_add_f32 %0, %0, %4\n\t"                                                                 \
            "s_mov_b64 exec, %1"                                                                       \
            : "+v"(part[0]), "=&s"(saved)                                                              \
            : "v"(keys), "v"(lane), "v"(a)                                                             \
            : "vcc", "scc")

template <int J, int Q>
__device__ __forceinline__ void add_hit(float (&part)[Q], uint32_t keys, uint32_t lane, float a, float b) {
    uint64_t saved;
    if constexpr (J == 0) { HGC_HIT_ASM("BYTE_0"); }
    else if constexpr (J == 1) { HGC_HIT_ASM("BYTE_1"); }
    else if constexpr (J == 2) { HGC_HIT_ASM("BYTE_2"); }
    else { HGC_HIT_ASM("BYTE_3"); }
    (void)saved;
    (void)b;
}
#undef HGC_HIT_ASM

// An entry whose record is of the kDense kind: the lanes its bits name fetch the max half of
// the gradient row when the entry's turn comes.
template <int VEC, int NB>
__device__ __forceinline__ void dense_entry(const RowMatrix &Gm, const BatchTable<VEC * NB> &tab,
                                            const uint32_t (&lane_bytes)[NB], uint32_t max_col_bytes, int li,
                                            uint32_t soff, const float (&xo)[NB][VEC], float (&part)[VEC * NB],
                                            float &val) {
    const uint32_t lane = (uint32_t)lane_id();
    const uint32_t *words = reinterpret_cast<const uint32_t *>(&tab.pair[li]);
    const uint32_t dbits = (words[lane >> 4] >> (2u * (lane & 15u))) & 3u;  // this lane's two bits of the 128
    float gx[NB][VEC];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        const uint32_t mine = NB == 2 ? (dbits >> b) & 1u : dbits;
        const bool in_row = lane_bytes[b] != kOutOfRange;
        Gm.load_at<VEC>(soff, (mine && in_row) ? lane_bytes[b] + max_col_bytes : kOutOfRange, gx[b]);
    }
    const float sw = __uint_as_float(tab.more[li].x);
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            const int q = b * VEC + e;
            const float gsel = ((dbits >> q) & 1u) ? gx[b][e] : 0.f;
            val = __builtin_fmaf(gsel, xo[b][e], val);
            part[q] = part[q] + gsel * sw;
        }
}

// Entries [c0, c0 + kGroup) of the current batch. FULL: all of them exist.
// Q = registers per lane (VEC * NB, 1 or 2).
template <int VEC, int NB, bool POW2K, bool FULL>
__device__ __forceinline__ void records_group(const RowMatrix &Gm, const BatchTable<VEC * NB> &tab,
                                              const uint32_t (&lane_bytes)[NB], uint32_t max_col_bytes, int c0, int cnt,
                                              uint64_t dense_mask, uint64_t many_mask, const float (&xo)[NB][VEC],
                                              const float (&xk)[NB][VEC], float (&acc)[NB][VEC], float kf,
                                              float (&val)[kGroup]) {
    constexpr int Q = VEC * NB;
    const uint32_t lane = (uint32_t)lane_id();
    const uint32_t dense8 = (uint32_t)(dense_mask >> c0), many8 = (uint32_t)(many_mask >> c0);
#pragma unroll
    for (int h = 0; h < kGroup; h += kRows) {
        uint32_t soff[kRows];
#pragma unroll
        for (int u = 0; u < kRows; ++u)  // the row offset as a scalar: the per-lane offset keeps its range check
            soff[u] = (uint32_t)__builtin_amdgcn_readfirstlane((int)tab.offs[c0 + h + u]);
        float gm[kRows][NB][VEC];
#pragma unroll
        for (int u = 0; u < kRows; ++u)
#pragma unroll
            for (int b = 0; b < NB; ++b) Gm.load_at<VEC>(soff[u], lane_bytes[b], gm[u][b]);
        __builtin_amdgcn_sched_barrier(0);  // all loads of the four are in flight before any arithmetic waits
#pragma unroll
        for (int u = 0; u < kRows; ++u) {
            const int li = c0 + h + u;
            if (!FULL && li >= cnt) break;  // wave-uniform
            const uint4 head = tab.head[li];
            const float swk = __uint_as_float(head.x);
            float part[Q];
#pragma unroll
            for (int b = 0; b < NB; ++b)
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    const float gv = gm[u][b][e];
                    // for a power-of-two K the exact scaling 1/K sits on the weight
                    part[b * VEC + e] = POW2K ? gv * swk : (gv / kf) * swk;
                    val[h + u] = __builtin_fmaf(gv, xk[b][e], val[h + u]);
                }
            if ((dense8 >> (h + u)) & 1u) {
                dense_entry<VEC, NB>(Gm, tab, lane_bytes, max_col_bytes, li, soff[u], xo, part, val[h + u]);
#pragma unroll
                for (int b = 0; b < NB; ++b)
#pragma unroll
                    for (int e = 0; e < VEC; ++e) acc[b][e] = acc[b][e] + part[b * VEC + e];
            } else {
                const uint4 pair = tab.pair[li];
                add_hit<0, Q>(part, head.y, lane, __uint_as_float(pair.x), __uint_as_float(pair.y));
                add_hit<1, Q>(part, head.y, lane, __uint_as_float(pair.z), __uint_as_float(pair.w));
                if ((many8 >> (h + u)) & 1u) {
                    const uint4 more = tab.more[li];
                    add_hit<2, Q>(part, head.y, lane, __uint_as_float(more.x), __uint_as_float(more.y));
                    add_hit<3, Q>(part, head.y, lane, __uint_as_float(more.z), __uint_as_float(more.w));
                    add_hit<0, Q>(part, head.z, lane, __uint_as_float(head.w), tab.tail[li]);
                }
#pragma unroll
                for (int b = 0; b < NB; ++b)
#pragma unroll
                    for (int e = 0; e < VEC; ++e) acc[b][e] = acc[b][e] + part[b * VEC + e];
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    }
}

// PARTIAL: F is not a multiple of 64 (VEC is 1 then); the lanes of the last block
// beyond F stay idle.
template <int VEC, int NB, bool POW2K, bool PARTIAL>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(5, 8))) void accumulate_grad_records_kernel(
    const float *__restrict__ g, const float *__restrict__ feat, const uint4 *__restrict__ records,
    const int *__restrict__ inv_off, const int *__restrict__ inv_slots, float *__restrict__ gw_list,
    float *__restrict__ gfeat, int n_vert, int K, int F, const FastDiv div_k, const int *__restrict__ idx,
    const int *__restrict__ order, const float kf) {
    constexpr int Q = VEC * NB;
    __shared__ BatchTable<Q> s_table[4];
    const int m = wave_vertex(order, n_vert);
    if (m >= n_vert) return;  // wave-uniform; the kernel has no workgroup barrier
    const int lane = lane_id();
    BatchTable<Q> &tab = s_table[threadIdx.x >> 6];
    const float inv_kf = 1.f / kf;  // exact when K is a power of two
    const double inv_kd = 1.0 / (double)kf;
    const int begin = inv_off[m], end = inv_off[m + 1];
    const RowMatrix Gm(g, n_vert, 2 * F);
    const uint32_t max_col_bytes = (uint32_t)F * 4u;
    const uint32_t g_row_bytes = (uint32_t)F * 8u;

    uint32_t lane_bytes[NB];
    float xo[NB][VEC], xk[NB][VEC], acc[NB][VEC];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        const int fb = (b * kWave + lane) * VEC;
        const bool in_row = !PARTIAL || fb < F;
        lane_bytes[b] = in_row ? (uint32_t)fb * 4u : kOutOfRange;
#pragma unroll
        for (int e = 0; e < VEC; ++e) xo[b][e] = 0.f;
        if (in_row) load_vec_once<VEC>(feat + (size_t)m * F + fb, xo[b]);
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            tab.own[fb + e] = xo[b][e];
            // the mean part of a weight gradient is (sum_f g*x) * (1/K) in double, rounded once;
            // here the factor sits on the own row
            xk[b][e] = (float)((double)xo[b][e] * inv_kd);
            acc[b][e] = 0.f;
        }
    }

    // first slot of the target's own row that names the target itself (-1: none);
    // later entries naming it are repeated self references
    int self_key = -1;
    for (int n0 = 0; n0 < K && self_key < 0; n0 += kWave) {
        const int n = n0 + lane;
        const uint64_t is_self = __ballot(n < K && idx[(size_t)m * K + min(n, K - 1)] == m);
        if (is_self != 0) self_key = n0 + __ffsll((unsigned long long)is_self) - 1;
    }
    for (int b0 = begin; b0 < end; b0 += kWave) {
        const int cnt = min(kWave, end - b0);
        const int e = min(b0 + lane, end - 1);
        const int slot_v = inv_slots[e];
        uint4 r0 = records[2 * (size_t)slot_v], r1 = records[2 * (size_t)slot_v + 1];
        const float w_v = __uint_as_float(r0.x);
        const int v = fast_div(slot_v, div_k);
        const int key_v = slot_v - v * K;
        // a repeated self reference takes part in the weight gradient like the first self slot
        // (the reference compares neighbour INDICES there) and carries no max part of the
        // feature gradient
        const bool repeated_self = v == m && key_v != self_key && lane < cnt;
        if (__ballot(repeated_self) != 0) {
            if (repeated_self) {
                const size_t s = (size_t)m * K + self_key;
                r0 = records[2 * s];
                r1 = records[2 * s + 1];
            }
        }
        wave_lds_fence();  // the previous batch's rows have been read, the own row is written
        const bool dense = (r0.y & kDense) != 0;
        const uint32_t n_hits = dense ? 0u : (r0.y & 7u);
        const float gmax[kRecordHits] = {__uint_as_float(r0.w), __uint_as_float(r1.x), __uint_as_float(r1.y),
                                         __uint_as_float(r1.z), __uint_as_float(r1.w)};
        const uint32_t fs[kRecordHits] = {(r0.y >> 8) & 255u, (r0.y >> 16) & 255u, r0.y >> 24, r0.z & 255u,
                                          (r0.z >> 8) & 255u};
        // listed hits: the max part of the entry's weight gradient, sum of g[v, F+f] * feat[m, f],
        // and the hits' addends of the feature gradient in the owner's first / second register
        float max_dot = 0.f;
        float pa[kRecordHits], pb[kRecordHits];
        uint32_t keys[kRecordHits];
#pragma unroll
        for (int j = 0; j < kRecordHits; ++j) {
            const bool live = (uint32_t)j < n_hits;
            const float x = tab.own[live ? fs[j] : 0u];
            max_dot = live ? __builtin_fmaf(gmax[j], x, max_dot) : max_dot;
            const float p = (live && !repeated_self) ? gmax[j] * w_v : 0.f;
            const bool second = owner_reg(fs[j], VEC) != 0;
            pa[j] = second ? 0.f : p;
            pb[j] = second ? p : 0.f;
            keys[j] = live ? owner_lane(fs[j], VEC) : kNoLane;
        }
        tab.offs[lane] = (uint32_t)v * g_row_bytes;
        tab.tail[lane] = pb[4];
        tab.head[lane] = make_uint4(__float_as_uint(POW2K ? w_v * inv_kf : w_v),
                                    keys[0] | keys[1] << 8 | keys[2] << 16 | keys[3] << 24, keys[4],
                                    __float_as_uint(pa[4]));
        tab.pair[lane] = dense ? make_uint4(r0.w, r1.x, r1.y, r1.z)
                               : make_uint4(__float_as_uint(pa[0]), __float_as_uint(pb[0]), __float_as_uint(pa[1]),
                                            __float_as_uint(pb[1]));
        tab.more[lane] = dense ? make_uint4(__float_as_uint(repeated_self ? 0.f : w_v), 0u, 0u, 0u)
                               : make_uint4(__float_as_uint(pa[2]), __float_as_uint(pb[2]), __float_as_uint(pa[3]),
                                            __float_as_uint(pb[3]));
        const uint64_t dense_mask = __ballot(dense && lane < cnt);
        const uint64_t many_mask = __ballot(n_hits > 2u && lane < cnt);
        wave_lds_fence();
        float dot = 0.f;  // lane L: the mean part of entry L's weight gradient
        for (int c0 = 0; c0 < cnt; c0 += kGroup) {
            float val[kGroup];
#pragma unroll
            for (int i = 0; i < kGroup; ++i) val[i] = 0.f;
            if (c0 + kGroup <= cnt)
                records_group<VEC, NB, POW2K, true>(Gm, tab, lane_bytes, max_col_bytes, c0, cnt, dense_mask, many_mask,
                                                    xo, xk, acc, kf, val);
            else
                records_group<VEC, NB, POW2K, false>(Gm, tab, lane_bytes, max_col_bytes, c0, cnt, dense_mask, many_mask,
                                                     xo, xk, acc, kf, val);
            const float r = transpose_reduce_group(val);  // lane L: entry c0 + (L & (kGroup - 1))
            dot = (lane & ~(kGroup - 1)) == c0 ? r : dot;
        }
        // in the order of the inverse list: one run of 4-byte values per target instead of a
        // scattered write per entry (weight_grad_to_table_kernel moves them to their slots)
        if (lane < cnt) gw_list[b0 + lane] = dot + max_dot;
    }
#pragma unroll
    for (int b = 0; b < NB; ++b)
        if (!PARTIAL || lane_bytes[b] != kOutOfRange) store_vec_once<VEC>(gfeat + (size_t)m * F + (lane_bytes[b] >> 2), acc[b]);
}

template <int VEC, int NB, bool PARTIAL>
int launch_records(const float *g, const float *feat, const uint4 *records, const int *inv_off, const int *inv_slots,
                   float *gw_list, float *gfeat, int n_vert, int K, int F, const int *idx, const int *order,
                   float divisor, hipStream_t s) {
    const dim3 grid(ceil_div(n_vert, 4)), block(256);
    const FastDiv div_k = make_fast_div(K);
    const bool pow2k = divisor == (float)(int)divisor && is_pow2((int)divisor);
    if (pow2k)
        accumulate_grad_records_kernel<VEC, NB, true, PARTIAL><<<grid, block, 0, s>>>(
            g, feat, records, inv_off, inv_slots, gw_list, gfeat, n_vert, K, F, div_k, idx, order, divisor);
    else
        accumulate_grad_records_kernel<VEC, NB, false, PARTIAL><<<grid, block, 0, s>>>(
            g, feat, records, inv_off, inv_slots, gw_list, gfeat, n_vert, K, F, div_k, idx, order, divisor);
    return check_launch("accumulate_grad_records_kernel");
}

// ---- pass 3: weight gradients from list order to their slots -------------------

// gw[inv_slots[e]] = gw_list[e] for the entries of all targets, four per thread. The
// scattered 4-byte writes of one stretch of the list fall into the rows of the source
// vertices around it; each XCD works on one contiguous stretch, so the lines stay in
// its L2 until they are full.
__global__ __launch_bounds__(256) void weight_grad_to_table_kernel(const int *__restrict__ inv_off,
                                                                   const int *__restrict__ inv_slots,
                                                                   const float *__restrict__ gw_list,
                                                                   float *__restrict__ gw, int n_vert) {
    const long long n_entries = inv_off[n_vert];
    const long long e0 = ((long long)xcd_contiguous_block(blockIdx.x, gridDim.x) * 256 + threadIdx.x) * 4;
    if (e0 + 4 <= n_entries) {
        const u32x4 slots = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(inv_slots + e0));
        const f32x4 vals = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(gw_list + e0));
        gw[slots.x] = vals.x;
        gw[slots.y] = vals.y;
        gw[slots.z] = vals.z;
        gw[slots.w] = vals.w;
    } else {
        for (long long e = e0; e < n_entries; ++e) gw[inv_slots[e]] = gw_list[e];
    }
}

// features per lane and blocks of 64 lanes of the gather pass for rows of F features; false: not covered
bool records_layout(int F, uintptr_t align_or, int &vec, int &nb) {
    const bool partial = F % kWave != 0;
    vec = partial ? 1 : std::min(2, wave_vec(F, align_or));
    nb = ceil_div(F, kWave * vec);
    return nb >= 1 && vec * nb <= 2;
}

}  // namespace

int launch_zero_padded_weight_grad(const int *inv_off, const int *inv_slots, float *gw, int n_vert, long long total,
                                   hipStream_t s);

static size_t record_bytes(int n_vert, int K) { return align_up((size_t)n_vert * K * kRecordWords * sizeof(uint32_t)); }

// Bytes of storage the record path needs for this shape (the records, then the weight
// gradients in list order), 0 where it does not apply:
// rows of 16 to 128 features addressed through 32-bit buffer offsets, slot bytes (K <= 254).
size_t accumulate_grad_records_bytes(int n_vert, int K, int F) {
    if (n_vert <= 0 || K < 1 || K > 254 || F < 16 || F > 2 * kWave) return 0;
    if ((unsigned long long)n_vert * (unsigned long long)(2 * F) * 4ull >= (1ull << 32)) return 0;
    return record_bytes(n_vert, K) + align_up((size_t)n_vert * K * sizeof(float));
}

// Where the record pass has measured faster than the gather with the slot table (MI355X; banded
// tables and kNN tables of 100 k to 1 M vertices, K = 16..64, F = 32..128): rows wider than K
// features with two hits or fewer per slot on average, 48 neighbours or more, and gathered rows
// that add up to more than the L2 caches keep. (Measured ratios of the two, records / slot bytes:
// K = 64, F = 128: 0.81 on a banded table of 200 k to 1 M vertices, 0.99 on a kNN table of 1 M;
// K = 64, F = 64: 0.93 banded, 1.30 kNN; K = 32: 0.99 to 1.26.)
bool accumulate_grad_records_pays(int n_vert, int K, int F) {
    return accumulate_grad_records_bytes(n_vert, K, F) != 0 && K >= 48 && F > K && F <= 2 * K &&
           (long long)n_vert * F >= (12ll << 20);
}

// Returns 1 when the shape is not covered (the caller then takes another path).
int launch_accumulate_grad_records(const float *g, const float *w, const float *feat, const unsigned char *maxslot,
                                   const int *inv_off, const int *inv_slots, float *gw, float *gfeat, int n_vert, int K,
                                   int F, const int *idx, const int *order, float divisor, void *records,
                                   size_t records_bytes, hipStream_t s) {
    const size_t need = accumulate_grad_records_bytes(n_vert, K, F);
    if (need == 0 || !records || records_bytes < need || !maxslot || !gw || !gfeat) return 1;
    if (((reinterpret_cast<uintptr_t>(records) | reinterpret_cast<uintptr_t>(inv_slots)) & 15u) != 0) return 1;
    const uintptr_t align_or = reinterpret_cast<uintptr_t>(g) | reinterpret_cast<uintptr_t>(feat) |
                               reinterpret_cast<uintptr_t>(gfeat);
    int vec, nb;
    if (!records_layout(F, align_or, vec, nb)) return 1;
    const bool partial = F % kWave != 0;

    uint4 *rec = static_cast<uint4 *>(records);
    float *gw_list = reinterpret_cast<float *>(static_cast<char *>(records) + record_bytes(n_vert, K));
    const size_t lds = (size_t)4 * K * (5 + 2 * kRecordHits) * sizeof(int);
    const dim3 grid(ceil_div(n_vert, 4));
    if (F <= kWave) hit_records_kernel<1><<<grid, 256, lds, s>>>(g, w, maxslot, rec, n_vert, K, F, vec);
    else hit_records_kernel<2><<<grid, 256, lds, s>>>(g, w, maxslot, rec, n_vert, K, F, vec);
    int rc = check_launch("hit_records_kernel");
    if (rc) return rc;
    rc = launch_zero_padded_weight_grad(inv_off, inv_slots, gw, n_vert, (long long)n_vert * K, s);
    if (rc) return rc;
#define HGC_ARGS g, feat, rec, inv_off, inv_slots, gw_list, gfeat, n_vert, K, F, idx, order, divisor, s
    if (partial) rc = nb == 1 ? launch_records<1, 1, true>(HGC_ARGS) : launch_records<1, 2, true>(HGC_ARGS);
    else if (vec == 2) rc = launch_records<2, 1, false>(HGC_ARGS);
    else rc = nb == 1 ? launch_records<1, 1, false>(HGC_ARGS) : launch_records<1, 2, false>(HGC_ARGS);
#undef HGC_ARGS
    if (rc) return rc;
    // the list has at most n_vert * K entries (fewer where slots are padded)
    const long long blocks = ceil_div((long long)n_vert * K, 1024ll);
    weight_grad_to_table_kernel<<<dim3((unsigned)blocks), 256, 0, s>>>(inv_off, inv_slots, gw_list, gw, n_vert);
    return check_launch("weight_grad_to_table_kernel");
}

}  // namespace hgc
