// GravNet neighbour accumulation: weighted mean and max over K neighbours
// (forward) and its gradients w.r.t. weights and features.
//
// Reference behaviour restated here:
//   modules/compiled/accumulate_knn_kernel.cc:48-81       (forward)
//   modules/compiled/accumulate_knn_grad_kernel.cc:24-165 (gradients)
//
// Roofline: HBM. Algorithmic bytes per vertex: forward 4*(2K + 4F)
// (indices, weights, features in, mean|max and arg-max out), gradient
// 4*(3K + 5F). The K-fold re-read of feature / gradient rows is a gather that
// must be served by L2 / Infinity Cache, not HBM.
//
// Layout: consecutive lanes hold consecutive features of one vertex (float4
// per lane when F % 4 == 0), so every gathered row is one coalesced request.
// The forward and the feature gradient add their terms in exactly the
// reference CPU order (slot order, resp. ascending (vertex, slot) per target
// through the inverse neighbour index), which makes them bit-identical to it;
// no float atomics anywhere.
#include "accumulate_rows.hpp"

#include <cstdlib>
#include <cstring>
#include <algorithm>

#include <rocprim/rocprim.hpp>

namespace hgc {

int launch_fill_i32(int *p, int value, long long n, hipStream_t s);
// accumulate_grad_fused.hip; returns 1 when the shape is not covered. gw == nullptr:
// feature gradient only (feat and idx are then not read).
int launch_accumulate_grad_fused(const float *g, const float *w, const float *feat, const int *maxidx,
                                 const unsigned char *maxslot, const int *inv_off, const int *inv_slots, float *gw,
                                 float *gfeat, int n_vert, int K, int F, int g_cols, bool mean_and_max, const int *idx,
                                 const int *order, float divisor, hipStream_t s);
// accumulate_grad_records.hip: both gradients with the max part read from per-slot
// records built in `records`; returns 1 when the shape is not covered or the storage is
// too small (accumulate_grad_records_bytes is 0 where the path does not apply).
size_t accumulate_grad_records_bytes(int n_vert, int K, int F);
bool accumulate_grad_records_pays(int n_vert, int K, int F);
int launch_accumulate_grad_records(const float *g, const float *w, const float *feat, const unsigned char *maxslot,
                                   const int *inv_off, const int *inv_slots, float *gw, float *gfeat, int n_vert, int K,
                                   int F, const int *idx, const int *order, float divisor, void *records,
                                   size_t records_bytes, hipStream_t s);

namespace {

using namespace acc;

// ------------------------------------------------------------------ forward


constexpr int kUnroll = 8;

// one thread per (vertex, VEC consecutive features); threads of one vertex are
// adjacent lanes
template <int VEC, bool MAX>
__global__ __launch_bounds__(256) void accumulate_fwd_kernel(const float *__restrict__ w, const float *__restrict__ feat,
                                                             const int *__restrict__ idx, float *__restrict__ out,
                                                             int *__restrict__ out_maxidx,
                                                             unsigned char *__restrict__ out_maxslot, int n_vert, int K,
                                                             int F, int out_cols, float kf) {
    const int tpv = F / VEC;  // threads per vertex
    const long long t = (long long)xcd_contiguous_block(blockIdx.x, gridDim.x) * blockDim.x + threadIdx.x;
    const int v = (int)(t / tpv);
    if (v >= n_vert) return;
    const int f0 = (int)(t - (long long)v * tpv) * VEC;

    const int *irow = idx + (size_t)v * K;
    const float *wrow = w + (size_t)v * K;
    float sum[VEC], best[VEC];
    int arg[VEC], aslot[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
        sum[e] = 0.f;
        best[e] = 0.f;
        arg[e] = 0;
        aslot[e] = -1;
    }

    for (int n0 = 0; n0 < K; n0 += kUnroll) {
        int j[kUnroll];
        float wn[kUnroll];
        float x[kUnroll][VEC];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const int n = n0 + u;
            j[u] = n < K ? irow[n] : -1;
            wn[u] = n < K ? wrow[n] : 0.f;
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const bool ok = (unsigned)j[u] < (unsigned)n_vert;
            load_vec<VEC>(feat + (size_t)(ok ? j[u] : 0) * F + f0, x[u]);
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const bool ok = (unsigned)j[u] < (unsigned)n_vert;
            const bool first = (n0 + u) == 0;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const float wf = x[u][e] * wn[u];
                const float s = sum[e] + wf;
                sum[e] = ok ? s : sum[e];
                if (MAX) {
                    const bool take = ok && (wf >= best[e] || first);
                    best[e] = take ? wf : best[e];
                    arg[e] = take ? j[u] : arg[e];
                    aslot[e] = take ? n0 + u : aslot[e];
                }
            }
        }
    }

    float mean[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) mean[e] = sum[e] / kf;
    store_vec<VEC>(out + (size_t)v * out_cols + f0, mean);
    if (MAX) {
        store_vec<VEC>(out + (size_t)v * out_cols + F + f0, best);
        store_vec_i<VEC>(out_maxidx + (size_t)v * F + f0, arg);
        if (out_maxslot) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                int sl = aslot[e];
                if (sl > 0 && arg[e] == v) {  // repeated self reference: report its first slot
                    for (int n = 0; n < sl; ++n)
                        if (irow[n] == v) {
                            sl = n;
                            break;
                        }
                }
                if (sl < 0) {  // no maximum: index 0 is reported, the slot that names vertex 0 is credited
                    for (int n = 0; n < K; ++n)
                        if (irow[n] == 0) {
                            sl = n;
                            break;
                        }
                }
                out_maxslot[(size_t)v * F + f0 + e] = (unsigned char)(sl < 0 ? 255 : sl);
            }
        }
    }
}


// ================================================================== wave-per-vertex kernels (F >= 64)
//
// One wave64 owns one vertex; lane l owns features [l*VEC, l*VEC+VEC) of every
// block of 64*VEC features. The vertex index is wave-uniform, so the neighbour
// indices and weights of its row come in through scalar loads, and gathered
// rows are fetched with buffer loads whose address is
//   descriptor base + scalar row offset + per-lane column offset,
// i.e. no vector ALU is spent on addressing. The scalar row offset is not part
// of the hardware's range check, so every row index is validated on the scalar
// side before it is used. Chunks of U neighbour slots without
// padding take a branch-free path with all U row loads in flight.


// one slot of the forward recurrence for the VEC features of this lane
template <int VEC, bool MAX, bool SEED>
__device__ __forceinline__ void fwd_slot(const float (&x)[VEC], float wn, int slot, float (&sum)[VEC],
                                         float (&best)[VEC], int (&arg)[VEC]) {
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
        const float wf = x[e] * wn;
        sum[e] = sum[e] + wf;
        if (MAX) {
            if (SEED) {  // slot 0 always seeds the maximum
                best[e] = wf;
                arg[e] = slot;
            } else {
                const bool take = wf >= best[e];  // ">=": a later slot wins ties
                best[e] = take ? wf : best[e];
                arg[e] = take ? slot : arg[e];
            }
        }
    }
}

// Up to U slots [n_begin, n_end) of a vertex's row where some have no neighbour,
// or the short last chunk of a row: index and weight of slot n_begin + l sit in
// lane l and are broadcast with v_readlane (no arrays of scalars to keep alive),
// all rows are in flight together, a slot without a neighbour fetches row 0 and
// is skipped. Returns n_begin so that the caller's loop advances as for a full chunk.
// (EXPW: the row's weights wait in LDS, w_lds[n] for slot n.)
template <int VEC, bool MAX, int U, bool EXPW>
__device__ __forceinline__ int partial_chunk(const RowMatrix &X, const int *__restrict__ irow,
                                             const float *__restrict__ wrow, const float *w_lds, int n_begin, int n_end,
                                             int n_vert, uint32_t lane_bytes, float (&sum)[VEC], float (&best)[VEC],
                                             int (&arg)[VEC]) {
    const int lane = lane_id();
    const int n_mine = min(n_begin + lane, n_end - 1);
    const int j_lane = n_begin + lane < n_end ? irow[n_mine] : -1;
    const float w_lane = EXPW ? 0.f : wrow[n_mine];
    const uint64_t valid = __ballot((uint32_t)j_lane < (uint32_t)n_vert);  // bit l: slot n_begin + l has a neighbour
    float x[U][VEC];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int j = __builtin_amdgcn_readlane(j_lane, u);
        X.load<VEC>((valid >> u) & 1ull ? j : 0, lane_bytes, x[u]);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        if (!((valid >> u) & 1ull)) continue;  // wave-uniform
        const float w = EXPW ? w_lds[n_begin + u]
                             : __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(w_lane), u));
        if (n_begin + u == 0)
            fwd_slot<VEC, MAX, true>(x[u], w, 0, sum, best, arg);
        else
            fwd_slot<VEC, MAX, false>(x[u], w, n_begin + u, sum, best, arg);
    }
    return n_begin;
}

// EXPW (rows of 64 slots or fewer): `w` holds distances; lane n turns the distance of slot n into
// the weight exp(-d) (modules/accknn_op.py:52, there a framework op of its own in front of the
// kernel), writes it to w_out for the gradient and to LDS, from where every lane reads the slots'
// weights (same address in all lanes) instead of the scalar loads.
template <int VEC, bool MAX, bool EXPW>
__global__ __launch_bounds__(256) void accumulate_fwd_wave_kernel(const float *__restrict__ w,
                                                                  const float *__restrict__ feat,
                                                                  const int *__restrict__ idx, float *__restrict__ out,
                                                                  int *__restrict__ out_maxidx,
                                                                  unsigned char *__restrict__ out_maxslot, int n_vert,
                                                                  int K, int F, int out_cols, float kf,
                                                                  const int *__restrict__ order,
                                                                  float *__restrict__ w_out) {
    constexpr int U = VEC == 4 ? 8 : 16;
    const int v = wave_vertex(order, n_vert);
    if (v >= n_vert) return;
    const int *irow = idx + (size_t)v * K;
    const float *wrow = w + (size_t)v * K;
    __shared__ float s_weights[EXPW ? 4 : 1][kWave];
    const float *w_lds = s_weights[EXPW ? threadIdx.x >> 6 : 0];
    if (EXPW) {
        const int n = lane_id();
        float w_n = 0.f;
        if (n < K) {
            w_n = expf(-wrow[n]);
            w_out[(size_t)v * K + n] = w_n;
        }
        s_weights[threadIdx.x >> 6][n] = w_n;
        wave_lds_fence();
    }
    const RowMatrix X(feat, n_vert, F);
    int first_self = -1;  // first slot that names the vertex itself (wave-uniform, scalar ALU)

    for (int fb = lane_id() * VEC; fb < F; fb += kWave * VEC) {
        const uint32_t lane_bytes = (uint32_t)fb * 4u;
        float sum[VEC], best[VEC];
        int arg[VEC];  // SLOT of the maximum, -1: none (translated to an index at the end)
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            sum[e] = 0.f;
            best[e] = 0.f;
            arg[e] = -1;
        }
        int n0 = 0;
        for (; n0 + U <= K; n0 += U) {
            int j[U];
            float wn[U];
            float x[U][VEC];
            uint32_t j_max = 0;  // unsigned: a negative index is the largest
#pragma unroll
            for (int u = 0; u < U; ++u) {
                j[u] = irow[n0 + u];
                wn[u] = EXPW ? w_lds[n0 + u] : wrow[n0 + u];
                j_max = max(j_max, (uint32_t)j[u]);
            }
            const bool all_valid = j_max < (uint32_t)n_vert;
            if (MAX) {
                int fs = -1;
#pragma unroll
                for (int u = U - 1; u >= 0; --u)
                    if (j[u] == v) fs = n0 + u;
                if (first_self < 0) first_self = fs;
            }
            if (all_valid) {  // wave-uniform: the common, padding-free chunk
#pragma unroll
                for (int u = 0; u < U; ++u) X.load<VEC>(j[u], lane_bytes, x[u]);
                if (n0 == 0) {
                    fwd_slot<VEC, MAX, true>(x[0], wn[0], 0, sum, best, arg);
#pragma unroll
                    for (int u = 1; u < U; ++u) fwd_slot<VEC, MAX, false>(x[u], wn[u], u, sum, best, arg);
                } else {
#pragma unroll
                    for (int u = 0; u < U; ++u) fwd_slot<VEC, MAX, false>(x[u], wn[u], n0 + u, sum, best, arg);
                }
            } else {
                n0 = partial_chunk<VEC, MAX, U, EXPW>(X, irow, wrow, w_lds, n0, n0 + U, n_vert, lane_bytes, sum, best,
                                                      arg);
            }
        }
        if (n0 < K) {  // K not a multiple of U
            if (MAX) {
                const int n_mine = min(n0 + lane_id(), K - 1);
                const uint64_t self = __ballot(n0 + lane_id() < K && irow[n_mine] == v);
                if (first_self < 0 && self) first_self = n0 + __builtin_ctzll(self);
            }
            if (K - n0 <= 4)
                partial_chunk<VEC, MAX, 4, EXPW>(X, irow, wrow, w_lds, n0, K, n_vert, lane_bytes, sum, best, arg);
            else if (K - n0 <= 8 || U == 8)
                partial_chunk<VEC, MAX, 8, EXPW>(X, irow, wrow, w_lds, n0, K, n_vert, lane_bytes, sum, best, arg);
            else
                partial_chunk<VEC, MAX, 16, EXPW>(X, irow, wrow, w_lds, n0, K, n_vert, lane_bytes, sum, best, arg);
        }
        float mean[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) mean[e] = sum[e] / kf;
        store_vec_once<VEC>(out + (size_t)v * out_cols + fb, mean);
        if (MAX) {
            store_vec_once<VEC>(out + (size_t)v * out_cols + F + fb, best);
            int argidx[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) argidx[e] = arg[e] < 0 ? 0 : irow[arg[e]];
            store_vec_i<VEC>(out_maxidx + (size_t)v * F + fb, argidx);
            if (out_maxslot) {
                // slot of the maximum; for a repeated self reference its first slot,
                // which is the one the reference's gradient credits. A feature without a
                // maximum (slot 0 empty, every product negative) reports index 0, and the
                // reference's gradient compares indices: it credits the slot that names
                // vertex 0, if the row has one.
                bool none = false;
#pragma unroll
                for (int e = 0; e < VEC; ++e) none = none || arg[e] < 0;
                int first_zero = -1;
                if (__ballot(none) != 0) {  // wave-uniform, rare
                    for (int n0z = 0; n0z < K && first_zero < 0; n0z += kWave) {
                        const int n = n0z + lane_id();
                        const uint64_t zero = __ballot(n < K && irow[min(n, K - 1)] == 0);
                        if (zero != 0) first_zero = n0z + __builtin_ctzll(zero);
                    }
                }
                uint32_t packed = 0;
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    int sl = arg[e];
                    if (sl < 0) sl = first_zero;
                    else if (argidx[e] == v) sl = first_self;
                    packed |= (uint32_t)(sl < 0 ? 255 : sl) << (8 * e);
                }
                unsigned char *dst = out_maxslot + (size_t)v * F + fb;
                if constexpr (VEC == 4) *reinterpret_cast<uint32_t *>(dst) = packed;
                else if constexpr (VEC == 2) *reinterpret_cast<uint16_t *>(dst) = (uint16_t)packed;
                else *dst = (unsigned char)packed;
            }
        }
    }
}


// one inverse-list entry of the feature gradient for the VEC features of this lane;
// `mi` holds arg-max indices compared with `key` = target vertex, or (SLOTS)
// arg-max slots compared with `key` = slot of this entry
template <int VEC, bool MAX, bool POW2K>
__device__ __forceinline__ void fgrad_entry(const float (&gm)[VEC], const float (&gx)[VEC], const int (&mi)[VEC],
                                            float wv, int key, bool count_max, float kf, float inv_k,
                                            float (&acc)[VEC]) {
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
        float part = POW2K ? gm[e] * inv_k : gm[e] / kf;
        part = part * wv;
        float part_max = 0.f;
        if (MAX) {
            const float pmx = gx[e] * wv;
            part_max = (mi[e] == key && count_max) ? pmx : 0.f;
        }
        const float add = part + part_max;
        acc[e] = acc[e] + add;
    }
}


// Feature slicing across XCDs: the rows this kernel gathers (gradient row +
// arg-max row of every vertex that names the target) span a window of the
// neighbour band times ~1.5 KB, more than one XCD's 4 MB L2 holds. With
// n_slices == 2 even XCDs work on the even 64*VEC-feature blocks of every row
// and odd XCDs on the odd ones, so each L2 caches only half of every row.
// (Workgroups are dealt round-robin to the 8 XCDs; a different dispatch order
// would only cost speed, not correctness.)
template <int VEC, bool MAX, bool POW2K, bool SLOTS>
__global__ __launch_bounds__(256) void feature_grad_wave_kernel(const float *__restrict__ g, const float *__restrict__ w,
                                                                const int *__restrict__ maxidx,
                                                                const unsigned char *__restrict__ maxslot,
                                                                const int *__restrict__ inv_off,
                                                                const int *__restrict__ inv_slots,
                                                                float *__restrict__ gfeat, int n_vert, int K, int F,
                                                                int g_cols, const FastDiv div_k, int n_slices, float kf,
                                                                const int *__restrict__ order) {
    constexpr int U = VEC == 4 ? 4 : 8;
    int m, first_block = 0;
    if (n_slices == 1) {
        m = wave_vertex(order, n_vert);
    } else {
        const int xcd = blockIdx.x % kNumXcd, seq = blockIdx.x / kNumXcd;
        const int per_xcd = gridDim.x / kNumXcd;
        first_block = xcd % n_slices;
        const int tile = (xcd / n_slices) * per_xcd + seq;
        const int i = __builtin_amdgcn_readfirstlane(tile * 4 + (int)(threadIdx.x >> 6));
        m = i < n_vert ? (order ? __builtin_amdgcn_readfirstlane(order[i]) : i) : n_vert;
    }
    if ((uint32_t)m >= (uint32_t)n_vert) return;
    const float inv_k = 1.f / kf;  // exact when the divisor is a power of two
    const int begin = inv_off[m], end = inv_off[m + 1];
    const RowMatrix G(g, n_vert, g_cols);
    const RowMatrix MI(maxidx, (MAX && !SLOTS) ? n_vert : 0, F);
    const __amdgpu_buffer_rsrc_t MS = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<unsigned char *>(maxslot), 0, (MAX && SLOTS) ? (int)(uint32_t)((size_t)n_vert * F) : 0, 0x00020000);
    const uint32_t max_col_bytes = (uint32_t)F * 4u;

    for (int fb = (first_block * kWave + lane_id()) * VEC; fb < F; fb += n_slices * kWave * VEC) {
        const uint32_t lane_bytes = (uint32_t)fb * 4u;
        float acc[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[e] = 0.f;
        bool self_seen = false;  // repeated self references carry the max part once
        if (begin < end) {
            // The scalar side (inverse-list slots, then the weights they address) runs
            // one chunk ahead of the vector side so that its latency is hidden behind
            // the row gathers. Entries past the end are clamped to the last one and
            // skipped in the arithmetic.
            const int last = end - 1;
            int slot_cur[U], slot_nxt[U];
            float w_cur[U];
#pragma unroll
            for (int u = 0; u < U; ++u) slot_cur[u] = inv_slots[min(begin + u, last)];
#pragma unroll
            for (int u = 0; u < U; ++u) w_cur[u] = w[slot_cur[u]];
#pragma unroll
            for (int u = 0; u < U; ++u) slot_nxt[u] = inv_slots[min(begin + U + u, last)];

            for (int e0 = begin; e0 < end; e0 += U) {
                int v[U], key[U];
                float gm[U][VEC], gx[U][VEC];
                int mi[U][VEC];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    v[u] = fast_div(slot_cur[u], div_k);
                    key[u] = SLOTS ? slot_cur[u] - v[u] * K : m;
                }
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    G.load<VEC>(v[u], lane_bytes, gm[u]);
                    if (MAX) {
                        if (SLOTS) {
                            load_slots<VEC>(MS, v[u], (uint32_t)F, (uint32_t)fb, mi[u]);
                        } else {
                            MI.load<VEC>(v[u], lane_bytes, mi[u]);
                            G.load<VEC>(v[u], lane_bytes + max_col_bytes, gx[u]);
                        }
                    }
                }
                // scalar prefetch for the next two chunks
                float w_nxt[U];
                int slot_nn[U];
#pragma unroll
                for (int u = 0; u < U; ++u) w_nxt[u] = w[slot_nxt[u]];
#pragma unroll
                for (int u = 0; u < U; ++u) slot_nn[u] = inv_slots[min(e0 + 2 * U + u, last)];

                if (MAX && SLOTS) {
                    // the max half of a gradient row is fetched only by the lanes whose
                    // feature has its maximum at this entry (about F/K lanes per row)
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        bool any = false;
#pragma unroll
                        for (int e = 0; e < VEC; ++e) {
                            any = any || mi[u][e] == key[u];
                            gx[u][e] = 0.f;
                        }
                        if (any) G.load<VEC>(v[u], lane_bytes + max_col_bytes, gx[u]);
                    }
                }
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    if (e0 + u >= end) break;  // wave-uniform
                    bool count_max = true;
                    if (!SLOTS && v[u] == m) {  // (the slot table already points at the first self slot)
                        count_max = !self_seen;
                        self_seen = true;
                    }
                    fgrad_entry<VEC, MAX, POW2K>(gm[u], gx[u], mi[u], w_cur[u], key[u], count_max, kf, inv_k, acc);
                }
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    slot_cur[u] = slot_nxt[u];
                    w_cur[u] = w_nxt[u];
                    slot_nxt[u] = slot_nn[u];
                }
            }
        }
        store_vec<VEC>(gfeat + (size_t)m * F + fb, acc);
    }
}


template <int VEC, bool MAX>
__global__ __launch_bounds__(256) void weight_grad_wave_kernel(const float *__restrict__ g, const float *__restrict__ feat,
                                                               const int *__restrict__ maxidx, const int *__restrict__ idx,
                                                               float *__restrict__ gw, int n_vert, int K, int F,
                                                               int g_cols, float kf,
                                                               const int *__restrict__ order) {
    constexpr int U = 8;
    constexpr int G = 16;  // slots per reduction group: 16 mean sums + 16 max sums = 32 values
    const int m = wave_vertex(order, n_vert);
    if (m >= n_vert) return;
    const int lane = lane_id();
    const int *irow = idx + (size_t)m * K;
    const double inv_k = 1.0 / (double)kf;
    const RowMatrix X(feat, n_vert, F);

    for (int l0 = 0; l0 < K; l0 += G) {
        float val[2 * G];
#pragma unroll
        for (int i = 0; i < 2 * G; ++i) val[i] = 0.f;
        for (int fb = lane * VEC; fb < F; fb += kWave * VEC) {
            const uint32_t lane_bytes = (uint32_t)fb * 4u;
            float gm[VEC], gx[VEC];
            int mi[VEC];
            load_vec<VEC>(g + (size_t)m * g_cols + fb, gm);
            if (MAX) {
                load_vec<VEC>(g + (size_t)m * g_cols + F + fb, gx);
                load_vec_i<VEC>(maxidx + (size_t)m * F + fb, mi);
            }
#pragma unroll
            for (int u0 = 0; u0 < G; u0 += U) {
                int j[U];
                float x[U][VEC];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int l = l0 + u0 + u;
                    j[u] = l < K ? irow[l] : -1;
                }
                // slots without a neighbour read row 0; an index outside [0, n_vert)
                // can never equal an arg-max index of a valid row, and the slot's
                // result is overwritten with 0 below
#pragma unroll
                for (int u = 0; u < U; ++u)
                    X.load<VEC>((uint32_t)j[u] < (uint32_t)n_vert ? j[u] : 0, lane_bytes, x[u]);
#pragma unroll
                for (int u = 0; u < U; ++u) {
#pragma unroll
                    for (int e = 0; e < VEC; ++e) {
                        val[u0 + u] = __builtin_fmaf(gm[e], x[u][e], val[u0 + u]);
                        if (MAX) {
                            const float t = __builtin_fmaf(gx[e], x[u][e], val[G + u0 + u]);
                            val[G + u0 + u] = (mi[e] == j[u]) ? t : val[G + u0 + u];
                        }
                    }
                }
            }
        }
        const float r = transpose_reduce_32(val);        // lanes 0..15 (mod 32): mean sums, 16..31: max sums
        const float r_max = __shfl_xor(r, 16, kWave);    // lane < 16 receives its max sum
        const int l = l0 + lane;
        if (lane < G && l < K) {
            const int j = irow[l];
            const bool ok = (unsigned)j < (unsigned)n_vert;
            const float mean = (float)((double)r * inv_k);
            gw[(size_t)m * K + l] = ok ? mean + r_max : 0.f;
        }
    }
}

// ------------------------------------------------------------------ inverse index

// The inverse index of a neighbour table without its first column, from the inverse
// index of the whole table: the entries of column 0 leave every target's list and
// flat slot v*K+n becomes v*(K-1)+n-1. One wave per target, its list across the lanes.
__global__ __launch_bounds__(256) void first_column_entries_kernel(const int *__restrict__ inv_off,
                                                                   const int *__restrict__ inv_slots, int n_vert,
                                                                   const acc::FastDiv div_k, int K,
                                                                   int *__restrict__ dropped) {
    const int m = blockIdx.x * (blockDim.x / kWave) + (int)(threadIdx.x / kWave);
    if (m > n_vert) return;
    int count = 0;
    if (m < n_vert) {
        const int begin = inv_off[m], end = inv_off[m + 1];
        for (int e = begin + lane_id(); e - lane_id() < end; e += kWave) {
            const int slot = e < end ? inv_slots[e] : 1;
            count += __popcll(__ballot(e < end && slot - acc::fast_div(slot, div_k) * K == 0));
        }
    }
    if (lane_id() == 0) dropped[m] = count;
}

__global__ __launch_bounds__(256) void drop_first_column_kernel(const int *__restrict__ inv_off,
                                                                const int *__restrict__ inv_slots,
                                                                const int *__restrict__ dropped_before, int n_vert,
                                                                const acc::FastDiv div_k, int K,
                                                                int *__restrict__ out_off,
                                                                int *__restrict__ out_slots) {
    const int m = blockIdx.x * (blockDim.x / kWave) + (int)(threadIdx.x / kWave);
    if (m > n_vert) return;
    int at = inv_off[m] - dropped_before[m];
    if (lane_id() == 0) out_off[m] = at;
    if (m == n_vert) return;
    const int begin = inv_off[m], end = inv_off[m + 1];
    for (int e = begin + lane_id(); e - lane_id() < end; e += kWave) {
        const int slot = e < end ? inv_slots[e] : 0;
        const int v = acc::fast_div(slot, div_k), n = slot - v * K;
        const bool keep = e < end && n != 0;
        const uint64_t kept = __ballot(keep);
        if (keep) out_slots[at + __popcll(kept & ((1ull << lane_id()) - 1ull))] = v * (K - 1) + n - 1;
        at += __popcll(kept);
    }
}

// ------------------------------------------------------------------ feature gradient

// gfeat[m, f] = sum over (v, n) naming m, ascending, of ((g[v,f]/K)*w[v,n] + max part)
template <int VEC, bool MAX, bool POW2K>
__global__ __launch_bounds__(256) void feature_grad_kernel(const float *__restrict__ g, const float *__restrict__ w,
                                                           const int *__restrict__ maxidx,
                                                           const int *__restrict__ inv_off,
                                                           const int *__restrict__ inv_slots,
                                                           float *__restrict__ gfeat, int n_vert, int K, int F,
                                                           int g_cols, float kf) {
    const int tpv = F / VEC;
    const long long t = (long long)xcd_contiguous_block(blockIdx.x, gridDim.x) * blockDim.x + threadIdx.x;
    const int m = (int)(t / tpv);
    if (m >= n_vert) return;
    const int f0 = (int)(t - (long long)m * tpv) * VEC;

    const float inv_k = 1.f / kf;  // exact when the divisor is a power of two
    float acc[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc[e] = 0.f;
    bool self_seen = false;

    const int begin = inv_off[m], end = inv_off[m + 1];
    constexpr int U = 4;
    for (int e0 = begin; e0 < end; e0 += U) {
        int slot[U], v[U];
        float wv[U];
        float gm[U][VEC], gx[U][VEC];
        int mi[U][VEC];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const bool live = e0 + u < end;
            slot[u] = live ? inv_slots[e0 + u] : 0;
            v[u] = live ? slot[u] / K : -1;
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int vv = v[u] < 0 ? 0 : v[u];
            wv[u] = w[slot[u]];
            load_vec<VEC>(g + (size_t)vv * g_cols + f0, gm[u]);
            if (MAX) {
                if constexpr (VEC == 4) {
                    const int4 q = *reinterpret_cast<const int4 *>(maxidx + (size_t)vv * F + f0);
                    mi[u][0] = q.x; mi[u][1] = q.y; mi[u][2] = q.z; mi[u][3] = q.w;
                } else {
                    mi[u][0] = maxidx[(size_t)vv * F + f0];
                }
                bool any = false;
#pragma unroll
                for (int e = 0; e < VEC; ++e) any = any || mi[u][e] == m;
                if (any) {
                    load_vec<VEC>(g + (size_t)vv * g_cols + F + f0, gx[u]);
                } else {
#pragma unroll
                    for (int e = 0; e < VEC; ++e) gx[u][e] = 0.f;
                }
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (v[u] < 0) continue;
            bool count_max = true;
            if (v[u] == m) {  // repeated self references carry the max part once
                count_max = !self_seen;
                self_seen = true;
            }
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                float part = POW2K ? gm[u][e] * inv_k : gm[u][e] / kf;
                part = part * wv[u];
                float part_max = 0.f;
                if (MAX) {
                    if (mi[u][e] == m && count_max) part_max = gx[u][e] * wv[u];
                }
                const float add = part + part_max;
                acc[e] = acc[e] + add;
            }
        }
    }
    store_vec<VEC>(gfeat + (size_t)m * F + f0, acc);
}

// ------------------------------------------------------------------ weight gradient

// gw[m, l] = (sum_f g[m,f]*feat[j,f]) / K + sum_f [j == maxidx[m,f]] g[m,F+f]*feat[j,f]
// The threads of one vertex each own VEC features; per neighbour slot they form
// their partial dot products and combine them with a butterfly over the lanes
// of the vertex. TPV (threads per vertex) must be a power of two <= 64.
template <int VEC, bool MAX>
__global__ __launch_bounds__(256) void weight_grad_kernel(const float *__restrict__ g, const float *__restrict__ feat,
                                                          const int *__restrict__ maxidx, const int *__restrict__ idx,
                                                          float *__restrict__ gw, int n_vert, int K, int F, int g_cols,
                                                          int tpv, float kf) {
    const long long t = (long long)xcd_contiguous_block(blockIdx.x, gridDim.x) * blockDim.x + threadIdx.x;
    const int m = (int)(t / tpv);
    const int sub = (int)(t - (long long)m * tpv);
    const bool live = m < n_vert;  // keep whole waves alive for the shuffles
    const int mm = live ? m : 0;

    // features owned by this thread: f = sub*VEC + e + i*tpv*VEC
    const int stride = tpv * VEC;
    const int *irow = idx + (size_t)mm * K;
    const double inv_k = 1.0 / (double)kf;

    for (int l0 = 0; l0 < K; l0 += kUnroll) {
        float pm[kUnroll], px[kUnroll];
        int j[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            j[u] = (l0 + u) < K ? irow[l0 + u] : -1;
            pm[u] = 0.f;
            px[u] = 0.f;
        }
        for (int fb = sub * VEC; fb < F; fb += stride) {
            float gm[VEC], gx[VEC];
            int mi[VEC];
            load_vec<VEC>(g + (size_t)mm * g_cols + fb, gm);
            if (MAX) {
                load_vec<VEC>(g + (size_t)mm * g_cols + F + fb, gx);
                if constexpr (VEC == 4) {
                    const int4 q = *reinterpret_cast<const int4 *>(maxidx + (size_t)mm * F + fb);
                    mi[0] = q.x; mi[1] = q.y; mi[2] = q.z; mi[3] = q.w;
                } else {
                    mi[0] = maxidx[(size_t)mm * F + fb];
                }
            }
            float x[kUnroll][VEC];
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) {
                const bool ok = (unsigned)j[u] < (unsigned)n_vert;
                load_vec<VEC>(feat + (size_t)(ok ? j[u] : 0) * F + fb, x[u]);
            }
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) {
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    pm[u] = pm[u] + gm[e] * x[u][e];
                    if (MAX) {
                        const float term = gx[e] * x[u][e];
                        px[u] = (mi[e] == j[u]) ? px[u] + term : px[u];
                    }
                }
            }
        }
        // butterfly over the tpv lanes of this vertex
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            for (int off = tpv >> 1; off > 0; off >>= 1) {
                pm[u] += __shfl_xor(pm[u], off, kWave);
                if (MAX) px[u] += __shfl_xor(px[u], off, kWave);
            }
        }
        if (live && sub == 0) {
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) {
                if (l0 + u < K) {
                    const bool ok = (unsigned)j[u] < (unsigned)n_vert;
                    const float mean = (float)((double)pm[u] * inv_k);
                    gw[(size_t)m * K + l0 + u] = ok ? mean + px[u] : 0.f;
                }
            }
        }
    }
}

}  // namespace
}  // namespace hgc

namespace hgc {

// Forward pass shared by accumulate_knn (divisor = K) and the feature gradient of
// push_knn (divisor = 1): out = (sum over the slots of w * feat[idx]) / divisor.
// d_out_weights == nullptr: d_distances are the weights. Otherwise they are distances, the weights
// exp(-d) are used and written to d_out_weights.
int accumulate_forward(const float *d_distances, const float *d_feat, const int *d_idxs, float *d_out_feat,
                       int *d_out_maxidxs, unsigned char *d_out_maxslots, int n_vert, int n_neigh, int n_feat,
                       int n_out_feat, int mean_and_max, float divisor, const int *d_order, float *d_out_weights,
                       hgc_stream_t stream) {
    HGC_REQUIRE(n_vert >= 0 && n_neigh >= 1 && n_feat >= 1, "bad sizes");
    HGC_REQUIRE(n_out_feat == n_feat * (mean_and_max ? 2 : 1), "n_out_feat must be n_feat * (mean_and_max ? 2 : 1)");
    // slots are numbered with 32 bits; matrices of any size (beyond 4 GiB: the thread-per-element kernels with
    // 64-bit offsets)
    HGC_REQUIRE((long long)n_vert * n_neigh < (1ll << 31), "n_vert * n_neigh must stay below 2^31");
    if (n_vert == 0) return HGC_OK;
    HGC_REQUIRE(d_distances && d_feat && d_idxs && d_out_feat, "null pointer");
    HGC_REQUIRE(!mean_and_max || d_out_maxidxs, "mean_and_max needs d_out_maxidxs");
    HGC_REQUIRE(!d_out_maxslots || n_neigh <= 254, "arg-max slots are bytes: n_neigh <= 254");
    hipStream_t s = as_stream(stream);
    const uintptr_t align_or = reinterpret_cast<uintptr_t>(d_feat) | reinterpret_cast<uintptr_t>(d_out_feat) |
                              reinterpret_cast<uintptr_t>(d_out_maxidxs);
    // the wave kernels address rows through 32-bit buffer offsets
    const bool fits_32bit = (unsigned long long)n_vert * (unsigned long long)n_out_feat * 4ull < (1ull << 32);
    const bool wave_kernel = n_feat >= 16 && fits_32bit;
    const bool exp_in_kernel = d_out_weights && wave_kernel && n_neigh <= kWave;
    if (d_out_weights && !exp_in_kernel) {  // the weights in a pass of their own, then as if they had been given
        const int rc = hgc_exp_neg(d_distances, d_out_weights, (long long)n_vert * n_neigh, stream);
        if (rc) return rc;
        d_distances = d_out_weights;
    }
    if (wave_kernel) {  // one wave per vertex (lanes beyond a short row stay idle)
        const int vec = wave_vec(n_feat, align_or);
        const dim3 grid(ceil_div(n_vert, 4)), block(256);
#define HGC_FWD(VEC, MAX, EXPW)                                                                                     \
    accumulate_fwd_wave_kernel<VEC, MAX, EXPW><<<grid, block, 0, s>>>(d_distances, d_feat, d_idxs, d_out_feat,         \
                                                                     d_out_maxidxs, d_out_maxslots, n_vert, n_neigh, \
                                                                     n_feat, n_out_feat, divisor, d_order, d_out_weights)
#define HGC_FWD_VEC(MAX, EXPW)                                                                                      \
    if (vec == 4) HGC_FWD(4, MAX, EXPW); else if (vec == 2) HGC_FWD(2, MAX, EXPW); else HGC_FWD(1, MAX, EXPW)
        if (mean_and_max) {
            if (exp_in_kernel) { HGC_FWD_VEC(true, true); } else { HGC_FWD_VEC(true, false); }
        } else {
            if (exp_in_kernel) { HGC_FWD_VEC(false, true); } else { HGC_FWD_VEC(false, false); }
        }
#undef HGC_FWD_VEC
#undef HGC_FWD
        return check_launch("accumulate_fwd_wave_kernel");
    }
    const bool vec4 = (n_feat % 4 == 0) && (align_or & 15u) == 0;
    const long long threads = (long long)n_vert * (vec4 ? n_feat / 4 : n_feat);
    const dim3 grid(ceil_div(threads, 256)), block(256);
    if (vec4) {
        if (mean_and_max)
            accumulate_fwd_kernel<4, true><<<grid, block, 0, s>>>(d_distances, d_feat, d_idxs, d_out_feat, d_out_maxidxs,
                                                                  d_out_maxslots, n_vert, n_neigh, n_feat, n_out_feat, divisor);
        else
            accumulate_fwd_kernel<4, false><<<grid, block, 0, s>>>(d_distances, d_feat, d_idxs, d_out_feat, d_out_maxidxs,
                                                                   d_out_maxslots, n_vert, n_neigh, n_feat, n_out_feat, divisor);
    } else {
        if (mean_and_max)
            accumulate_fwd_kernel<1, true><<<grid, block, 0, s>>>(d_distances, d_feat, d_idxs, d_out_feat, d_out_maxidxs,
                                                                  d_out_maxslots, n_vert, n_neigh, n_feat, n_out_feat, divisor);
        else
            accumulate_fwd_kernel<1, false><<<grid, block, 0, s>>>(d_distances, d_feat, d_idxs, d_out_feat, d_out_maxidxs,
                                                                   d_out_maxslots, n_vert, n_neigh, n_feat, n_out_feat, divisor);
    }
    return check_launch("accumulate_fwd_kernel");
}

}  // namespace hgc

using namespace hgc;

extern "C" {

int hgc_accumulate_knn_slots(const float *d_distances, const float *d_feat, const int *d_idxs, float *d_out_feat,
                             int *d_out_maxidxs, unsigned char *d_out_maxslots, const int *d_vertex_order, int n_vert,
                             int n_neigh, int n_feat, int n_out_feat, int n_moments, int mean_and_max,
                             hgc_stream_t stream) {
    (void)n_moments;  // carried by the reference op, never used by its kernels
    return accumulate_forward(d_distances, d_feat, d_idxs, d_out_feat, d_out_maxidxs, d_out_maxslots, n_vert, n_neigh,
                              n_feat, n_out_feat, mean_and_max, (float)n_neigh, d_vertex_order, nullptr, stream);
}

int hgc_accumulate_knn_exp_slots(const float *d_distances, const float *d_feat, const int *d_idxs, float *d_out_feat,
                                 int *d_out_maxidxs, unsigned char *d_out_maxslots, float *d_out_weights,
                                 const int *d_vertex_order, int n_vert, int n_neigh, int n_feat, int n_out_feat,
                                 int n_moments, int mean_and_max, hgc_stream_t stream) {
    (void)n_moments;
    HGC_REQUIRE(n_vert <= 0 || d_out_weights, "null pointer");
    HGC_REQUIRE(((reinterpret_cast<uintptr_t>(d_distances) | reinterpret_cast<uintptr_t>(d_out_weights)) & 15u) == 0,
                "distances and weights must start on 16-byte boundaries");
    return accumulate_forward(d_distances, d_feat, d_idxs, d_out_feat, d_out_maxidxs, d_out_maxslots, n_vert, n_neigh,
                              n_feat, n_out_feat, mean_and_max, (float)n_neigh, d_vertex_order, d_out_weights, stream);
}

int hgc_accumulate_knn(const float *d_distances, const float *d_feat, const int *d_idxs, float *d_out_feat,
                       int *d_out_maxidxs, int n_vert, int n_neigh, int n_feat, int n_out_feat, int n_moments,
                       int mean_and_max, hgc_stream_t stream) {
    return hgc_accumulate_knn_slots(d_distances, d_feat, d_idxs, d_out_feat, d_out_maxidxs, nullptr, nullptr, n_vert,
                                    n_neigh, n_feat, n_out_feat, n_moments, mean_and_max, stream);
}

size_t hgc_inverse_index_without_first_column_workspace_bytes(int n_vert) {
    size_t temp = 0;
    (void)rocprim::exclusive_scan(nullptr, temp, (const int *)nullptr, (int *)nullptr, 0, (size_t)std::max(n_vert, 0) + 1,
                                  rocprim::plus<int>(), (hipStream_t) nullptr);
    return align_up(temp) + 2 * align_up(((size_t)std::max(n_vert, 0) + 1) * sizeof(int));
}

int hgc_inverse_index_without_first_column(const int *d_inv_offsets, const int *d_inv_slots, int n_vert, int n_neigh,
                                           int *d_out_offsets, int *d_out_slots, void *workspace,
                                           size_t workspace_bytes, hgc_stream_t stream) {
    HGC_REQUIRE(n_vert >= 0 && n_neigh >= 2, "needs a table of at least two columns");
    HGC_REQUIRE(d_out_offsets, "null pointer");
    hipStream_t s = as_stream(stream);
    if (n_vert == 0) return launch_fill_i32(d_out_offsets, 0, 1, s);
    HGC_REQUIRE(d_inv_offsets && d_inv_slots && d_out_slots, "null pointer");
    if (!workspace || !aligned256(workspace) ||
        workspace_bytes < hgc_inverse_index_without_first_column_workspace_bytes(n_vert))
        return fail(HGC_ERR_WORKSPACE, "inverse index workspace missing, misaligned or too small");
    Carver carve(workspace);
    int *dropped = carve.take<int>((size_t)n_vert + 1);
    int *dropped_before = carve.take<int>((size_t)n_vert + 1);
    void *temp = carve.base + carve.used;
    size_t temp_bytes = workspace_bytes - carve.used;
    const int blocks = ceil_div((long long)n_vert + 1, 256 / kWave);
    const acc::FastDiv div_k = acc::make_fast_div(n_neigh);
    first_column_entries_kernel<<<blocks, 256, 0, s>>>(d_inv_offsets, d_inv_slots, n_vert, div_k, n_neigh, dropped);
    int rc = check_launch("first_column_entries");
    if (rc) return rc;
    HGC_HIP(rocprim::exclusive_scan(temp, temp_bytes, dropped, dropped_before, 0, (size_t)n_vert + 1,
                                    rocprim::plus<int>(), s));
    drop_first_column_kernel<<<blocks, 256, 0, s>>>(d_inv_offsets, d_inv_slots, dropped_before, n_vert, div_k,
                                                    n_neigh, d_out_offsets, d_out_slots);
    return check_launch("drop_first_column");
}

}  // extern "C"

namespace hgc {

// Gradient shared by accumulate_knn_grad (divisor = K) and push_knn (divisor = 1).
// Either output may be null: the weight gradient needs neither the inverse index
// nor the weights, the feature gradient needs neither the features nor the
// neighbour table.
int accumulate_gradient(const float *d_grad_from_out_features, const float *d_distances, const float *d_feat,
                        const int *d_max_feat_indices, const unsigned char *d_max_slots, const int *d_neigh_indices,
                        const int *d_inv_offsets, const int *d_inv_slots, float *d_out_grad_distances,
                        float *d_out_grad_features, int n_vert, int n_neigh, int n_feat, int n_grad_from_out_feat,
                        int mean_and_max, float divisor, const int *d_order, void *records, size_t records_bytes,
                        hgc_stream_t stream) {
    const bool want_w = d_out_grad_distances != nullptr, want_f = d_out_grad_features != nullptr;
    HGC_REQUIRE(n_vert >= 0 && n_neigh >= 1 && n_feat >= 1, "bad sizes");
    HGC_REQUIRE(n_grad_from_out_feat == n_feat * (mean_and_max ? 2 : 1),
                "gradient width must be n_feat * (mean_and_max ? 2 : 1)");
    HGC_REQUIRE((long long)n_vert * n_neigh < (1ll << 31), "n_vert * n_neigh must stay below 2^31");
    if (n_vert == 0) return HGC_OK;
    HGC_REQUIRE(d_grad_from_out_features && (want_w || want_f), "null pointer");
    HGC_REQUIRE(!want_w || (d_feat && d_neigh_indices), "null pointer");
    HGC_REQUIRE(!want_f || (d_distances && d_inv_offsets && d_inv_slots), "null pointer");
    HGC_REQUIRE(!mean_and_max || d_max_feat_indices, "mean_and_max needs d_max_feat_indices");
    hipStream_t s = as_stream(stream);
    const uintptr_t align_or = reinterpret_cast<uintptr_t>(d_grad_from_out_features) | reinterpret_cast<uintptr_t>(d_feat) |
                               reinterpret_cast<uintptr_t>(d_max_feat_indices) |
                               reinterpret_cast<uintptr_t>(d_out_grad_features);
    const bool pow2k = divisor == (float)(int)divisor && is_pow2((int)divisor);

    const bool fits_32bit = (unsigned long long)n_vert * (unsigned long long)(2 * n_feat) * 4ull < (1ull << 32);
    // both gradients from one gather pass where that kernel covers the shape (rows of
    // 16 to 256 features), or the mean-only feature gradient alone: the gather without
    // the dot products
    if (fits_32bit && want_f && want_w && mean_and_max && d_max_slots && records) {
        const int rc = launch_accumulate_grad_records(d_grad_from_out_features, d_distances, d_feat, d_max_slots,
                                                      d_inv_offsets, d_inv_slots, d_out_grad_distances,
                                                      d_out_grad_features, n_vert, n_neigh, n_feat, d_neigh_indices,
                                                      d_order, divisor, records, records_bytes, s);
        if (rc <= 0) return rc;  // 1: shape not covered
    }
    if (fits_32bit && want_f && (want_w || !mean_and_max)) {
        const int rc = launch_accumulate_grad_fused(d_grad_from_out_features, d_distances, d_feat, d_max_feat_indices,
                                                    d_max_slots, d_inv_offsets, d_inv_slots, d_out_grad_distances,
                                                    d_out_grad_features, n_vert, n_neigh, n_feat, n_grad_from_out_feat,
                                                    mean_and_max != 0, d_neigh_indices, d_order, divisor, s);
        if (rc <= 0) return rc;  // 1: shape not covered, use the two-kernel path
    }
    if (n_feat >= kWave && fits_32bit) {  // one wave per vertex, rows addressed through 32-bit buffer offsets
        const bool use_slots = d_max_slots != nullptr && n_neigh <= 254;
        const int vec = wave_vec(n_feat, align_or);
        const dim3 grid(ceil_div(n_vert, 4)), block(256);
        const FastDiv div_k = make_fast_div(n_neigh);
#define HGC_FGW(VEC, MAX, P2, SL)                                                                                      \
    feature_grad_wave_kernel<VEC, MAX, P2, SL><<<fg_grid, block, 0, s>>>(                                              \
        d_grad_from_out_features, d_distances, d_max_feat_indices, d_max_slots, d_inv_offsets, d_inv_slots,            \
        d_out_grad_features, n_vert, n_neigh, n_feat, n_grad_from_out_feat, div_k, n_slices, divisor, d_order)
#define HGC_FGW_V(VEC)                                                                                   \
    do {                                                                                                 \
        if (mean_and_max && use_slots) { if (pow2k) HGC_FGW(VEC, true, true, true); else HGC_FGW(VEC, true, false, true); } \
        else if (mean_and_max) { if (pow2k) HGC_FGW(VEC, true, true, false); else HGC_FGW(VEC, true, false, false); } \
        else { if (pow2k) HGC_FGW(VEC, false, true, false); else HGC_FGW(VEC, false, false, false); }       \
    } while (0)
        // two feature slices as soon as a row has two or more 64-feature blocks
        // Without the slot table a gathered row is 1.5 KB (gradient row + arg-max
        // indices) and the neighbour window overflows one XCD's L2: slice. With it
        // the row shrinks to 640 B plus a few lanes of the max half and the wider
        // unsliced loads win.
        const int n_slices = (n_feat >= 2 * kWave && mean_and_max && !use_slots) ? 2 : 1;
        const int fg_vec = n_slices == 1 ? vec : wave_vec(n_feat / 2, align_or);
        const int tiles = ceil_div(n_vert, 4);
        const dim3 fg_grid(n_slices == 1 ? tiles : kNumXcd * ceil_div(tiles, kNumXcd / n_slices));
        if (want_f) {
            if (fg_vec == 4) HGC_FGW_V(4); else if (fg_vec == 2) HGC_FGW_V(2); else HGC_FGW_V(1);
        }
#undef HGC_FGW_V
#undef HGC_FGW
        int rc = check_launch("feature_grad_wave_kernel");
        if (rc || !want_w) return rc;
#define HGC_WGW(VEC, MAX)                                                                                       \
    weight_grad_wave_kernel<VEC, MAX><<<grid, block, 0, s>>>(d_grad_from_out_features, d_feat, d_max_feat_indices, \
                                                            d_neigh_indices, d_out_grad_distances, n_vert, n_neigh, \
                                                            n_feat, n_grad_from_out_feat, divisor, d_order)
        if (mean_and_max) {
            if (vec == 4) HGC_WGW(4, true); else if (vec == 2) HGC_WGW(2, true); else HGC_WGW(1, true);
        } else {
            if (vec == 4) HGC_WGW(4, false); else if (vec == 2) HGC_WGW(2, false); else HGC_WGW(1, false);
        }
#undef HGC_WGW
        return check_launch("weight_grad_wave_kernel");
    }

    const bool vec4 = (n_feat % 4 == 0) && (align_or & 15u) == 0;

    // ---- feature gradient ----
    if (want_f) {
        const long long threads = (long long)n_vert * (vec4 ? n_feat / 4 : n_feat);
        const dim3 grid(ceil_div(threads, 256)), block(256);
#define HGC_FG(VEC, MAX, P2)                                                                                      \
    feature_grad_kernel<VEC, MAX, P2><<<grid, block, 0, s>>>(d_grad_from_out_features, d_distances, d_max_feat_indices, \
                                                            d_inv_offsets, d_inv_slots, d_out_grad_features, n_vert, \
                                                            n_neigh, n_feat, n_grad_from_out_feat, divisor)
        if (vec4) {
            if (mean_and_max) { if (pow2k) HGC_FG(4, true, true); else HGC_FG(4, true, false); }
            else              { if (pow2k) HGC_FG(4, false, true); else HGC_FG(4, false, false); }
        } else {
            if (mean_and_max) { if (pow2k) HGC_FG(1, true, true); else HGC_FG(1, true, false); }
            else              { if (pow2k) HGC_FG(1, false, true); else HGC_FG(1, false, false); }
        }
#undef HGC_FG
        int rc = check_launch("feature_grad_kernel");
        if (rc) return rc;
    }

    // ---- weight gradient ----
    if (want_w) {
        // threads per vertex: largest power of two <= min(64, F/VEC)
        const int vec = vec4 ? 4 : 1;
        int tpv = 1;
        while (tpv * 2 <= std::min(64, n_feat / vec)) tpv *= 2;
        const long long threads = (long long)n_vert * tpv;
        const dim3 grid(ceil_div(threads, 256)), block(256);
        if (vec4) {
            if (mean_and_max)
                weight_grad_kernel<4, true><<<grid, block, 0, s>>>(d_grad_from_out_features, d_feat, d_max_feat_indices,
                                                                   d_neigh_indices, d_out_grad_distances, n_vert, n_neigh,
                                                                   n_feat, n_grad_from_out_feat, tpv, divisor);
            else
                weight_grad_kernel<4, false><<<grid, block, 0, s>>>(d_grad_from_out_features, d_feat, d_max_feat_indices,
                                                                    d_neigh_indices, d_out_grad_distances, n_vert, n_neigh,
                                                                    n_feat, n_grad_from_out_feat, tpv, divisor);
        } else {
            if (mean_and_max)
                weight_grad_kernel<1, true><<<grid, block, 0, s>>>(d_grad_from_out_features, d_feat, d_max_feat_indices,
                                                                   d_neigh_indices, d_out_grad_distances, n_vert, n_neigh,
                                                                   n_feat, n_grad_from_out_feat, tpv, divisor);
            else
                weight_grad_kernel<1, false><<<grid, block, 0, s>>>(d_grad_from_out_features, d_feat, d_max_feat_indices,
                                                                    d_neigh_indices, d_out_grad_distances, n_vert, n_neigh,
                                                                    n_feat, n_grad_from_out_feat, tpv, divisor);
        }
        return check_launch("weight_grad_kernel");
    }
    return HGC_OK;
}

}  // namespace hgc

extern "C" {

int hgc_accumulate_knn_grad_slots(const float *d_grad_from_out_features, const float *d_distances, const float *d_feat,
                                  const int *d_max_feat_indices, const unsigned char *d_max_slots,
                                  const int *d_neigh_indices, const int *d_inv_offsets, const int *d_inv_slots,
                                  const int *d_vertex_order, float *d_out_grad_distances, float *d_out_grad_features,
                                  int n_vert, int n_neigh, int n_feat, int n_grad_from_out_feat, int n_moments,
                                  int mean_and_max, hgc_stream_t stream) {
    (void)n_moments;
    HGC_REQUIRE(n_vert <= 0 || (d_out_grad_distances && d_out_grad_features), "null pointer");
    return accumulate_gradient(d_grad_from_out_features, d_distances, d_feat, d_max_feat_indices, d_max_slots,
                               d_neigh_indices, d_inv_offsets, d_inv_slots, d_out_grad_distances, d_out_grad_features,
                               n_vert, n_neigh, n_feat, n_grad_from_out_feat, mean_and_max, (float)n_neigh,
                               d_vertex_order, nullptr, 0, stream);
}

size_t hgc_accumulate_knn_grad_records_workspace_bytes(int n_vert, int n_neigh, int n_feat, int mean_and_max) {
    return mean_and_max ? accumulate_grad_records_bytes(n_vert, n_neigh, n_feat) : 0;
}

int hgc_accumulate_knn_grad_records_pays(int n_vert, int n_neigh, int n_feat, int mean_and_max) {
    return mean_and_max && accumulate_grad_records_pays(n_vert, n_neigh, n_feat) ? 1 : 0;
}

int hgc_accumulate_knn_grad_records(const float *d_grad_from_out_features, const float *d_distances, const float *d_feat,
                                    const int *d_max_feat_indices, const unsigned char *d_max_slots,
                                    const int *d_neigh_indices, const int *d_inv_offsets, const int *d_inv_slots,
                                    const int *d_vertex_order, float *d_out_grad_distances, float *d_out_grad_features,
                                    int n_vert, int n_neigh, int n_feat, int n_grad_from_out_feat, int n_moments,
                                    int mean_and_max, void *workspace, size_t workspace_bytes, hgc_stream_t stream) {
    (void)n_moments;
    HGC_REQUIRE(n_vert <= 0 || (d_out_grad_distances && d_out_grad_features), "null pointer");
    const size_t need = hgc_accumulate_knn_grad_records_workspace_bytes(n_vert, n_neigh, n_feat, mean_and_max);
    if (need != 0 && d_max_slots && (!workspace || !aligned256(workspace) || workspace_bytes < need))
        return fail(HGC_ERR_WORKSPACE, "accumulate_knn_grad_records workspace missing, misaligned or too small");
    return accumulate_gradient(d_grad_from_out_features, d_distances, d_feat, d_max_feat_indices, d_max_slots,
                               d_neigh_indices, d_inv_offsets, d_inv_slots, d_out_grad_distances, d_out_grad_features,
                               n_vert, n_neigh, n_feat, n_grad_from_out_feat, mean_and_max, (float)n_neigh,
                               d_vertex_order, need != 0 ? workspace : nullptr, workspace_bytes, stream);
}

int hgc_accumulate_knn_grad(const float *d_grad_from_out_features, const float *d_distances, const float *d_feat,
                            const int *d_max_feat_indices, const int *d_neigh_indices, const int *d_inv_offsets,
                            const int *d_inv_slots, float *d_out_grad_distances, float *d_out_grad_features,
                            int n_vert, int n_neigh, int n_feat, int n_grad_from_out_feat, int n_moments,
                            int mean_and_max, hgc_stream_t stream) {
    return hgc_accumulate_knn_grad_slots(d_grad_from_out_features, d_distances, d_feat, d_max_feat_indices, nullptr,
                                         d_neigh_indices, d_inv_offsets, d_inv_slots, nullptr, d_out_grad_distances,
                                         d_out_grad_features, n_vert, n_neigh, n_feat, n_grad_from_out_feat, n_moments,
                                         mean_and_max, stream);
}

}  // extern "C"
