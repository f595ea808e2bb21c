// Gradient of the GravNet neighbour accumulation, both outputs from ONE gather
// pass over the inverse neighbour index.
//
// Reference behaviour restated here:
//   modules/compiled/accumulate_knn_grad_kernel.cc:36-97   (feature gradient)
//   modules/compiled/accumulate_knn_grad_kernel.cc:99-165  (weight gradient)
//
// For an entry (v, n) of target m's inverse list (idx[v, n] == m) the gradient
// row g[v, :] is needed twice: the feature gradient of m accumulates
// (g[v,f]/K)*w[v,n] (+ the max part), and the weight gradient of slot (v, n) is
// the dot product of g[v, :] with feat[m, :] -- the wave's own row. One wave per
// target therefore gathers every gradient row once, adds it to its feature
// gradient in ascending (v, n) order (the reference CPU kernel's order, so the
// result is bit-identical to it) and reduces the dot products of 16 entries at
// a time across its lanes, writing each weight gradient to its own slot.
//
// The same kernel without the dot products (no weight gradient wanted, mean
// only) is the ordered gather push_knn needs: out[m] = sum of w[v,n] * feat[v].
//
// Scalar-unit economy: the per-entry metadata (flat slot -> vertex, row offset,
// weight, arg-max key) is computed by the 64 lanes for 64 entries at once and
// broadcast per entry with v_readlane; the hot loop carries no scalar loads and
// no scalar address arithmetic.
#include "accumulate_rows.hpp"

#include <algorithm>
#include <cstdlib>

namespace hgc {

namespace {

using namespace acc;

constexpr int kRows = 4;    // gathered rows in flight per load batch
constexpr int kGroup = 16;  // entries per cross-lane reduction

// Arg-max information of one gathered row for the VEC features of a lane:
// SLOTS: VEC slot bytes packed in one word, else VEC neighbour indices.
template <int VEC, bool SLOTS>
struct ArgInfo {
    uint32_t v[SLOTS ? 1 : VEC];
};

// Does byte E of `packed` equal the wave-uniform `key`? One SDWA compare that
// leaves the lane mask in scalar registers, where the selects below consume it.
template <int E>
__device__ __forceinline__ bool slot_byte_is(uint32_t packed, uint32_t key) {
    uint64_t mask;
    if constexpr (E == 0) asm("v_cmp_eq_u32_sdwa %0, %1, %2 src0_sel:BYTE_0 src1_sel:DWORD" : "=s"(mask) : "v"(packed), "s"(key));
    else if constexpr (E == 1) asm("v_cmp_eq_u32_sdwa %0, %1, %2 src0_sel:BYTE_1 src1_sel:DWORD" : "=s"(mask) : "v"(packed), "s"(key));
    else if constexpr (E == 2) asm("v_cmp_eq_u32_sdwa %0, %1, %2 src0_sel:BYTE_2 src1_sel:DWORD" : "=s"(mask) : "v"(packed), "s"(key));
    else asm("v_cmp_eq_u32_sdwa %0, %1, %2 src0_sel:BYTE_3 src1_sel:DWORD" : "=s"(mask) : "v"(packed), "s"(key));
    return __builtin_amdgcn_inverse_ballot_w64(mask);
}

template <int VEC, bool SLOTS>
__device__ __forceinline__ void arg_hits(const ArgInfo<VEC, SLOTS> &ai, uint32_t key, bool (&hit)[VEC]) {
    if constexpr (SLOTS) {
        hit[0] = slot_byte_is<0>(ai.v[0], key);
        if constexpr (VEC >= 2) hit[1] = slot_byte_is<1>(ai.v[0], key);
        if constexpr (VEC >= 4) {
            hit[2] = slot_byte_is<2>(ai.v[0], key);
            hit[3] = slot_byte_is<3>(ai.v[0], key);
        }
    } else {
#pragma unroll
        for (int e = 0; e < VEC; ++e) hit[e] = ai.v[e] == key;
    }
}

template <int VEC>
__device__ __forceinline__ uint32_t load_slot_bytes(__amdgpu_buffer_rsrc_t rsrc, uint32_t row_byte_offset,
                                                    uint32_t lane_col) {
    if constexpr (VEC == 4) return __builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)lane_col, (int)row_byte_offset, 0);
    else if constexpr (VEC == 2) return __builtin_amdgcn_raw_buffer_load_b16(rsrc, (int)lane_col, (int)row_byte_offset, 0);
    else return __builtin_amdgcn_raw_buffer_load_b8(rsrc, (int)lane_col, (int)row_byte_offset, 0);
}

// 16 partial sums per lane in; afterwards lane L holds the sum over all 64 lanes
// of value index (L & 15). Fixed butterfly: deterministic summation order.
__device__ __forceinline__ float transpose_reduce_16(float (&val)[kGroup]) {
    const int lane = lane_id();
#pragma unroll
    for (int h = kGroup / 2; h >= 1; h >>= 1) {
        const bool upper = (lane & h) != 0;
#pragma unroll
        for (int i = 0; i < h; ++i) {
            const float a = val[i], b = val[i + h];
            const float send = upper ? a : b;
            const float keep = upper ? b : a;
            val[i] = keep + __shfl_xor(send, h, kWave);
        }
    }
    float r = val[0];
#pragma unroll
    for (int h = kGroup; h < kWave; h <<= 1) r = r + __shfl_xor(r, h, kWave);
    return r;
}

// With arg-max slots a row's byte offset (a multiple of 512) and the entry's
// slot share one word, so that one cross-lane read brings both.
constexpr int kKeyBits = 9;
constexpr uint32_t kKeyMask = (1u << kKeyBits) - 1u;
// a per-lane buffer offset no matrix reaches: the hardware range check turns
// the load into "return 0" without a memory access
constexpr uint32_t kOutOfRange = 0xfffffff0u;

// Entries [c, c+16) of the current 64-entry batch. FAST: all 16 exist and none
// is a repeated self reference.
//
// Feature gradient addend of one entry, per feature: ((g/K)*w) + (hit ? g_max*w : 0),
// added in list order -- the reference's terms in its order. Two rewrites keep
// the bits and save vector instructions: for a power-of-two K the exact
// scaling 1/K moves onto the weight (wk = w/K, identical unless g/K is
// subnormal), and the max part is formed as (hit ? g_max : 0) * w, whose zero
// may carry the weight's sign, which cannot change a sum that started at +0
// (it would differ for an infinite weight only).
template <int VEC, int NB, bool MAX, bool POW2K, bool SLOTS, bool FAST, bool WGRAD, bool PARTIAL>
__device__ __forceinline__ void grad_group(const RowMatrix &Gm, const RowMatrix &MI, __amdgpu_buffer_rsrc_t MS,
                                           const uint32_t (&lane_bytes)[NB], uint32_t max_col_bytes,
                                           uint32_t g_row_bytes, int c, int cnt,
                                           uint64_t repmask, int self_key, int m, uint32_t offkey_v, float w_v,
                                           float wk_v, const float (&xo)[NB][VEC], const float (&xk)[NB][VEC],
                                           float (&acc)[NB][VEC], float kf, float (&val)[kGroup]) {
#pragma unroll
    for (int h = 0; h < kGroup; h += kRows) {
        uint32_t soff[kRows], skey[kRows];
        float sw[kRows], swk[kRows];
        bool rep[kRows], live[kRows];
#pragma unroll
        for (int u = 0; u < kRows; ++u) {
            const int li = c + h + u;  // lanes past the end of the list hold a copy of its last entry
            const uint32_t ok = (uint32_t)__builtin_amdgcn_readlane((int)offkey_v, li);
            if (MAX && SLOTS && PARTIAL) {  // vertex and slot share the word, the row offset is a scalar multiply away
                soff[u] = (ok >> kKeyBits) * g_row_bytes;
                skey[u] = ok & kKeyMask;
            } else {
                soff[u] = (MAX && SLOTS) ? (ok & ~kKeyMask) : ok;
                skey[u] = (MAX && SLOTS) ? (ok & kKeyMask) : (uint32_t)m;
            }
            sw[u] = __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(w_v), li));
            swk[u] = POW2K ? __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(wk_v), li)) : 0.f;
            rep[u] = false;
            live[u] = true;
            if (!FAST) {
                live[u] = li < cnt;
                rep[u] = ((repmask >> li) & 1ull) != 0;
                if (MAX && SLOTS && rep[u]) skey[u] = (uint32_t)self_key;
            }
        }
        // arg-max tables first (they gate the loads of the max half), then the mean half
        ArgInfo<VEC, SLOTS> ai[kRows][NB];
        float gm[kRows][NB][VEC], gx[kRows][NB][VEC];
        bool hit[kRows][NB][VEC];
        if (MAX) {
#pragma unroll
            for (int u = 0; u < kRows; ++u)
#pragma unroll
                for (int b = 0; b < NB; ++b) {
                    if constexpr (SLOTS) ai[u][b].v[0] = load_slot_bytes<VEC>(MS, soff[u] >> 3, lane_bytes[b] >> 2);
                    else MI.load_at<VEC>(soff[u] >> 1, lane_bytes[b], ai[u][b].v);
                }
        }
#pragma unroll
        for (int u = 0; u < kRows; ++u)
#pragma unroll
            for (int b = 0; b < NB; ++b) Gm.load_at<VEC>(soff[u], lane_bytes[b], gm[u][b]);
        if (MAX) {
            // the max half of a gradient row is fetched only by the lanes whose
            // feature has its maximum at this entry (about F/K lanes per row); the
            // other lanes aim out of range and receive 0
#pragma unroll
            for (int u = 0; u < kRows; ++u)
#pragma unroll
                for (int b = 0; b < NB; ++b) {
                    arg_hits<VEC, SLOTS>(ai[u][b], skey[u], hit[u][b]);
                    bool any = false;
#pragma unroll
                    for (int e = 0; e < VEC; ++e) any = any || hit[u][b][e];
                    // a lane beyond the last feature (rows that do not fill their last block of
                    // 64) aims every load out of range and so only ever holds zeros
                    if (PARTIAL) any = any && lane_bytes[b] != kOutOfRange;
                    Gm.load_at<VEC>(soff[u], any ? lane_bytes[b] + max_col_bytes : kOutOfRange, gx[u][b]);
                }
        }
#pragma unroll
        for (int u = 0; u < kRows; ++u) {
            if (!FAST && !live[u]) break;  // wave-uniform
#pragma unroll
            for (int b = 0; b < NB; ++b)
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    const float g = gm[u][b][e];
                    const float part = POW2K ? g * swk[u] : (g / kf) * sw[u];
                    // weight gradient of slot (v, n): partial dot products with the wave's own row
                    if (WGRAD) val[h + u] = __builtin_fmaf(g, xk[b][e], val[h + u]);
                    if (MAX) {
                        // a lane with one hit among its VEC features has loaded all of them
                        const float gsel = (VEC == 1 || hit[u][b][e]) ? gx[u][b][e] : 0.f;
                        if (WGRAD) val[h + u] = __builtin_fmaf(gsel, xo[b][e], val[h + u]);
                        // repeated self references carry the max part once, at the first self slot
                        const float part_max = (!FAST && rep[u]) ? 0.f : gsel * sw[u];
                        const float add = part + part_max;
                        acc[b][e] = acc[b][e] + add;
                    } else {
                        acc[b][e] = acc[b][e] + part;  // the reference's "+ 0" cannot change the sum
                    }
                }
        }
        // keep the loads of the next rows behind this arithmetic: without it the
        // scheduler hoists every load of the group and the kernel loses occupancy
        __builtin_amdgcn_sched_barrier(0);
    }
}

// WGRAD false: feature gradient only (feat, idx and gw are not touched); kf is
// what the mean part is divided by (K for the accumulation, 1 for a plain push).
// PARTIAL: F is not a multiple of 64 (VEC is 1 then); the lanes of the last block
// beyond F stay idle.
template <int VEC, int NB, bool MAX, bool POW2K, bool SLOTS, bool WGRAD, bool PARTIAL>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(5, 8))) void accumulate_grad_fused_kernel(
    const float *__restrict__ g, const float *__restrict__ w, const float *__restrict__ feat,
    const int *__restrict__ maxidx, const unsigned char *__restrict__ maxslot, const int *__restrict__ inv_off,
    const int *__restrict__ inv_slots, float *__restrict__ gw, float *__restrict__ gfeat, int n_vert, int K, int F,
    int g_cols, const FastDiv div_k, const int *__restrict__ idx, const int *__restrict__ order, const float kf) {
    const int m = wave_vertex(order, n_vert);
    if (m >= n_vert) return;
    const int lane = lane_id();
    const float inv_kf = 1.f / kf;  // exact when K is a power of two
    const double inv_kd = 1.0 / (double)kf;
    const int begin = inv_off[m], end = inv_off[m + 1];
    const RowMatrix Gm(g, n_vert, g_cols);
    const RowMatrix MI(maxidx, (MAX && !SLOTS) ? n_vert : 0, F);
    const __amdgpu_buffer_rsrc_t MS = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<unsigned char *>(maxslot), 0, (MAX && SLOTS) ? (int)(uint32_t)((size_t)n_vert * F) : 0, 0x00020000);
    const uint32_t max_col_bytes = (uint32_t)F * 4u;
    const uint32_t g_row_bytes = (uint32_t)g_cols * 4u;

    uint32_t lane_bytes[NB];
    float xo[NB][VEC], xk[NB][VEC], acc[NB][VEC];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        const int fb = (b * kWave + lane) * VEC;
        const bool in_row = !PARTIAL || fb < F;
        lane_bytes[b] = in_row ? (uint32_t)fb * 4u : kOutOfRange;
#pragma unroll
        for (int e = 0; e < VEC; ++e) xo[b][e] = 0.f;
        if (WGRAD && in_row) load_vec<VEC>(feat + (size_t)m * F + fb, xo[b]);
#pragma unroll
        for (int e = 0; e < VEC; ++e) xk[b][e] = (float)((double)xo[b][e] * inv_kd);
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[b][e] = 0.f;
    }

    // first slot of the target's own row that names the target itself (-1: none);
    // later entries naming it are repeated self references
    int self_key = -1;
    for (int n0 = 0; MAX && n0 < K && self_key < 0; n0 += kWave) {
        const int n = n0 + lane;
        const uint64_t is_self = __ballot(n < K && idx[(size_t)m * K + min(n, K - 1)] == m);
        if (is_self != 0) self_key = n0 + __ffsll((unsigned long long)is_self) - 1;
    }
    for (int b0 = begin; b0 < end; b0 += kWave) {
        const int cnt = min(kWave, end - b0);
        const int e = min(b0 + lane, end - 1);
        const int slot_v = inv_slots[e];
        const float w_v = w[slot_v];
        const int v = fast_div(slot_v, div_k);
        const int key_v = slot_v - v * K;
        // row offset of the entry's vertex, with the entry's slot in its low bits
        // (rows that are no multiple of 512 bytes have no free low bits: vertex and slot are packed instead)
        const uint32_t offkey_v = (MAX && SLOTS && PARTIAL)
                                      ? ((uint32_t)v << kKeyBits) | (uint32_t)key_v
                                      : (uint32_t)v * g_row_bytes | ((MAX && SLOTS) ? (uint32_t)key_v : 0u);
        const float wk_v = w_v * inv_kf;
        const uint64_t repmask = MAX ? __ballot(v == m && key_v != self_key && lane < cnt) : 0ull;
        for (int c = 0; c < cnt; c += kGroup) {
            float val[kGroup];
#pragma unroll
            for (int i = 0; i < kGroup; ++i) val[i] = 0.f;
            const bool fast = (c + kGroup <= cnt) && ((repmask >> c) & ((1ull << kGroup) - 1)) == 0;
            if (fast)
                grad_group<VEC, NB, MAX, POW2K, SLOTS, true, WGRAD, PARTIAL>(Gm, MI, MS, lane_bytes, max_col_bytes, g_row_bytes, c, cnt, repmask,
                                                                    self_key, m, offkey_v, w_v, wk_v, xo, xk, acc, kf, val);
            else
                grad_group<VEC, NB, MAX, POW2K, SLOTS, false, WGRAD, PARTIAL>(Gm, MI, MS, lane_bytes, max_col_bytes, g_row_bytes, c, cnt, repmask,
                                                                     self_key, m, offkey_v, w_v, wk_v, xo, xk, acc, kf, val);
            if (WGRAD) {
                const float r = transpose_reduce_16(val);  // lane L: entry c + (L & 15)
                const int dst = __shfl(slot_v, c + (lane & (kGroup - 1)), kWave);
                if (lane < kGroup && c + lane < cnt) gw[dst] = r;
            }
        }
    }
#pragma unroll
    for (int b = 0; b < NB; ++b)
        if (!PARTIAL || lane_bytes[b] != kOutOfRange) store_vec<VEC>(gfeat + (size_t)m * F + (lane_bytes[b] >> 2), acc[b]);
}

// weight gradient of padded slots (index < 0 or out of range): they sort to the
// tail of the inverse list, past the last target's entries
__global__ __launch_bounds__(256) void zero_padded_weight_grad_kernel(const int *__restrict__ inv_off,
                                                                      const int *__restrict__ inv_slots,
                                                                      float *__restrict__ gw, int n_vert, long long total) {
    const long long first = inv_off[n_vert];
    for (long long i = first + (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (long long)gridDim.x * blockDim.x)
        gw[inv_slots[i]] = 0.f;
}

template <int VEC, int NB, bool PARTIAL>
int launch_fused(const float *g, const float *w, const float *feat, const int *maxidx, const unsigned char *maxslot,
                 const int *inv_off, const int *inv_slots, float *gw, float *gfeat, int n_vert, int K, int F, int g_cols,
                 bool mean_and_max, const int *idx, const int *order, float divisor, bool want_w, hipStream_t s) {
    const dim3 grid(ceil_div(n_vert, 4)), block(256);
    const FastDiv div_k = make_fast_div(K);
    const bool pow2k = divisor == (float)(int)divisor && is_pow2((int)divisor);
    const bool slots = mean_and_max && maxslot != nullptr;
#define HGC_FUSED(MAX, P2, SL, WG)                                                                                       \
    accumulate_grad_fused_kernel<VEC, NB, MAX, P2, SL, WG, PARTIAL><<<grid, block, 0, s>>>(g, w, feat, maxidx, maxslot, inv_off, \
                                                                                  inv_slots, gw, gfeat, n_vert, K, F,    \
                                                                                  g_cols, div_k, idx, order, divisor)
    if (!want_w) { if (pow2k) HGC_FUSED(false, true, false, false); else HGC_FUSED(false, false, false, false); }
    else if (mean_and_max && slots) { if (pow2k) HGC_FUSED(true, true, true, true); else HGC_FUSED(true, false, true, true); }
    else if (mean_and_max) { if (pow2k) HGC_FUSED(true, true, false, true); else HGC_FUSED(true, false, false, true); }
    else { if (pow2k) HGC_FUSED(false, true, false, true); else HGC_FUSED(false, false, false, true); }
#undef HGC_FUSED
    return check_launch("accumulate_grad_fused_kernel");
}

}  // namespace

int launch_zero_padded_weight_grad(const int *inv_off, const int *inv_slots, float *gw, int n_vert, long long total,
                                   hipStream_t s) {
    zero_padded_weight_grad_kernel<<<256, 256, 0, s>>>(inv_off, inv_slots, gw, n_vert, total);
    return check_launch("zero_padded_weight_grad_kernel");
}

int launch_accumulate_grad_fused(const float *g, const float *w, const float *feat, const int *maxidx,
                                 const unsigned char *maxslot, const int *inv_off, const int *inv_slots, float *gw,
                                 float *gfeat, int n_vert, int K, int F, int g_cols, bool mean_and_max, const int *idx,
                                 const int *order, float divisor, hipStream_t s) {
    // gw == nullptr: the feature gradient alone (mean only; with the max part the two-kernel path does it)
    const bool want_w = gw != nullptr;
    if (F < 16 || (!want_w && mean_and_max)) return 1;
    const bool partial = F % kWave != 0;  // the last block of 64 lanes is not full
    if (partial && n_vert >= (1 << (32 - kKeyBits))) return 1;  // vertex and slot share one word there
    const uintptr_t align_or = reinterpret_cast<uintptr_t>(g) | reinterpret_cast<uintptr_t>(feat) |
                               reinterpret_cast<uintptr_t>(maxidx) | reinterpret_cast<uintptr_t>(gfeat);
    // rows are addressed through 32-bit buffer offsets
    if ((unsigned long long)n_vert * (unsigned long long)g_cols * 4ull >= (1ull << 32)) return 1;
    if (maxslot && K > 254) maxslot = nullptr;
    const int vec = partial ? 1 : wave_vec(F, align_or);
    const int nb = ceil_div(F, kWave * vec);
    // wider rows would not fit the register budget that keeps 5+ waves per SIMD resident
    if (nb < 1 || vec * nb > 4) return 1;

    if (want_w) {
        const int rc = launch_zero_padded_weight_grad(inv_off, inv_slots, gw, n_vert, (long long)n_vert * K, s);
        if (rc) return rc;
    }
#define HGC_ARGS                                                                                                   \
    g, w, feat, maxidx, maxslot, inv_off, inv_slots, gw, gfeat, n_vert, K, F, g_cols, mean_and_max, idx, order, divisor, \
        want_w, s
    if (partial) {
        switch (nb) {
            case 1: return launch_fused<1, 1, true>(HGC_ARGS);
            case 2: return launch_fused<1, 2, true>(HGC_ARGS);
            case 3: return launch_fused<1, 3, true>(HGC_ARGS);
        }
        return 1;
    }
    switch (vec * 10 + nb) {
        case 11: return launch_fused<1, 1, false>(HGC_ARGS);
        case 12: return launch_fused<1, 2, false>(HGC_ARGS);
        case 13: return launch_fused<1, 3, false>(HGC_ARGS);
        case 21: return launch_fused<2, 1, false>(HGC_ARGS);
        case 22: return launch_fused<2, 2, false>(HGC_ARGS);
        case 41: return launch_fused<4, 1, false>(HGC_ARGS);
    }
#undef HGC_ARGS
    return 1;
}

}  // namespace hgc
