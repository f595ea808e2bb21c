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
#include "hgc_common.hpp"

#include <cstring>
#include <algorithm>

#include <rocprim/rocprim.hpp>

namespace hgc {

int launch_fill_i32(int *p, int value, long long n, hipStream_t s);

namespace {

// ------------------------------------------------------------------ forward

template <int VEC>
struct FeatVec;
template <>
struct FeatVec<4> {
    using type = float4;
};
template <>
struct FeatVec<1> {
    using type = float;
};

template <int VEC>
__device__ __forceinline__ void load_vec(const float *p, float (&x)[VEC]) {
    if constexpr (VEC == 4) {
        const float4 v = *reinterpret_cast<const float4 *>(p);
        x[0] = v.x; x[1] = v.y; x[2] = v.z; x[3] = v.w;
    } else {
        x[0] = *p;
    }
}

template <int VEC>
__device__ __forceinline__ void store_vec(float *p, const float (&x)[VEC]) {
    if constexpr (VEC == 4) {
        *reinterpret_cast<float4 *>(p) = make_float4(x[0], x[1], x[2], x[3]);
    } else {
        *p = x[0];
    }
}

template <int VEC>
__device__ __forceinline__ void store_vec_i(int *p, const int (&x)[VEC]) {
    if constexpr (VEC == 4) {
        *reinterpret_cast<int4 *>(p) = make_int4(x[0], x[1], x[2], x[3]);
    } else {
        *p = x[0];
    }
}

constexpr int kUnroll = 8;

// one thread per (vertex, VEC consecutive features); threads of one vertex are
// adjacent lanes
template <int VEC, bool MAX>
__global__ __launch_bounds__(256) void accumulate_fwd_kernel(const float *__restrict__ w, const float *__restrict__ feat,
                                                             const int *__restrict__ idx, float *__restrict__ out,
                                                             int *__restrict__ out_maxidx, int n_vert, int K, int F,
                                                             int out_cols) {
    const int tpv = F / VEC;  // threads per vertex
    const long long t = (long long)xcd_contiguous_block(blockIdx.x, gridDim.x) * blockDim.x + threadIdx.x;
    const int v = (int)(t / tpv);
    if (v >= n_vert) return;
    const int f0 = (int)(t - (long long)v * tpv) * VEC;

    const int *irow = idx + (size_t)v * K;
    const float *wrow = w + (size_t)v * K;
    float sum[VEC], best[VEC];
    int arg[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
        sum[e] = 0.f;
        best[e] = 0.f;
        arg[e] = 0;
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
                }
            }
        }
    }

    const float kf = (float)K;
    float mean[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) mean[e] = sum[e] / kf;
    store_vec<VEC>(out + (size_t)v * out_cols + f0, mean);
    if (MAX) {
        store_vec<VEC>(out + (size_t)v * out_cols + F + f0, best);
        store_vec_i<VEC>(out_maxidx + (size_t)v * F + f0, arg);
    }
}

// ------------------------------------------------------------------ inverse index

__global__ __launch_bounds__(256) void inverse_keys_kernel(const int *__restrict__ idx, unsigned int *__restrict__ keys,
                                                           int *__restrict__ slots, long long total, int n_vert) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int j = idx[i];
    keys[i] = (unsigned)j < (unsigned)n_vert ? (unsigned)j : (unsigned)n_vert;  // invalid -> sorts last
    slots[i] = (int)i;
}

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

// ------------------------------------------------------------------ feature gradient

// gfeat[m, f] = sum over (v, n) naming m, ascending, of ((g[v,f]/K)*w[v,n] + max part)
template <int VEC, bool MAX, bool POW2K>
__global__ __launch_bounds__(256) void feature_grad_kernel(const float *__restrict__ g, const float *__restrict__ w,
                                                           const int *__restrict__ maxidx,
                                                           const int *__restrict__ inv_off,
                                                           const int *__restrict__ inv_slots,
                                                           float *__restrict__ gfeat, int n_vert, int K, int F,
                                                           int g_cols) {
    const int tpv = F / VEC;
    const long long t = (long long)xcd_contiguous_block(blockIdx.x, gridDim.x) * blockDim.x + threadIdx.x;
    const int m = (int)(t / tpv);
    if (m >= n_vert) return;
    const int f0 = (int)(t - (long long)m * tpv) * VEC;

    const float kf = (float)K;
    const float inv_k = 1.f / kf;  // exact when K is a power of two
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
                                                          int tpv) {
    const long long t = (long long)xcd_contiguous_block(blockIdx.x, gridDim.x) * blockDim.x + threadIdx.x;
    const int m = (int)(t / tpv);
    const int sub = (int)(t - (long long)m * tpv);
    const bool live = m < n_vert;  // keep whole waves alive for the shuffles
    const int mm = live ? m : 0;

    // features owned by this thread: f = sub*VEC + e + i*tpv*VEC
    const int stride = tpv * VEC;
    const int *irow = idx + (size_t)mm * K;
    const double inv_k = 1.0 / (double)(float)K;

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

int inverse_key_bits(int n_vert) {
    int bits = 1;
    while (bits < 32 && (1ll << bits) <= (long long)n_vert) ++bits;  // keys go up to n_vert inclusive
    return bits;
}

bool is_pow2(int x) { return x > 0 && (x & (x - 1)) == 0; }

}  // namespace
}  // namespace hgc

using namespace hgc;

extern "C" {

int hgc_accumulate_knn(const float *d_distances, const float *d_feat, const int *d_idxs, float *d_out_feat,
                       int *d_out_maxidxs, int n_vert, int n_neigh, int n_feat, int n_out_feat, int n_moments,
                       int mean_and_max, hgc_stream_t stream) {
    (void)n_moments;  // carried by the reference op, never used by its kernels
    HGC_REQUIRE(n_vert >= 0 && n_neigh >= 1 && n_feat >= 1, "bad sizes");
    HGC_REQUIRE(n_out_feat == n_feat * (mean_and_max ? 2 : 1), "n_out_feat must be n_feat * (mean_and_max ? 2 : 1)");
    HGC_REQUIRE((long long)n_vert * std::max(n_neigh, 2 * n_feat) < (1ll << 31), "tensor too large for int32 indexing");
    if (n_vert == 0) return HGC_OK;
    HGC_REQUIRE(d_distances && d_feat && d_idxs && d_out_feat, "null pointer");
    HGC_REQUIRE(!mean_and_max || d_out_maxidxs, "mean_and_max needs d_out_maxidxs");
    hipStream_t s = as_stream(stream);
    const bool vec4 = (n_feat % 4 == 0) && ((reinterpret_cast<uintptr_t>(d_feat) | reinterpret_cast<uintptr_t>(d_out_feat) |
                                             reinterpret_cast<uintptr_t>(d_out_maxidxs)) & 15u) == 0;
    const long long threads = (long long)n_vert * (vec4 ? n_feat / 4 : n_feat);
    const dim3 grid(ceil_div(threads, 256)), block(256);
    if (vec4) {
        if (mean_and_max)
            accumulate_fwd_kernel<4, true><<<grid, block, 0, s>>>(d_distances, d_feat, d_idxs, d_out_feat, d_out_maxidxs,
                                                                  n_vert, n_neigh, n_feat, n_out_feat);
        else
            accumulate_fwd_kernel<4, false><<<grid, block, 0, s>>>(d_distances, d_feat, d_idxs, d_out_feat, d_out_maxidxs,
                                                                   n_vert, n_neigh, n_feat, n_out_feat);
    } else {
        if (mean_and_max)
            accumulate_fwd_kernel<1, true><<<grid, block, 0, s>>>(d_distances, d_feat, d_idxs, d_out_feat, d_out_maxidxs,
                                                                  n_vert, n_neigh, n_feat, n_out_feat);
        else
            accumulate_fwd_kernel<1, false><<<grid, block, 0, s>>>(d_distances, d_feat, d_idxs, d_out_feat, d_out_maxidxs,
                                                                   n_vert, n_neigh, n_feat, n_out_feat);
    }
    return check_launch("accumulate_fwd_kernel");
}

size_t hgc_inverse_neighbour_index_workspace_bytes(int n_vert, int n_neigh) {
    const size_t total = std::max<size_t>((size_t)n_vert * n_neigh, 1);
    size_t temp = 0;
    (void)rocprim::radix_sort_pairs(nullptr, temp, (const unsigned int *)nullptr, (unsigned int *)nullptr,
                                    (const int *)nullptr, (int *)nullptr, total, 0,
                                    inverse_key_bits(std::max(n_vert, 1)), (hipStream_t) nullptr);
    return align_up(temp) + 3 * align_up(total * sizeof(int));
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
    Carver carve(workspace);
    unsigned int *keys = carve.take<unsigned int>(total);
    unsigned int *keys_sorted = carve.take<unsigned int>(total);
    int *slots = carve.take<int>(total);
    void *temp = carve.base + carve.used;
    size_t temp_bytes = workspace_bytes - carve.used;
    inverse_keys_kernel<<<ceil_div(total, 256), 256, 0, s>>>(d_idxs, keys, slots, total, n_vert);
    int rc = check_launch("inverse_keys");
    if (rc) return rc;
    // stable: inside one target the flat slots stay ascending, i.e. (vertex, slot) order
    HGC_HIP(rocprim::radix_sort_pairs(temp, temp_bytes, keys, keys_sorted, slots, d_inv_slots, (size_t)total, 0,
                                      inverse_key_bits(n_vert), s));
    inverse_offsets_kernel<<<ceil_div((long long)n_vert + 1, 256), 256, 0, s>>>(keys_sorted, total, d_inv_offsets, n_vert);
    return check_launch("inverse_offsets");
}

int hgc_accumulate_knn_grad(const float *d_grad_from_out_features, const float *d_distances, const float *d_feat,
                            const int *d_max_feat_indices, const int *d_neigh_indices, const int *d_inv_offsets,
                            const int *d_inv_slots, float *d_out_grad_distances, float *d_out_grad_features,
                            int n_vert, int n_neigh, int n_feat, int n_grad_from_out_feat, int n_moments,
                            int mean_and_max, hgc_stream_t stream) {
    (void)n_moments;
    HGC_REQUIRE(n_vert >= 0 && n_neigh >= 1 && n_feat >= 1, "bad sizes");
    HGC_REQUIRE(n_grad_from_out_feat == n_feat * (mean_and_max ? 2 : 1),
                "gradient width must be n_feat * (mean_and_max ? 2 : 1)");
    HGC_REQUIRE((long long)n_vert * std::max(n_neigh, 2 * n_feat) < (1ll << 31), "tensor too large for int32 indexing");
    if (n_vert == 0) return HGC_OK;
    HGC_REQUIRE(d_grad_from_out_features && d_distances && d_feat && d_neigh_indices && d_inv_offsets &&
                    d_inv_slots && d_out_grad_distances && d_out_grad_features,
                "null pointer");
    HGC_REQUIRE(!mean_and_max || d_max_feat_indices, "mean_and_max needs d_max_feat_indices");
    hipStream_t s = as_stream(stream);
    const uintptr_t align_or = reinterpret_cast<uintptr_t>(d_grad_from_out_features) | reinterpret_cast<uintptr_t>(d_feat) |
                               reinterpret_cast<uintptr_t>(d_max_feat_indices) |
                               reinterpret_cast<uintptr_t>(d_out_grad_features);
    const bool vec4 = (n_feat % 4 == 0) && (align_or & 15u) == 0;
    const bool pow2k = is_pow2(n_neigh);

    // ---- feature gradient ----
    {
        const long long threads = (long long)n_vert * (vec4 ? n_feat / 4 : n_feat);
        const dim3 grid(ceil_div(threads, 256)), block(256);
#define HGC_FG(VEC, MAX, P2)                                                                                      \
    feature_grad_kernel<VEC, MAX, P2><<<grid, block, 0, s>>>(d_grad_from_out_features, d_distances, d_max_feat_indices, \
                                                            d_inv_offsets, d_inv_slots, d_out_grad_features, n_vert, \
                                                            n_neigh, n_feat, n_grad_from_out_feat)
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
    {
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
                                                                   n_feat, n_grad_from_out_feat, tpv);
            else
                weight_grad_kernel<4, false><<<grid, block, 0, s>>>(d_grad_from_out_features, d_feat, d_max_feat_indices,
                                                                    d_neigh_indices, d_out_grad_distances, n_vert, n_neigh,
                                                                    n_feat, n_grad_from_out_feat, tpv);
        } else {
            if (mean_and_max)
                weight_grad_kernel<1, true><<<grid, block, 0, s>>>(d_grad_from_out_features, d_feat, d_max_feat_indices,
                                                                   d_neigh_indices, d_out_grad_distances, n_vert, n_neigh,
                                                                   n_feat, n_grad_from_out_feat, tpv);
            else
                weight_grad_kernel<1, false><<<grid, block, 0, s>>>(d_grad_from_out_features, d_feat, d_max_feat_indices,
                                                                    d_neigh_indices, d_out_grad_distances, n_vert, n_neigh,
                                                                    n_feat, n_grad_from_out_feat, tpv);
        }
        return check_launch("weight_grad_kernel");
    }
}

}  // extern "C"
