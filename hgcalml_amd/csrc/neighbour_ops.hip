// Ops next to the accumulate path that run over the same neighbour table:
//   * coordinate gradient of the kNN distances (SelectKnnGrad),
//   * push_knn forward and gradient.
//
// Reference behaviour restated here:
//   modules/compiled/select_knn_grad_kernel.cu.cc:81-164
//   modules/compiled/push_knn_kernel.cc:40-62
//   modules/compiled/push_knn_grad_kernel.cc:23-71
//   modules/compiled/local_distance_kernel.cc:18-70
//
// The reference's device kernels scatter with atomicAdd; here every scatter is
// an ordered gather through the inverse neighbour index (ascending (vertex,
// slot) per target), so results do not depend on scheduling.
#include "accumulate_rows.hpp"

#include <algorithm>

namespace hgc {

// accumulate.hip
int accumulate_forward(const float *d_distances, const float *d_feat, const int *d_idxs, float *d_out_feat,
                       int *d_out_maxidxs, unsigned char *d_out_maxslots, int n_vert, int n_neigh, int n_feat,
                       int n_out_feat, int mean_and_max, float divisor, const int *d_order, float *d_out_weights,
                       hgc_stream_t stream);
int accumulate_gradient(const float *d_grad_from_out_features, const float *d_distances, const float *d_feat,
                        const int *d_max_feat_indices, const unsigned char *d_max_slots, const int *d_neigh_indices,
                        const int *d_inv_offsets, const int *d_inv_slots, float *d_out_grad_distances,
                        float *d_out_grad_features, int n_vert, int n_neigh, int n_feat, int n_grad_from_out_feat,
                        int mean_and_max, float divisor, const int *d_order, void *records, size_t records_bytes,
                        hgc_stream_t stream);

namespace {

// One thread per (vertex i, coordinate c). d(dist_ik)/d(x_i) summed over the
// vertex's own neighbours first, in slot order, then the terms of every (v, n)
// that names i, in ascending (v, n) order. Each term is formed in double and
// rounded once, as the reference's `2. * g * (x_k - x_i)` is. With a processing
// order (a permutation of the vertices, e.g. the kNN's bin order) neighbouring
// threads work on vertices that share neighbours, whose coordinates then come
// from the first-level cache; the results do not depend on it.
__global__ __launch_bounds__(256) void select_knn_grad_kernel(const float *__restrict__ grad_dist,
                                                              const int *__restrict__ idx,
                                                              const float *__restrict__ coord,
                                                              const int *__restrict__ inv_off,
                                                              const int *__restrict__ inv_slots,
                                                              float *__restrict__ grad_coord, int n_vert, int K, int C,
                                                              const acc::FastDiv div_k,
                                                              const int *__restrict__ order) {
    const long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const int r = (int)(t / C);
    if (r >= n_vert) return;
    const int c = (int)(t - (long long)r * C);
    const int i = order ? order[r] : r;
    if ((uint32_t)i >= (uint32_t)n_vert) return;  // not a permutation: that vertex is left out
    const float xi = coord[(size_t)i * C + c];

    // loads of U slots are issued together; the additions stay in slot / list order
    constexpr int U = 8;
    float sum = 0.f;
    for (int n0 = 0; n0 < K; n0 += U) {
        int k[U];
        float g[U], xk[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int n = min(n0 + u, K - 1);
            k[u] = idx[(size_t)i * K + n];
            g[u] = grad_dist[(size_t)i * K + n];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const bool ok = n0 + u < K && k[u] >= 0 && k[u] < n_vert;
            k[u] = ok ? k[u] : -1;
            xk[u] = coord[(size_t)(ok ? k[u] : i) * C + c];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (k[u] < 0) continue;
            const float diff = xk[u] - xi;
            sum = (float)((double)sum - 2. * (double)g[u] * (double)diff);
        }
    }
    const int begin = inv_off[i], end = inv_off[i + 1];
    for (int e0 = begin; e0 < end; e0 += U) {
        int slot[U];
        float g[U], xv[U];
#pragma unroll
        for (int u = 0; u < U; ++u) slot[u] = inv_slots[min(e0 + u, end - 1)];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            g[u] = grad_dist[slot[u]];
            xv[u] = coord[(size_t)acc::fast_div(slot[u], div_k) * C + c];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (e0 + u >= end) break;
            const float diff = xi - xv[u];
            const float add = (float)(2. * (double)g[u] * (double)diff);
            sum = sum + add;
        }
    }
    grad_coord[(size_t)i * C + c] = sum;
}

// one thread per (vertex, slot): serial fp32 sum over the coordinates, 0 for a
// missing neighbour and for the vertex itself (order: see select_knn_grad_kernel)
__global__ __launch_bounds__(256) void local_distance_kernel(const int *__restrict__ idx,
                                                             const float *__restrict__ coord,
                                                             float *__restrict__ dist, int C, int n_in_vert,
                                                             long long total, int K, const int *__restrict__ order,
                                                             int n_out_vert) {
    long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= total) return;
    int i = (int)(t / K);
    if (order) {
        const int n = (int)(t - (long long)i * K);
        i = order[i];
        if ((uint32_t)i >= (uint32_t)n_out_vert) return;  // not a permutation: that vertex is left out
        t = (long long)i * K + n;
    }
    const int j = idx[t];
    float dsq = 0.f;
    if (j >= 0 && j < n_in_vert && j != i) {
        for (int c = 0; c < C; ++c) {
            const float d = coord[(size_t)i * C + c] - coord[(size_t)j * C + c];
            dsq = dsq + d * d;
        }
    }
    dist[t] = dsq;
}

// Gradient of push_knn, both outputs from one gather: a wave owns vertex v,
// fetches the upstream gradient rows of its K neighbours once and forms
//   feat_grad[v, f] = sum_n grad[idx[v,n], f] * w[v,n]   (serial, slot order: the reference's sum)
//   w_grad[v, n]    = sum_f grad[idx[v,n], f] * feat[v, f]
// the second as per-lane partial dot products that a fixed transpose-butterfly
// reduces for 32 slots at a time. Lane l owns features [l*VEC, l*VEC+VEC) of each
// of the NB blocks of 64*VEC features.
template <int VEC, int NB>
__global__ __launch_bounds__(256) void push_grad_wave_kernel(const float *__restrict__ grad, const float *__restrict__ w,
                                                             const float *__restrict__ feat, const int *__restrict__ idx,
                                                             float *__restrict__ feat_grad, float *__restrict__ w_grad,
                                                             int n_vert, int K, int F) {
    using namespace acc;
    constexpr int G = 32;  // slots per reduction
    constexpr int U = 8;   // gathered rows in flight
    const int v = wave_vertex(nullptr, n_vert);
    if (v >= n_vert) return;
    const int lane = lane_id();
    const int *irow = idx + (size_t)v * K;
    const float *wrow = w + (size_t)v * K;
    const RowMatrix X(grad, n_vert, F);
    uint32_t lane_bytes[NB];
    float own[NB][VEC], sum[NB][VEC];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        const int fb = (b * kWave + lane) * VEC;
        lane_bytes[b] = (uint32_t)fb * 4u;
        load_vec<VEC>(feat + (size_t)v * F + fb, own[b]);
#pragma unroll
        for (int e = 0; e < VEC; ++e) sum[b][e] = 0.f;
    }
    for (int l0 = 0; l0 < K; l0 += G) {
        float val[G];
#pragma unroll
        for (int i = 0; i < G; ++i) val[i] = 0.f;
#pragma unroll
        for (int u0 = 0; u0 < G; u0 += U) {
            if (l0 + u0 >= K) break;  // wave-uniform
            int j[U];
            float wl[U];
            float x[U][NB][VEC];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int l = min(l0 + u0 + u, K - 1);
                j[u] = l0 + u0 + u < K ? irow[l] : -1;
                wl[u] = wrow[l];
            }
            // slots without a neighbour read row 0 and are left out of the sum; their
            // weight gradient is overwritten with 0 below
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int b = 0; b < NB; ++b)
                    X.load<VEC>((uint32_t)j[u] < (uint32_t)n_vert ? j[u] : 0, lane_bytes[b], x[u][b]);
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const bool valid = (uint32_t)j[u] < (uint32_t)n_vert;  // wave-uniform
#pragma unroll
                for (int b = 0; b < NB; ++b)
#pragma unroll
                    for (int e = 0; e < VEC; ++e) {
                        val[u0 + u] = __builtin_fmaf(own[b][e], x[u][b][e], val[u0 + u]);
                        if (valid) sum[b][e] = sum[b][e] + x[u][b][e] * wl[u];
                    }
            }
        }
        const float r = transpose_reduce_32(val);  // lane L: slot l0 + (L & 31)
        const int l = l0 + lane;
        if (lane < G && l < K) w_grad[(size_t)v * K + l] = (uint32_t)irow[l] < (uint32_t)n_vert ? r : 0.f;
    }
#pragma unroll
    for (int b = 0; b < NB; ++b) store_vec<VEC>(feat_grad + (size_t)v * F + (lane_bytes[b] >> 2), sum[b]);
}

// returns 1 when the shape is not covered
int launch_push_grad_wave(const float *grad, const float *w, const float *feat, const int *idx, float *feat_grad,
                          float *w_grad, int n_vert, int K, int F, hipStream_t s) {
    using namespace acc;
    if (F % kWave != 0 || (unsigned long long)n_vert * (unsigned long long)F * 4ull >= (1ull << 32)) return 1;
    const uintptr_t align_or = reinterpret_cast<uintptr_t>(grad) | reinterpret_cast<uintptr_t>(feat) |
                               reinterpret_cast<uintptr_t>(feat_grad);
    const int vec = wave_vec(F, align_or);
    const int nb = F / (kWave * vec);
    const dim3 grid(ceil_div(n_vert, 4)), block(256);
#define HGC_PUSH_GRAD(VEC, NB) \
    push_grad_wave_kernel<VEC, NB><<<grid, block, 0, s>>>(grad, w, feat, idx, feat_grad, w_grad, n_vert, K, F)
    switch (vec * 10 + nb) {
        case 11: HGC_PUSH_GRAD(1, 1); break;
        case 12: HGC_PUSH_GRAD(1, 2); break;
        case 13: HGC_PUSH_GRAD(1, 3); break;
        case 21: HGC_PUSH_GRAD(2, 1); break;
        case 41: HGC_PUSH_GRAD(4, 1); break;
        default: return 1;
    }
#undef HGC_PUSH_GRAD
    return check_launch("push_grad_wave_kernel");
}

}  // namespace
}  // namespace hgc

using namespace hgc;

namespace {

// weights of AccumulateKnn, w = exp(-d) (modules/accknn_op.py:52), and the chain rule back to
// the distances, gd = -(gw * w): one pass each instead of two framework kernels
__global__ __launch_bounds__(256) void exp_neg_kernel(const float *__restrict__ d, float *__restrict__ w,
                                                      long long n) {
    const long long i = ((long long)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (i + 4 <= n) {
        const float4 v = *reinterpret_cast<const float4 *>(d + i);
        *reinterpret_cast<float4 *>(w + i) = float4{expf(-v.x), expf(-v.y), expf(-v.z), expf(-v.w)};
    } else {
        for (long long j = i; j < n; ++j) w[j] = expf(-d[j]);
    }
}

__global__ __launch_bounds__(256) void exp_neg_grad_kernel(const float *__restrict__ gw, const float *__restrict__ w,
                                                           float *__restrict__ gd, long long n) {
    const long long i = ((long long)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (i + 4 <= n) {
        const float4 a = *reinterpret_cast<const float4 *>(gw + i), b = *reinterpret_cast<const float4 *>(w + i);
        *reinterpret_cast<float4 *>(gd + i) = float4{-(a.x * b.x), -(a.y * b.y), -(a.z * b.z), -(a.w * b.w)};
    } else {
        for (long long j = i; j < n; ++j) gd[j] = -(gw[j] * w[j]);
    }
}


// ---- feature-weighted moments of the neighbours' coordinates ----------------------
//
// modules/neighbour_covariance_op.py:8-62 builds, with w = exp(-distsq) and a = the
// (activated) features,
//   S[v,f]       = sum_n w[v,n] a[j,f]
//   mean[v,f,c]  = sum_n w[v,n] a[j,f] x[j,c] / (S[v,f] + 1e-3)
//   cov[v,f,c,d] = sum_n w[v,n] a[j,f] (x[j,c] - mean[j,f,c]) (x[j,d] - mean[j,f,d]) / (S[v,f] + 1e-3)
// (j = idx[v,n]; every neighbour is centred on ITS OWN mean) out of three mean-only
// accumulations over matrices of F, F*C and F*C*C columns that it materialises first.
// Here two passes over the neighbour table do it, one thread per (vertex, feature): the
// first gathers a[j,f] and x[j,:], the second a[j,f], x[j,:] and mean[j,f,:] and forms the
// C*C products in registers. The sums run over the slots in order and every term is formed
// as the composition forms it -- ((x*a)*w, ((cen_c*cen_d)*a)*w, the sum divided by K and
// multiplied by K again as the accumulation's mean is) -- so the results are its bits.

__device__ __forceinline__ float divide_no_nan(float a, float b) { return b == 0.f ? 0.f : a / b; }

template <int C>
__global__ __launch_bounds__(256) void neighbour_means_kernel(const float *__restrict__ coords,
                                                              const float *__restrict__ weights,
                                                              const float *__restrict__ feats, const int *__restrict__ idx,
                                                              float *__restrict__ sumw, float *__restrict__ means,
                                                              const int *__restrict__ order, int n_vert, int n_feat,
                                                              int n_neigh) {
    const long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const int i = (int)(t / n_feat);
    if (i >= n_vert) return;
    const int f = (int)(t - (long long)i * n_feat);
    const int v = order ? order[i] : i;  // processing order with locality: results do not depend on it
    if ((unsigned)v >= (unsigned)n_vert) return;
    const float kf = (float)n_neigh;
    float s = 0.f, sc[C];
#pragma unroll
    for (int c = 0; c < C; ++c) sc[c] = 0.f;
    for (int n = 0; n < n_neigh; ++n) {
        const int j = idx[(size_t)v * n_neigh + n];
        if ((unsigned)j >= (unsigned)n_vert) continue;
        const float w = weights[(size_t)v * n_neigh + n];
        const float a = feats[(size_t)j * n_feat + f];
        s = s + a * w;
#pragma unroll
        for (int c = 0; c < C; ++c) sc[c] = sc[c] + (coords[(size_t)j * C + c] * a) * w;
    }
    const float S = (s / kf) * kf;
    sumw[(size_t)v * n_feat + f] = S;
#pragma unroll
    for (int c = 0; c < C; ++c) means[((size_t)v * n_feat + f) * C + c] = divide_no_nan((sc[c] / kf) * kf, S + 1e-3f);
}

template <int C>
__global__ __launch_bounds__(256) void neighbour_covariance_kernel(const float *__restrict__ coords,
                                                                   const float *__restrict__ weights,
                                                                   const float *__restrict__ feats,
                                                                   const int *__restrict__ idx,
                                                                   const float *__restrict__ sumw,
                                                                   const float *__restrict__ means, float *__restrict__ cov,
                                                                   const int *__restrict__ order, int n_vert, int n_feat,
                                                                   int n_neigh) {
    const long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const int i = (int)(t / n_feat);
    if (i >= n_vert) return;
    const int f = (int)(t - (long long)i * n_feat);
    const int v = order ? order[i] : i;
    if ((unsigned)v >= (unsigned)n_vert) return;
    const float kf = (float)n_neigh;
    float acc[C][C];  // the lower triangle is accumulated, the products are symmetric bit for bit
#pragma unroll
    for (int c = 0; c < C; ++c)
#pragma unroll
        for (int d = 0; d < C; ++d) acc[c][d] = 0.f;
    for (int n = 0; n < n_neigh; ++n) {
        const int j = idx[(size_t)v * n_neigh + n];
        if ((unsigned)j >= (unsigned)n_vert) continue;
        const float w = weights[(size_t)v * n_neigh + n];
        const float a = feats[(size_t)j * n_feat + f];
        float cen[C];
#pragma unroll
        for (int c = 0; c < C; ++c) cen[c] = coords[(size_t)j * C + c] - means[((size_t)j * n_feat + f) * C + c];
#pragma unroll
        for (int c = 0; c < C; ++c)
#pragma unroll
            for (int d = 0; d <= c; ++d) acc[c][d] = acc[c][d] + ((cen[c] * cen[d]) * a) * w;
    }
    const float den = sumw[(size_t)v * n_feat + f] + 1e-3f;
    float *out = cov + ((size_t)v * n_feat + f) * C * C;
#pragma unroll
    for (int c = 0; c < C; ++c)
#pragma unroll
        for (int d = 0; d < C; ++d) out[c * C + d] = divide_no_nan((acc[c > d ? c : d][c > d ? d : c] / kf) * kf, den);
}

template <int C>
int launch_neighbour_covariance(const float *coords, const float *weights, const float *feats, const int *idx, float *cov,
                                float *means, float *sumw, const int *order, int n_vert, int n_feat, int n_neigh,
                                hipStream_t s) {
    const int blocks = ceil_div((long long)n_vert * n_feat, 256);
    neighbour_means_kernel<C><<<blocks, 256, 0, s>>>(coords, weights, feats, idx, sumw, means, order, n_vert, n_feat,
                                                     n_neigh);
    int rc = check_launch("neighbour_means_kernel");
    if (rc) return rc;
    neighbour_covariance_kernel<C><<<blocks, 256, 0, s>>>(coords, weights, feats, idx, sumw, means, cov, order, n_vert,
                                                          n_feat, n_neigh);
    return check_launch("neighbour_covariance_kernel");
}

}  // namespace

extern "C" {

int hgc_neighbour_covariance(const float *d_coords, const float *d_weights, const float *d_feats, const int *d_n_idxs,
                             const int *d_vertex_order, float *d_covariance, float *d_means, float *d_sum_weights,
                             int n_vert, int n_coords, int n_feat, int n_neigh, hgc_stream_t stream) {
    HGC_REQUIRE(n_vert >= 0 && n_coords >= 1 && n_feat >= 1 && n_neigh >= 1, "bad sizes");
    if (n_coords > 6) return fail(HGC_ERR_UNSUPPORTED, "neighbour covariance is built for up to 6 coordinates");
    HGC_REQUIRE((long long)n_vert * std::max(n_neigh, n_feat * n_coords * n_coords) < (1ll << 31),
                "tensor too large for int32 indexing");
    if (n_vert == 0) return HGC_OK;
    HGC_REQUIRE(d_coords && d_weights && d_feats && d_n_idxs && d_covariance && d_means && d_sum_weights, "null pointer");
    hipStream_t s = as_stream(stream);
#define HGC_COV(C)                                                                                                  \
    case C:                                                                                                         \
        return launch_neighbour_covariance<C>(d_coords, d_weights, d_feats, d_n_idxs, d_covariance, d_means,        \
                                              d_sum_weights, d_vertex_order, n_vert, n_feat, n_neigh, s)
    switch (n_coords) {
        HGC_COV(1);
        HGC_COV(2);
        HGC_COV(3);
        HGC_COV(4);
        HGC_COV(5);
        HGC_COV(6);
    }
#undef HGC_COV
    return HGC_ERR_UNSUPPORTED;
}

int hgc_select_knn_grad_ordered(const float *d_grad_dist, const int *d_indices, const float *d_dist,
                                const float *d_coord, const int *d_inv_offsets, const int *d_inv_slots,
                                const int *d_vertex_order, float *d_grad_coord, int n_vert, int n_neigh, int n_coords,
                                hgc_stream_t stream) {
    (void)d_dist;  // carried by the reference op, not used by its kernels
    HGC_REQUIRE(n_vert >= 0 && n_neigh >= 1 && n_coords >= 1, "bad sizes");
    HGC_REQUIRE((long long)n_vert * std::max(n_neigh, n_coords) < (1ll << 31), "tensor too large for int32 indexing");
    if (n_vert == 0) return HGC_OK;
    HGC_REQUIRE(d_grad_dist && d_indices && d_coord && d_inv_offsets && d_inv_slots && d_grad_coord, "null pointer");
    const long long threads = (long long)n_vert * n_coords;
    select_knn_grad_kernel<<<ceil_div(threads, 256), 256, 0, as_stream(stream)>>>(
        d_grad_dist, d_indices, d_coord, d_inv_offsets, d_inv_slots, d_grad_coord, n_vert, n_neigh, n_coords,
        acc::make_fast_div(n_neigh), d_vertex_order);
    return check_launch("select_knn_grad_kernel");
}

int hgc_select_knn_grad(const float *d_grad_dist, const int *d_indices, const float *d_dist, const float *d_coord,
                        const int *d_inv_offsets, const int *d_inv_slots, float *d_grad_coord, int n_vert, int n_neigh,
                        int n_coords, hgc_stream_t stream) {
    return hgc_select_knn_grad_ordered(d_grad_dist, d_indices, d_dist, d_coord, d_inv_offsets, d_inv_slots, nullptr,
                                       d_grad_coord, n_vert, n_neigh, n_coords, stream);
}

int hgc_local_distance_ordered(const int *d_neigh_idxs, const float *d_coords, const int *d_vertex_order,
                               float *d_distances, int n_coords, int n_in_vert, int n_out_vert, int n_neigh,
                               hgc_stream_t stream) {
    HGC_REQUIRE(n_in_vert >= 0 && n_out_vert >= 0 && n_out_vert <= n_in_vert && n_neigh >= 1 && n_coords >= 1,
                "bad sizes");
    HGC_REQUIRE((long long)n_out_vert * n_neigh < (1ll << 31), "tensor too large for int32 indexing");
    if (n_out_vert == 0) return HGC_OK;
    HGC_REQUIRE(d_neigh_idxs && d_coords && d_distances, "null pointer");
    const long long total = (long long)n_out_vert * n_neigh;
    local_distance_kernel<<<ceil_div(total, 256), 256, 0, as_stream(stream)>>>(
        d_neigh_idxs, d_coords, d_distances, n_coords, n_in_vert, total, n_neigh, d_vertex_order, n_out_vert);
    return check_launch("local_distance_kernel");
}

int hgc_local_distance(const int *d_neigh_idxs, const float *d_coords, float *d_distances, int n_coords, int n_in_vert,
                       int n_out_vert, int n_neigh, hgc_stream_t stream) {
    return hgc_local_distance_ordered(d_neigh_idxs, d_coords, nullptr, d_distances, n_coords, n_in_vert, n_out_vert,
                                      n_neigh, stream);
}

int hgc_push_knn_ordered(const float *d_weights, const float *d_feat, const int *d_idxs, const int *d_inv_offsets,
                         const int *d_inv_slots, const int *d_vertex_order, float *d_out_feat, int n_vert, int n_neigh,
                         int n_feat, hgc_stream_t stream) {
    (void)d_idxs;  // the inverse index carries all the op needs of the neighbour table
    HGC_REQUIRE(n_vert <= 0 || d_out_feat, "null pointer");
    // out[m, f] = sum over (v, n) naming m of feat[v, f] * w[v, n]: the mean-only
    // feature gradient of the accumulation with `feat` as upstream gradient, not divided by K
    return accumulate_gradient(d_feat, d_weights, nullptr, nullptr, nullptr, nullptr, d_inv_offsets, d_inv_slots,
                               nullptr, d_out_feat, n_vert, n_neigh, n_feat, n_feat, 0, 1.f, d_vertex_order, nullptr, 0,
                               stream);
}

int hgc_push_knn(const float *d_weights, const float *d_feat, const int *d_idxs, const int *d_inv_offsets,
                 const int *d_inv_slots, float *d_out_feat, int n_vert, int n_neigh, int n_feat, hgc_stream_t stream) {
    return hgc_push_knn_ordered(d_weights, d_feat, d_idxs, d_inv_offsets, d_inv_slots, nullptr, d_out_feat, n_vert,
                                n_neigh, n_feat, stream);
}

int hgc_push_knn_grad(const float *d_grad, const float *d_weights, const float *d_feat, const int *d_idxs,
                      float *d_feat_grad, float *d_w_grad, int n_vert, int n_neigh, int n_feat, hgc_stream_t stream) {
    HGC_REQUIRE(n_vert <= 0 || (d_feat_grad && d_w_grad), "null pointer");
    HGC_REQUIRE(n_vert >= 0 && n_neigh >= 1 && n_feat >= 1, "bad sizes");
    HGC_REQUIRE((long long)n_vert * n_neigh < (1ll << 31), "n_vert * n_neigh must stay below 2^31");
    if (n_vert == 0) return HGC_OK;
    HGC_REQUIRE(d_grad && d_weights && d_feat && d_idxs, "null pointer");
    {
        // both gradients from one gather pass where that kernel covers the shape
        const int rc = launch_push_grad_wave(d_grad, d_weights, d_feat, d_idxs, d_feat_grad, d_w_grad, n_vert, n_neigh,
                                             n_feat, as_stream(stream));
        if (rc <= 0) return rc;
    }
    // feat_grad[v, f] = sum_n grad[idx[v,n], f] * w[v,n]: the mean-only forward over `grad`, not divided by K
    int rc = accumulate_forward(d_weights, d_grad, d_idxs, d_feat_grad, nullptr, nullptr, n_vert, n_neigh, n_feat,
                                n_feat, 0, 1.f, nullptr, nullptr, stream);
    if (rc) return rc;
    // w_grad[v, n] = sum_f grad[idx[v,n], f] * feat[v, f]: the weight gradient with the roles of the
    // vertex's own row (feat) and the gathered rows (grad) as in the accumulation's
    return accumulate_gradient(d_feat, nullptr, d_grad, nullptr, nullptr, d_idxs, nullptr, nullptr, d_w_grad, nullptr,
                               n_vert, n_neigh, n_feat, n_feat, 0, 1.f, nullptr, nullptr, 0, stream);
}

int hgc_exp_neg(const float *d_distances, float *d_weights, long long n_values, hgc_stream_t stream) {
    HGC_REQUIRE(n_values >= 0, "bad sizes");
    if (n_values == 0) return HGC_OK;
    HGC_REQUIRE(d_distances && d_weights, "null pointer");
    HGC_REQUIRE(((reinterpret_cast<uintptr_t>(d_distances) | reinterpret_cast<uintptr_t>(d_weights)) & 15u) == 0,
                "arrays must start on a 16-byte boundary");
    exp_neg_kernel<<<ceil_div(ceil_div(n_values, 4), 256), 256, 0, as_stream(stream)>>>(d_distances, d_weights,
                                                                                       n_values);
    return check_launch("exp_neg");
}

int hgc_exp_neg_grad(const float *d_weight_grad, const float *d_weights, float *d_distance_grad, long long n_values,
                     hgc_stream_t stream) {
    HGC_REQUIRE(n_values >= 0, "bad sizes");
    if (n_values == 0) return HGC_OK;
    HGC_REQUIRE(d_weight_grad && d_weights && d_distance_grad, "null pointer");
    HGC_REQUIRE(((reinterpret_cast<uintptr_t>(d_weight_grad) | reinterpret_cast<uintptr_t>(d_weights) |
                  reinterpret_cast<uintptr_t>(d_distance_grad)) & 15u) == 0,
                "arrays must start on a 16-byte boundary");
    exp_neg_grad_kernel<<<ceil_div(ceil_div(n_values, 4), 256), 256, 0, as_stream(stream)>>>(
        d_weight_grad, d_weights, d_distance_grad, n_values);
    return check_launch("exp_neg_grad");
}

}  // extern "C"
