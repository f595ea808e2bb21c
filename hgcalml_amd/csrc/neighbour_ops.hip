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
                       int n_out_feat, int mean_and_max, float divisor, const int *d_order, hgc_stream_t stream);
int accumulate_gradient(const float *d_grad_from_out_features, const float *d_distances, const float *d_feat,
                        const int *d_max_feat_indices, const unsigned char *d_max_slots, const int *d_neigh_indices,
                        const int *d_inv_offsets, const int *d_inv_slots, float *d_out_grad_distances,
                        float *d_out_grad_features, int n_vert, int n_neigh, int n_feat, int n_grad_from_out_feat,
                        int mean_and_max, float divisor, const int *d_order, hgc_stream_t stream);

namespace {

// One thread per (vertex i, coordinate c). d(dist_ik)/d(x_i) summed over the
// vertex's own neighbours first, in slot order, then the terms of every (v, n)
// that names i, in ascending (v, n) order. Each term is formed in double and
// rounded once, as the reference's `2. * g * (x_k - x_i)` is.
__global__ __launch_bounds__(256) void select_knn_grad_kernel(const float *__restrict__ grad_dist,
                                                              const int *__restrict__ idx,
                                                              const float *__restrict__ coord,
                                                              const int *__restrict__ inv_off,
                                                              const int *__restrict__ inv_slots,
                                                              float *__restrict__ grad_coord, int n_vert, int K, int C,
                                                              const acc::FastDiv div_k) {
    const long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const int i = (int)(t / C);
    if (i >= n_vert) return;
    const int c = (int)(t - (long long)i * C);
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
// missing neighbour and for the vertex itself
__global__ __launch_bounds__(256) void local_distance_kernel(const int *__restrict__ idx,
                                                             const float *__restrict__ coord,
                                                             float *__restrict__ dist, int C, int n_in_vert,
                                                             long long total, int K) {
    const long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= total) return;
    const int i = (int)(t / K);
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

}  // namespace
}  // namespace hgc

using namespace hgc;

extern "C" {

int hgc_select_knn_grad(const float *d_grad_dist, const int *d_indices, const float *d_dist, const float *d_coord,
                        const int *d_inv_offsets, const int *d_inv_slots, float *d_grad_coord, int n_vert, int n_neigh,
                        int n_coords, hgc_stream_t stream) {
    (void)d_dist;  // carried by the reference op, not used by its kernels
    HGC_REQUIRE(n_vert >= 0 && n_neigh >= 1 && n_coords >= 1, "bad sizes");
    HGC_REQUIRE((long long)n_vert * std::max(n_neigh, n_coords) < (1ll << 31), "tensor too large for int32 indexing");
    if (n_vert == 0) return HGC_OK;
    HGC_REQUIRE(d_grad_dist && d_indices && d_coord && d_inv_offsets && d_inv_slots && d_grad_coord, "null pointer");
    const long long threads = (long long)n_vert * n_coords;
    select_knn_grad_kernel<<<ceil_div(threads, 256), 256, 0, as_stream(stream)>>>(
        d_grad_dist, d_indices, d_coord, d_inv_offsets, d_inv_slots, d_grad_coord, n_vert, n_neigh, n_coords,
        acc::make_fast_div(n_neigh));
    return check_launch("select_knn_grad_kernel");
}

int hgc_local_distance(const int *d_neigh_idxs, const float *d_coords, float *d_distances, int n_coords, int n_in_vert,
                       int n_out_vert, int n_neigh, hgc_stream_t stream) {
    HGC_REQUIRE(n_in_vert >= 0 && n_out_vert >= 0 && n_out_vert <= n_in_vert && n_neigh >= 1 && n_coords >= 1,
                "bad sizes");
    HGC_REQUIRE((long long)n_out_vert * n_neigh < (1ll << 31), "tensor too large for int32 indexing");
    if (n_out_vert == 0) return HGC_OK;
    HGC_REQUIRE(d_neigh_idxs && d_coords && d_distances, "null pointer");
    const long long total = (long long)n_out_vert * n_neigh;
    local_distance_kernel<<<ceil_div(total, 256), 256, 0, as_stream(stream)>>>(d_neigh_idxs, d_coords, d_distances,
                                                                              n_coords, n_in_vert, total, n_neigh);
    return check_launch("local_distance_kernel");
}

int hgc_push_knn(const float *d_weights, const float *d_feat, const int *d_idxs, const int *d_inv_offsets,
                 const int *d_inv_slots, float *d_out_feat, int n_vert, int n_neigh, int n_feat, hgc_stream_t stream) {
    (void)d_idxs;  // the inverse index carries all the op needs of the neighbour table
    HGC_REQUIRE(n_vert <= 0 || d_out_feat, "null pointer");
    // out[m, f] = sum over (v, n) naming m of feat[v, f] * w[v, n]: the mean-only
    // feature gradient of the accumulation with `feat` as upstream gradient, not divided by K
    return accumulate_gradient(d_feat, d_weights, nullptr, nullptr, nullptr, nullptr, d_inv_offsets, d_inv_slots,
                               nullptr, d_out_feat, n_vert, n_neigh, n_feat, n_feat, 0, 1.f, nullptr, stream);
}

int hgc_push_knn_grad(const float *d_grad, const float *d_weights, const float *d_feat, const int *d_idxs,
                      float *d_feat_grad, float *d_w_grad, int n_vert, int n_neigh, int n_feat, hgc_stream_t stream) {
    HGC_REQUIRE(n_vert <= 0 || (d_feat_grad && d_w_grad), "null pointer");
    // feat_grad[v, f] = sum_n grad[idx[v,n], f] * w[v,n]: the mean-only forward over `grad`, not divided by K
    int rc = accumulate_forward(d_weights, d_grad, d_idxs, d_feat_grad, nullptr, nullptr, n_vert, n_neigh, n_feat,
                                n_feat, 0, 1.f, nullptr, stream);
    if (rc) return rc;
    // w_grad[v, n] = sum_f grad[idx[v,n], f] * feat[v, f]: the weight gradient with the roles of the
    // vertex's own row (feat) and the gathered rows (grad) as in the accumulation's
    return accumulate_gradient(d_feat, nullptr, d_grad, nullptr, nullptr, d_idxs, nullptr, nullptr, d_w_grad, nullptr,
                               n_vert, n_neigh, n_feat, n_feat, 0, 1.f, nullptr, stream);
}

}  // extern "C"
