// Measurement aid: the bare row gather of the accumulation kernels.
//
// One wave64 per vertex fetches the K rows its neighbour table names (same
// buffer loads, same 16 rows in flight as the forward kernel) and only adds
// them up. Its run time is the floor any one-wave-per-vertex formulation of
// modules/compiled/accumulate_knn_kernel.cc:48-81 can reach on this part, i.e.
// the rate at which L2 delivers K-fold re-read rows to the compute units.
#include "accumulate_rows.hpp"

namespace hgc {
namespace {

using namespace acc;

template <int VEC>
__global__ __launch_bounds__(256) void row_gather_probe_kernel(const float *__restrict__ feat,
                                                               const int *__restrict__ idx, float *__restrict__ out,
                                                               int n_vert, int K, int F) {
    constexpr int U = 16;
    const int v = wave_vertex();
    if (v >= n_vert) return;
    const int *irow = idx + (size_t)v * K;
    const RowMatrix X(feat, n_vert, F);
    for (int fb = lane_id() * VEC; fb < F; fb += kWave * VEC) {
        const uint32_t lane_bytes = (uint32_t)fb * 4u;
        float sum[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) sum[e] = 0.f;
        int n0 = 0;
        for (; n0 + U <= K; n0 += U) {  // full chunks: all U row loads in flight
            float x[U][VEC];
            int j[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int jj = irow[n0 + u];
                j[u] = (uint32_t)jj < (uint32_t)n_vert ? jj : v;  // slots without a neighbour re-read the own row
            }
#pragma unroll
            for (int u = 0; u < U; ++u) X.load<VEC>(j[u], lane_bytes, x[u]);
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int e = 0; e < VEC; ++e) sum[e] += x[u][e];
        }
        for (; n0 < K; ++n0) {  // K not a multiple of U
            const int jj = irow[n0];
            float xs[VEC];
            X.load<VEC>((uint32_t)jj < (uint32_t)n_vert ? jj : v, lane_bytes, xs);
#pragma unroll
            for (int e = 0; e < VEC; ++e) sum[e] += xs[e];
        }
        store_vec<VEC>(out + (size_t)v * F + fb, sum);
    }
}

}  // namespace
}  // namespace hgc

using namespace hgc;

extern "C" int hgc_probe_row_gather(const float *d_feat, const int *d_idxs, float *d_out, int n_vert, int n_neigh,
                                    int n_feat, hgc_stream_t stream) {
    HGC_REQUIRE(n_vert >= 0 && n_neigh >= 1 && n_feat >= kWave && n_feat % kWave == 0,
                "the probe covers rows that are a multiple of 64 features");
    HGC_REQUIRE((unsigned long long)n_vert * (unsigned long long)n_feat * 4ull < (1ull << 32),
                "rows are addressed through 32-bit buffer offsets");
    if (n_vert == 0) return HGC_OK;
    HGC_REQUIRE(d_feat && d_idxs && d_out, "null pointer");
    const uintptr_t align_or = reinterpret_cast<uintptr_t>(d_feat) | reinterpret_cast<uintptr_t>(d_out);
    const int vec = wave_vec(n_feat, align_or);
    const dim3 grid(ceil_div(n_vert, 4)), block(256);
    hipStream_t s = as_stream(stream);
    if (vec == 4) row_gather_probe_kernel<4><<<grid, block, 0, s>>>(d_feat, d_idxs, d_out, n_vert, n_neigh, n_feat);
    else if (vec == 2) row_gather_probe_kernel<2><<<grid, block, 0, s>>>(d_feat, d_idxs, d_out, n_vert, n_neigh, n_feat);
    else row_gather_probe_kernel<1><<<grid, block, 0, s>>>(d_feat, d_idxs, d_out, n_vert, n_neigh, n_feat);
    return check_launch("row_gather_probe_kernel");
}
