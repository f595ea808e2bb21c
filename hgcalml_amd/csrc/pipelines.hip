// Whole-wrapper entry points: the complete device-side sequence of a reference
// Python wrapper behind one C call, so that a caller pays one launch sequence
// and one workspace instead of a dozen framework ops.
//
//   hgc_binned_select_knn_pipeline  modules/binned_select_knn_op.py:33-104
//     (bounding box and grid, bin assignment, grouping by bin with the inputs
//      moved along, search, un-sort)
#include "hgc_common.hpp"

#include <algorithm>

using namespace hgc;

namespace {

struct KnnPipelineLayout {
    size_t shift, bin_width, n_bins, sorting, bounds, scoords, sflat, sbinass, sdir, grouping_ws, total;
    int total_bins_bound;
};

KnnPipelineLayout knn_layout(int n_vert, int n_coords, int n_bin_dims, int n_rs, int n_bins_scalar, int use_direction) {
    KnnPipelineLayout L{};
    // every per-dimension bin count is at most n_bins_scalar + 1
    long long bound = n_rs - 1;
    for (int i = 0; i < n_bin_dims; ++i) bound = std::min<long long>(bound * (n_bins_scalar + 1), 1ll << 40);
    L.total_bins_bound = (int)std::min<long long>(bound, (1ll << 31) - 2);
    const size_t n = std::max(n_vert, 1);
    size_t off = 0;
    auto take = [&](size_t bytes) {
        size_t at = off;
        off += align_up(bytes);
        return at;
    };
    L.shift = take(8 * sizeof(float));
    L.bin_width = take(sizeof(float));
    L.n_bins = take(8 * sizeof(int));
    L.sorting = take(n * sizeof(int));
    L.bounds = take((((size_t)L.total_bins_bound << bin_grouping_sub_shift(L.total_bins_bound)) + 1) * sizeof(int));
    L.scoords = take(n * n_coords * sizeof(float));
    L.sflat = take(n * sizeof(int));
    L.sbinass = take(n * (n_bin_dims + 1) * sizeof(int));
    L.sdir = take(use_direction ? n * sizeof(int) : 0);
    L.grouping_ws = take(bin_grouping_workspace_bytes(n_vert, L.total_bins_bound));
    L.total = off;
    return L;
}

}  // namespace

extern "C" {

size_t hgc_binned_select_knn_pipeline_workspace_bytes(int n_vert, int n_coords, int n_rs, int n_bins_scalar,
                                                      int max_bin_dims, int use_direction) {
    const int n_bin_dims = std::min(max_bin_dims, n_coords);
    if (n_vert < 0 || n_coords < 1 || n_rs < 2 || n_bins_scalar < 1 || n_bin_dims < 1 || n_bin_dims > 5) return 0;
    return knn_layout(n_vert, n_coords, n_bin_dims, n_rs, n_bins_scalar, use_direction).total;
}

int hgc_binned_select_knn_pipeline(const float *d_coords, const int *d_row_splits, const int *d_direction,
                                   int n_vert, int n_coords, int n_rs, int n_neigh, int n_bins_scalar,
                                   int max_bin_dims, int tf_compat, float max_radius, int *d_indices,
                                   float *d_dist, int *d_out_sorting, void *workspace, size_t workspace_bytes,
                                   hgc_stream_t stream) {
    const int n_bin_dims = std::min(max_bin_dims, n_coords);
    HGC_REQUIRE(n_vert >= 0 && n_rs >= 2, "bad sizes");
    HGC_REQUIRE(n_bins_scalar >= 1, "n_bins must be positive");
    HGC_REQUIRE(n_bin_dims > 1, "BinnedSelectKnnOp expects at least 2 binning dimensions.");
    HGC_REQUIRE(n_bin_dims < 6, "BinnedSelectKnnOp expects maximum 5 binning dimensions.");
    if (n_vert == 0) return HGC_OK;
    HGC_REQUIRE(d_coords && d_row_splits && d_indices && d_dist, "null pointer");
    const int use_direction = d_direction != nullptr;
    const KnnPipelineLayout L = knn_layout(n_vert, n_coords, n_bin_dims, n_rs, n_bins_scalar, use_direction);
    HGC_REQUIRE(L.total_bins_bound < (1ll << 31) - 2, "bin table overflows int32: fewer bins or events per call");
    if (!workspace || !aligned256(workspace) || workspace_bytes < L.total)
        return fail(HGC_ERR_WORKSPACE, "kNN pipeline workspace missing, misaligned or too small");
    char *ws = static_cast<char *>(workspace);
    float *shift = reinterpret_cast<float *>(ws + L.shift);
    float *bin_width = reinterpret_cast<float *>(ws + L.bin_width);
    int *n_bins = reinterpret_cast<int *>(ws + L.n_bins);
    int *sorting = d_out_sorting ? d_out_sorting : reinterpret_cast<int *>(ws + L.sorting);
    int *bounds = reinterpret_cast<int *>(ws + L.bounds);
    float *scoords = reinterpret_cast<float *>(ws + L.scoords);
    int *sflat = reinterpret_cast<int *>(ws + L.sflat);
    int *sbinass = reinterpret_cast<int *>(ws + L.sbinass);
    int *sdir = use_direction ? reinterpret_cast<int *>(ws + L.sdir) : nullptr;

    // The search needs the points grouped by bin, not a particular order inside a
    // bin: its results are in the caller's index space and in canonical order.
    const int rc = bin_grouping(d_coords, d_row_splits, d_direction, n_vert, n_coords, n_bin_dims, n_rs, n_bins_scalar,
                                L.total_bins_bound, shift, bin_width, n_bins, bounds, sorting, scoords, sflat, sbinass,
                                sdir, ws + L.grouping_ws, L.total - L.grouping_ws, as_stream(stream));
    if (rc) return rc;
    return binned_select_knn_strided(scoords, sflat, sdir, sbinass, bounds, bin_grouping_sub_shift(L.total_bins_bound),
                                     n_bins, bin_width, sorting, shift, max_radius, d_indices, d_dist, n_vert, n_neigh,
                                     n_coords, n_bin_dims, L.total_bins_bound + 1, tf_compat, use_direction,
                                     as_stream(stream));
}

}  // extern "C"
