/*
 * hgcalml_amd — C ABI of the MI355X (gfx950) implementation of HGCalML's
 * custom-op hot path: binned kNN, GravNet neighbour accumulation (forward and
 * gradient) and object-condensation condensate assignment.
 *
 * Conventions
 *   - Every pointer named d_* is DEVICE memory owned by the caller. Nothing
 *     user visible is allocated by the library; scratch memory is passed in as
 *     (workspace, workspace_bytes) and sized by the matching *_workspace_bytes
 *     query. Workspace pointers must be 256-byte aligned.
 *   - All tensors are dense row-major, `int` is int32, `float` is fp32.
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream). All
 *     work is enqueued on it; no call synchronises the device.
 *   - Return value: 0 on success, a negative hgc_status otherwise. Argument
 *     errors are detected on the host before anything is launched.
 *   - The library keeps no state between calls except three per-THREAD
 *     settings: the text of the last error (hgc_last_error), the device status
 *     word (hgc_set_status_word) and the choice of the kNN search grid
 *     (hgc_set_knn_grid). A setting made on one thread is not seen by calls made
 *     on another (e.g. by an autograd engine's backward threads): set it on the
 *     thread that makes the call, as the Python wrappers do right before each
 *     call. Calls are re-entrant; calls that share output or workspace buffers
 *     must be ordered by the caller.
 *
 * Each entry point names the reference interface it replaces (paths relative
 * to the HGCalML tree). The reference boundary is the functor
 * `XOpFunctor<Device,int>::operator()(device, raw pointers..., sizes...)`
 * declared in modules/compiled/X_kernel.h; argument order follows it.
 */
#ifndef HGCALML_AMD_H_
#define HGCALML_AMD_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *hgc_stream_t;

enum hgc_status {
    HGC_OK = 0,
    HGC_ERR_INVALID_ARGUMENT = -1, /* shape / range / null-pointer check failed */
    HGC_ERR_WORKSPACE = -2,        /* workspace missing, misaligned or too small */
    HGC_ERR_LAUNCH = -3,           /* the HIP runtime reported an error */
    HGC_ERR_UNSUPPORTED = -4       /* valid for the reference, not built here */
};

/* Library version (major*10000 + minor*100 + patch). */
int hgc_version(void);

/* Human readable text for the last error raised on the calling thread. */
const char *hgc_last_error(void);

/* Data errors. The reference's kernels print a line and carry on with a
 * fallback when they meet bad DATA (a coordinate outside the grid goes to bin 0,
 * modules/compiled/bin_by_coordinates_kernel.cc:75-78; a shell bin beyond the
 * boundary table is skipped, binned_select_knn_kernel.cc:146-149; an index
 * beyond the replacement table is left alone, index_replacer_kernel.cc:35-38),
 * and the Python wrapper refuses non finite coordinates
 * (modules/bin_by_coordinates_op.py:46, tf.debugging.check_numerics). Here the
 * fallbacks are the same and the print becomes a bit in a device status word:
 * after hgc_set_status_word(d_word) every call made by the calling thread ORs
 * the hgc_data_flag bits of what its kernels met into *d_word (one int32 of
 * device memory, owned and zeroed by the caller, read after the stream has been
 * synchronised). NULL (the initial state) switches the reporting off. The
 * setting is per thread; it adds no launch and no synchronisation. */
enum hgc_data_flag {
    HGC_FLAG_COORDINATE_OUT_OF_GRID = 1,  /* a binned coordinate fell outside the grid: bin 0 in that dimension */
    HGC_FLAG_COORDINATE_NOT_FINITE = 2,   /* NaN or Inf among the binned coordinates */
    HGC_FLAG_BIN_BEYOND_TABLE = 4,        /* kNN: a bin of the walk lies beyond d_bin_boundaries: skipped */
    HGC_FLAG_REPLACEMENT_OUT_OF_RANGE = 8, /* index replacer: entry >= n_replacements: left untouched */
    HGC_FLAG_SHELL_TOO_WIDE = 16          /* kNN: a query's walk reached a shell of 2^22 or more rows of bins
                                             inside the grid and within reach, and ended there */
};
int hgc_set_status_word(int *d_word);
/* The calling thread's status word (NULL: none registered on this thread). */
int *hgc_get_status_word(void);

/* ------------------------------------------------------------------ */
/* Spatial binning                                                     */
/* ------------------------------------------------------------------ */

/* Total number of bins = prod(n_bins) * (n_rs - 1); host arithmetic.
 * Replaces BinByCoordinatesNbinsHelperOpFunctor
 * (modules/compiled/bin_by_coordinates_kernel.h, _kernel.cc:17-35), without
 * its device-to-host copy: n_bins is a HOST array here. */
int hgc_bin_by_coordinates_total_bins(const int *h_n_bins, int n_nbins, int n_rs,
                                      int *h_out_total_bins);

/* Per point: per-dimension bin index int(coord / bin_width) (fallback 0 when
 * out of range), event index from the row splits, flat bin index (event
 * major, last coordinate fastest) and optionally the bin populations.
 * Replaces BinByCoordinatesOpFunctor
 * (modules/compiled/bin_by_coordinates_kernel.h, _kernel.cc:46-156).
 *   d_coords [n_vert, n_coords], d_rs [n_rs], d_binswidth [1], d_n_bins [n_coords]
 *   d_assigned_bin [n_vert, n_coords+1], d_flat_assigned_bin [n_vert],
 *   d_n_per_bin [n_total_bins] (zeroed by the call; written only if calc_n_per_bin) */
int hgc_bin_by_coordinates(const float *d_coords, const int *d_rs,
                           const float *d_binswidth, const int *d_n_bins,
                           int *d_assigned_bin, int *d_flat_assigned_bin, int *d_n_per_bin,
                           int n_vert, int n_coords, int n_rs, int n_total_bins,
                           int calc_n_per_bin, hgc_stream_t stream);

/* Same kernel with the wrapper's pre-processing fused in: reads the first
 * n_bin_dims columns of a [n_vert, coord_stride] matrix and subtracts
 * d_shift[c] (may be NULL) before dividing. Replaces the slice and the
 * `coordinates -= min` of modules/bin_by_coordinates_op.py:49-52 and
 * modules/binned_select_knn_op.py:65-69. d_n_out_of_range (may be NULL) counts
 * coordinates that fell outside the grid (the reference prints them). */
int hgc_bin_by_coordinates_strided(const float *d_coords, int coord_stride, const float *d_shift,
                                   const int *d_rs, const float *d_binswidth, const int *d_n_bins,
                                   int *d_assigned_bin, int *d_flat_assigned_bin, int *d_n_per_bin,
                                   int *d_n_out_of_range,
                                   int n_vert, int n_bin_dims, int n_rs, int n_total_bins,
                                   int calc_n_per_bin, hgc_stream_t stream);

/* Bounding box and grid parameters, entirely on the device (no host sync).
 * Replaces the TF glue of modules/bin_by_coordinates_op.py:46-71:
 *   shift = column minimum (0 if pre_normalized), extent = max - shift,
 *   +1 where the column is constant, +1e-3, non finite -> 1;
 *   n_bins_scalar > 0: bin_width = max_d(extent_d / n_bins_scalar), else the
 *   given d_bin_width_in[0]; n_bins_d = int(extent_d / bin_width + 1).
 *   d_shift [n_bin_dims], d_bin_width [1], d_n_bins [n_bin_dims] are outputs. */
size_t hgc_bin_setup_workspace_bytes(int n_vert, int n_bin_dims);
int hgc_bin_setup(const float *d_coords, int coord_stride, int n_vert, int n_bin_dims,
                  int pre_normalized, int n_bins_scalar, const float *d_bin_width_in,
                  float *d_shift, float *d_bin_width, int *d_n_bins,
                  void *workspace, size_t workspace_bytes, hgc_stream_t stream);

/* Stable sort of the points by flat bin index plus the bin boundary table.
 * Replaces tf.argsort + cumsum of modules/binned_select_knn_op.py:72-84 and
 * tf.argsort + segment_ids_to_row_splits of modules/assign_condensate_op.py:276-284.
 *   d_sorting [n_vert]: original index of the i-th point in bin order
 *   d_bin_boundaries [n_total_bins+1]: start of every bin in that order */
size_t hgc_sort_by_bin_workspace_bytes(int n_vert, int n_total_bins);
int hgc_sort_by_bin(const int *d_flat_bin, int n_vert, int n_total_bins,
                    int *d_sorting, int *d_bin_boundaries,
                    void *workspace, size_t workspace_bytes, hgc_stream_t stream);

/* out[i, :] = in[d_rows[i], :] for rows of `width` 4-byte elements (the
 * gather_nd calls of modules/binned_select_knn_op.py:74-79). */
int hgc_gather_rows(const void *d_in, const int *d_rows, void *d_out, int n_rows, int width,
                    hgc_stream_t stream);

/* ------------------------------------------------------------------ */
/* Binned k nearest neighbours                                         */
/* ------------------------------------------------------------------ */

/* Exact kNN inside each event over bin-sorted points.
 * Replaces BinnedSelectKnnOpFunctor
 * (modules/compiled/binned_select_knn_kernel.h, _kernel.cc:47-282).
 *   d_coord [n_vert, n_coords] (bin-sorted), d_bin_idx [n_vert],
 *   d_direction [n_vert] (read only if use_direction),
 *   d_dim_bin_idx [n_vert, n_bin_dim+1], d_bin_boundaries [n_bboundaries],
 *   d_n_bins [n_bin_dim], d_bin_width [1];
 *   d_indices, d_dist [n_vert, n_neigh].
 * Output convention: slot 0 is the point itself; slots 1.. hold the neighbours
 * in ascending (distance^2, index) order; missing neighbours are (-1, 0.0)
 * (or (self, 0.0) if tf_compat) at the tail. The reference leaves the slots in
 * fill/replacement order; the neighbour SET is the same except where the K-th
 * and (K+1)-th distances are exactly equal, where the lower index is kept.
 * Supported: 2 <= n_bin_dim <= 5, n_coords >= 2, n_neigh >= 1 without an upper
 * bound (up to 513 the sorted list lives in registers; beyond that the search
 * runs once per window of 512 ranks and is correspondingly slow),
 * n_vert * n_neigh < 2^31, coordinate matrix below 4 GiB. A shell at distance d is walked as rows of
 * bins along the last binned dimension, those of its (2d+1)^(n_bin_dim-1) rows that are inside
 * the grid and within reach of the search; a query whose walk would reach a shell of 2^22 such
 * rows or more (grids far finer than the points are dense, e.g. 5 binned dimensions with more
 * than 45 bins each) ends there and sets HGC_FLAG_SHELL_TOO_WIDE in the status word;
 * without a registered status word that is silent and the rows of such queries
 * can miss neighbours (hgc_binned_select_knn_pipeline refuses such grids on the
 * host instead, whatever the status word). */
int hgc_binned_select_knn(const float *d_coord, const int *d_bin_idx, const int *d_direction,
                          const int *d_dim_bin_idx, const int *d_bin_boundaries,
                          const int *d_n_bins, const float *d_bin_width,
                          int *d_indices, float *d_dist,
                          int n_vert, int n_neigh, int n_coords, int n_bin_dim,
                          int n_bboundaries, int tf_compat, int use_direction,
                          hgc_stream_t stream);

/* Same search with the wrapper's post-processing fused in
 * (modules/binned_select_knn_op.py:92-95: IndexReplacer, two scatter_nd and the
 * idx<0 -> distance 0 rule) and the radius cut of
 * modules/compiled/select_knn_kernel.cc:158,244-245:
 *   d_sorting (may be NULL) [n_vert]: original index of each sorted point; when
 *     given, neighbour indices are reported in original index space, rows are
 *     written at their original position and ties are broken by original index;
 *   d_shift (may be NULL) [n_bin_dim]: what the binning subtracted from the
 *     binned coordinates (hgc_bin_setup); only sharpens the pruning of far bins;
 *   max_radius > 0: neighbours with distance^2 > max_radius^2 are dropped. */
int hgc_binned_select_knn_fused(const float *d_coord, const int *d_bin_idx, const int *d_direction,
                                const int *d_dim_bin_idx, const int *d_bin_boundaries,
                                const int *d_n_bins, const float *d_bin_width,
                                const int *d_sorting, const float *d_shift, float max_radius,
                                int *d_indices, float *d_dist,
                                int n_vert, int n_neigh, int n_coords, int n_bin_dim,
                                int n_bboundaries, int tf_compat, int use_direction,
                                hgc_stream_t stream);

/* The whole wrapper modules/binned_select_knn_op.py:33-104 in one call:
 * bounding box and grid, bin assignment, grouping by bin with the inputs moved
 * along, search and un-sort. Inputs and outputs are
 * in the caller's order and index space: d_coords [n_vert, n_coords],
 * d_row_splits [n_rs], d_direction [n_vert] or NULL; d_indices, d_dist
 * [n_vert, n_neigh]. d_out_sorting (may be NULL) [n_vert] receives the bin
 * order of the points (original index of the i-th point in bin order; the
 * order inside a bin is unspecified and can differ from run to run, the
 * neighbour results do not depend on it), a useful d_vertex_order for the
 * accumulation. No host synchronisation.
 *
 * The neighbour sets of an exact search do not depend on the grid it walks, so
 * by default the pipeline searches on a grid of its own choice (up to four
 * binned dimensions, about one point per bin at 64 neighbours and finer for
 * fewer; where all of three or four coordinates are binned and 48 neighbours or
 * more are asked for, a second grid of half the bin width nested inside for the
 * queries of crowded bins) and takes n_bins_scalar and
 * max_bin_dims only for the reference's argument checks; hgc_set_knn_grid(1)
 * makes the calling thread's later calls bin exactly as asked
 * (n_bins_scalar bins over min(max_bin_dims, n_coords) dimensions),
 * hgc_set_knn_grid(0) returns to the default. The workspace query covers both,
 * for any number of neighbours. */
int hgc_set_knn_grid(int use_callers_grid);
/* The calling thread's setting (0: the library's own grid, the initial state). */
int hgc_get_knn_grid(void);
size_t hgc_binned_select_knn_pipeline_workspace_bytes(int n_vert, int n_coords, int n_rs,
                                                      int n_bins_scalar, int max_bin_dims,
                                                      int use_direction);
int hgc_binned_select_knn_pipeline(const float *d_coords, const int *d_row_splits,
                                   const int *d_direction, int n_vert, int n_coords, int n_rs,
                                   int n_neigh, int n_bins_scalar, int max_bin_dims, int tf_compat,
                                   float max_radius, int *d_indices, float *d_dist, int *d_out_sorting,
                                   void *workspace, size_t workspace_bytes, hgc_stream_t stream);

/* hgc_binned_select_knn_pipeline for callers that cannot allocate device memory
 * (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc): same arguments without the workspace, same results. It has no
 * counterpart in the reference. The scratch memory is an array of
 * HGC_STATIC_SCRATCH_BYTES inside the library's device image; every GPU the
 * library is used on holds it from the first call to the end of the process.
 * The call allocates and frees nothing. A problem whose
 * hgc_binned_select_knn_pipeline_workspace_bytes(...) exceeds
 * HGC_STATIC_SCRATCH_BYTES is refused with HGC_ERR_WORKSPACE (N = 150,000 points
 * with 4 coordinates, one event and n_bins = 30 need 42.1 MiB). All calls on
 * one GPU share that GPU's array: calls that overlap on one GPU (different
 * streams or threads) race and must be ordered by the caller. The first call on
 * a device looks the array's address up (hipGetSymbolAddress, under a lock):
 * make it outside a stream capture. */
#define HGC_STATIC_SCRATCH_BYTES (64u << 20)
int hgc_binned_select_knn_pipeline_static(const float *d_coords, const int *d_row_splits,
                                          const int *d_direction, int n_vert, int n_coords, int n_rs,
                                          int n_neigh, int n_bins_scalar, int max_bin_dims, int tf_compat,
                                          float max_radius, int *d_indices, float *d_dist,
                                          int *d_out_sorting, hgc_stream_t stream);

/* out[i] = v < 0 ? v : replacements[v]; entries with v >= n_replacements are
 * left untouched. Replaces IndexReplacerOpFunctor
 * (modules/compiled/index_replacer_kernel.h, _kernel.cc:17-42). */
int hgc_index_replacer(const int *d_to_be_replaced, const int *d_replacements, int *d_replaced,
                       int n_to_be_replaced, int n_replacements, hgc_stream_t stream);

/* ------------------------------------------------------------------ */
/* Neighbour accumulation (GravNet aggregation)                        */
/* ------------------------------------------------------------------ */

/* out[v, f] = sum_n w[v,n] * feat[idx[v,n], f] / K (slot order, fp32), and if
 * mean_and_max: out[v, F+f] = max_n (...) with d_out_maxidxs[v,f] = the
 * neighbour index that attained it (later slot wins ties; slot 0 seeds).
 * Negative (and out-of-range) indices are skipped.
 * Replaces AccumulateKnnOpFunctor
 * (modules/compiled/accumulate_knn_kernel.h, _kernel.cc:27-83).
 *   d_distances [n_vert, n_neigh] are the WEIGHTS (the wrapper applies exp(-d)),
 *   d_feat [n_vert, n_feat], d_idxs [n_vert, n_neigh],
 *   d_out_feat [n_vert, n_out_feat] with n_out_feat = n_feat * (mean_and_max ? 2 : 1),
 *   d_out_maxidxs [n_vert, n_feat] (written only if mean_and_max). */
int hgc_accumulate_knn(const float *d_distances, const float *d_feat, const int *d_idxs,
                       float *d_out_feat, int *d_out_maxidxs,
                       int n_vert, int n_neigh, int n_feat, int n_out_feat,
                       int n_moments, int mean_and_max, hgc_stream_t stream);

/* hgc_accumulate_knn that also reports, as one byte per (vertex, feature), the
 * neighbour SLOT that attained the maximum (for a repeated self reference the
 * first slot naming the vertex, which is the one the reference's gradient
 * credits; where no slot attained it -- slot 0 empty and every product
 * negative -- the reference reports index 0 and its gradient credits the slot
 * that names vertex 0, so that slot is reported, 255 if the row has none). Has no counterpart in the reference, which re-derives the
 * slot in the gradient by comparing indices; it exists so that the gradient
 * gathers 1 byte instead of 4 per (neighbour, feature). Needs n_neigh <= 254
 * and, like the reference, indices that are unique in a row apart from
 * repeated self references. d_out_maxslots [n_vert, n_feat] may be NULL.
 *
 * d_vertex_order (may be NULL) [n_vert]: a permutation of the vertices, the
 * order in which they are worked on. Results do not depend on it. When the
 * neighbour table comes from a kNN over shuffled points, vertices that are
 * adjacent in memory share no neighbours and every gathered row misses L2;
 * given the kNN's bin order (d_out_sorting of hgc_binned_select_knn_pipeline)
 * concurrent waves work on spatial neighbours and share their rows (measured
 * 1.9x on the forward, N=150k, K=64, F=64). Honoured for n_feat >= 16. */
int hgc_accumulate_knn_slots(const float *d_distances, const float *d_feat, const int *d_idxs,
                             float *d_out_feat, int *d_out_maxidxs, unsigned char *d_out_maxslots,
                             const int *d_vertex_order,
                             int n_vert, int n_neigh, int n_feat, int n_out_feat,
                             int n_moments, int mean_and_max, hgc_stream_t stream);

/* hgc_accumulate_knn_slots for the AccumulateKnn wrapper: d_distances are
 * distances, the weights are exp(-d) (modules/accknn_op.py:52, there a
 * framework op of its own in front of the kernel) and are also written to
 * d_out_weights [n_vert, n_neigh], which the gradient calls take as their
 * d_distances. For rows of 64 slots or fewer and 16 features or more the
 * exponential is taken inside the accumulation kernel, otherwise by hgc_exp_neg
 * first; the results are the same bits as hgc_exp_neg followed by
 * hgc_accumulate_knn_slots. d_distances and d_out_weights on 16-byte
 * boundaries. No single counterpart in the reference (its wrapper's op and
 * its kernel in one call). */
int hgc_accumulate_knn_exp_slots(const float *d_distances, const float *d_feat, const int *d_idxs,
                                 float *d_out_feat, int *d_out_maxidxs,
                                 unsigned char *d_out_maxslots, float *d_out_weights,
                                 const int *d_vertex_order,
                                 int n_vert, int n_neigh, int n_feat, int n_out_feat,
                                 int n_moments, int mean_and_max, hgc_stream_t stream);

/* Inverse neighbour index: for every vertex m the list of (vertex, slot)
 * pairs that name m, ascending. Built once per neighbour table and reused by
 * every gradient call on it.
 *   d_inv_offsets [n_vert+1], d_inv_slots [n_vert*n_neigh] (flat slot v*K+n) */
size_t hgc_inverse_neighbour_index_workspace_bytes(int n_vert, int n_neigh);
int hgc_inverse_neighbour_index(const int *d_idxs, int n_vert, int n_neigh,
                                int *d_inv_offsets, int *d_inv_slots,
                                void *workspace, size_t workspace_bytes, hgc_stream_t stream);

/* The inverse neighbour index of a table without its first column (GravNet
 * drops the self column of the kNN result before it accumulates,
 * modules/GravNetLayersRagged.py:3095-3283), derived from the index of the whole
 * [n_vert, n_neigh] table in one pass instead of a second sort. No counterpart in
 * the reference. d_out_offsets [n_vert+1], d_out_slots [n_vert*(n_neigh-1)]. */
size_t hgc_inverse_index_without_first_column_workspace_bytes(int n_vert);
int hgc_inverse_index_without_first_column(const int *d_inv_offsets, const int *d_inv_slots,
                                           int n_vert, int n_neigh, int *d_out_offsets,
                                           int *d_out_slots, void *workspace, size_t workspace_bytes,
                                           hgc_stream_t stream);

/* Gradients of hgc_accumulate_knn w.r.t. the weights and the features.
 * Replaces AccumulateKnnGradOpFunctor
 * (modules/compiled/accumulate_knn_grad_kernel.h, _kernel.cc:24-227); the
 * contended atomicAdd of the reference's device path becomes an ordered
 * gather through the inverse neighbour index, which reproduces the CPU
 * kernel's summation order for the feature gradient.
 *   d_grad_from_out_features [n_vert, n_grad_from_out_feat]
 *     (n_grad_from_out_feat == 2*n_feat selects mean_and_max),
 *   d_distances (weights), d_feat, d_max_feat_indices [n_vert, n_feat], d_neigh_indices,
 *   d_inv_offsets / d_inv_slots from hgc_inverse_neighbour_index,
 *   d_out_grad_distances [n_vert, n_neigh], d_out_grad_features [n_vert, n_feat]. */
int hgc_accumulate_knn_grad(const float *d_grad_from_out_features, const float *d_distances,
                            const float *d_feat, const int *d_max_feat_indices,
                            const int *d_neigh_indices,
                            const int *d_inv_offsets, const int *d_inv_slots,
                            float *d_out_grad_distances, float *d_out_grad_features,
                            int n_vert, int n_neigh, int n_feat, int n_grad_from_out_feat,
                            int n_moments, int mean_and_max, hgc_stream_t stream);

/* hgc_accumulate_knn_grad with the arg-max slot table of
 * hgc_accumulate_knn_slots (d_max_slots [n_vert, n_feat], may be NULL: then
 * identical to hgc_accumulate_knn_grad). Same results, less gather traffic.
 * d_vertex_order (may be NULL): as for hgc_accumulate_knn_slots. */
int hgc_accumulate_knn_grad_slots(const float *d_grad_from_out_features, const float *d_distances,
                                  const float *d_feat, const int *d_max_feat_indices,
                                  const unsigned char *d_max_slots, const int *d_neigh_indices,
                                  const int *d_inv_offsets, const int *d_inv_slots,
                                  const int *d_vertex_order,
                                  float *d_out_grad_distances, float *d_out_grad_features,
                                  int n_vert, int n_neigh, int n_feat, int n_grad_from_out_feat,
                                  int n_moments, int mean_and_max, hgc_stream_t stream);

/* hgc_accumulate_knn_grad_slots with scratch memory for one 32-byte record and
 * one 4-byte result per (vertex, slot): a streaming pass over the vertices first
 * collects, for every slot, the weight, which features have their maximum there
 * (from d_max_slots) and their upstream gradients; the gather over the inverse
 * index then reads one record per entry instead of a weight, a line of slot
 * bytes and scattered pieces of the max half of the gradient row, and writes the
 * weight gradients in the order of the inverse list; a last streaming pass moves
 * them to their slots. Same results as
 * hgc_accumulate_knn_grad_slots (feature gradient bit for bit; the weight
 * gradient's max part is added after the mean part instead of inside it). Has
 * no counterpart in the reference. The workspace query returns 0 for shapes the
 * record pass does not cover (n_feat outside 16..128, n_neigh > 254, gradient
 * matrix of 4 GiB or more, !mean_and_max); the call then behaves exactly like
 * hgc_accumulate_knn_grad_slots and accepts a NULL workspace, as it does when
 * d_max_slots is NULL. hgc_accumulate_knn_grad_records_pays says where the
 * record pass has measured faster (n_neigh >= 48, n_neigh < n_feat <= 2 n_neigh
 * and n_vert * n_feat of 12 Mi elements or more: cfg4 5.8 -> 4.7 ms); elsewhere
 * hgc_accumulate_knn_grad_slots is the better call. */
size_t hgc_accumulate_knn_grad_records_workspace_bytes(int n_vert, int n_neigh, int n_feat,
                                                       int mean_and_max);
int hgc_accumulate_knn_grad_records_pays(int n_vert, int n_neigh, int n_feat, int mean_and_max);
int hgc_accumulate_knn_grad_records(const float *d_grad_from_out_features, const float *d_distances,
                                    const float *d_feat, const int *d_max_feat_indices,
                                    const unsigned char *d_max_slots, const int *d_neigh_indices,
                                    const int *d_inv_offsets, const int *d_inv_slots,
                                    const int *d_vertex_order,
                                    float *d_out_grad_distances, float *d_out_grad_features,
                                    int n_vert, int n_neigh, int n_feat, int n_grad_from_out_feat,
                                    int n_moments, int mean_and_max,
                                    void *workspace, size_t workspace_bytes, hgc_stream_t stream);

/* ------------------------------------------------------------------ */
/* Ops over the same neighbour table, either side of the accumulation  */
/* ------------------------------------------------------------------ */

/* Gradient of the kNN squared distances w.r.t. the coordinates: the
 * registered gradient of BinnedSelectKnn (modules/binned_select_knn_op.py:107-118).
 * Replaces SelectKnnGradOpFunctor (modules/compiled/select_knn_grad_kernel.h;
 * its CPU body is empty, the arithmetic is that of _kernel.cu.cc:81-164):
 *   grad_coord[i,c] = - sum_n 2 g[i,n] (x[idx[i,n],c] - x[i,c])
 *                     + sum over (v,n) with idx[v,n] == i of 2 g[v,n] (x[i,c] - x[v,c]).
 * The second sum runs over the inverse neighbour index in ascending (v,n)
 * order instead of the reference's atomicAdd. Indices < 0 or >= n_vert are
 * skipped. d_dist is accepted for signature parity and not read.
 *   d_grad_dist, d_dist [n_vert, n_neigh], d_indices [n_vert, n_neigh],
 *   d_coord, d_grad_coord [n_vert, n_coords]. */
int hgc_select_knn_grad(const float *d_grad_dist, const int *d_indices, const float *d_dist,
                        const float *d_coord, const int *d_inv_offsets, const int *d_inv_slots,
                        float *d_grad_coord, int n_vert, int n_neigh, int n_coords,
                        hgc_stream_t stream);
/* The same with a processing order of the vertices (d_vertex_order [n_vert], a
 * permutation, may be NULL; d_out_sorting of hgc_binned_select_knn_pipeline is
 * a good one): same results, about 1.4x faster on neighbour tables of shuffled
 * points. No counterpart in the reference. */
int hgc_select_knn_grad_ordered(const float *d_grad_dist, const int *d_indices, const float *d_dist,
                                const float *d_coord, const int *d_inv_offsets, const int *d_inv_slots,
                                const int *d_vertex_order, float *d_grad_coord,
                                int n_vert, int n_neigh, int n_coords, hgc_stream_t stream);

/* distances[i,n] = |x_i - x_idx[i,n]|^2 (serial fp32 sum over the coordinates),
 * 0 where idx[i,n] < 0 or idx[i,n] == i. Replaces LocalDistanceOpFunctor
 * (modules/compiled/local_distance_kernel.h, _kernel.cc:18-70), same argument
 * order. Its registered gradient is hgc_select_knn_grad
 * (modules/local_distance_op.py:24-40).
 *   d_neigh_idxs, d_distances [n_out_vert, n_neigh], d_coords [n_in_vert, n_coords]. */
int hgc_local_distance(const int *d_neigh_idxs, const float *d_coords, float *d_distances,
                       int n_coords, int n_in_vert, int n_out_vert, int n_neigh,
                       hgc_stream_t stream);
/* The same with a processing order of the n_out_vert vertices (may be NULL), as
 * for hgc_select_knn_grad_ordered: same results, 0.16 -> 0.12 ms at N=150k,
 * K=64, C=4 on shuffled points. No counterpart in the reference. */
int hgc_local_distance_ordered(const int *d_neigh_idxs, const float *d_coords,
                               const int *d_vertex_order, float *d_distances,
                               int n_coords, int n_in_vert, int n_out_vert, int n_neigh,
                               hgc_stream_t stream);

/* Feature-weighted mean and covariance of the neighbours' coordinates, as the
 * wrapper modules/neighbour_covariance_op.py:8-62 composes them from three
 * mean-only accumulations over matrices of F, F*C and F*C*C columns: with
 * j = idx[v,n],
 *   S[v,f]       = sum_n w[v,n] a[j,f]
 *   mean[v,f,c]  = sum_n w[v,n] a[j,f] x[j,c] / (S[v,f] + 1e-3)
 *   cov[v,f,c,d] = sum_n w[v,n] a[j,f] (x[j,c] - mean[j,f,c]) (x[j,d] - mean[j,f,d]) / (S[v,f] + 1e-3)
 * (every neighbour centred on its own mean; sums in slot order, divided and
 * multiplied by K as the accumulation's mean is; a zero denominator gives 0).
 * Two passes over the table, nothing of F*C*C columns is materialised as
 * input. d_weights are exp(-distsq) and d_feats the activated features
 * (sigmoid + 1e-3), both formed by the caller. The compiled
 * NeighbourCovarianceOpFunctor of the reference
 * (modules/compiled/neighbour_covariance_kernel.h: unweighted, lower triangle,
 * centred on the accumulating vertex) is not what that wrapper calls and is not
 * built. n_coords <= 6.
 *   d_coords [n_vert, n_coords], d_weights, d_n_idxs [n_vert, n_neigh],
 *   d_feats [n_vert, n_feat]; outputs d_covariance [n_vert, n_feat, n_coords^2],
 *   d_means [n_vert, n_feat, n_coords], d_sum_weights [n_vert, n_feat] (S).
 *   d_vertex_order (may be NULL): as for hgc_accumulate_knn_slots. */
int hgc_neighbour_covariance(const float *d_coords, const float *d_weights, const float *d_feats,
                             const int *d_n_idxs, const int *d_vertex_order, float *d_covariance,
                             float *d_means, float *d_sum_weights, int n_vert, int n_coords, int n_feat,
                             int n_neigh, hgc_stream_t stream);

/* out[m,f] = sum over (v,n) with idx[v,n] == m of feat[v,f] * w[v,n]
 * (idx < 0: no neighbour). Replaces PushKnnOpFunctor
 * (modules/compiled/push_knn_kernel.h, _kernel.cc:40-62); the additions of
 * one target happen in ascending (v,n) order, which is the CPU kernel's, so
 * the result is bit-identical to it. */
int hgc_push_knn(const float *d_weights, const float *d_feat, const int *d_idxs,
                 const int *d_inv_offsets, const int *d_inv_slots, float *d_out_feat,
                 int n_vert, int n_neigh, int n_feat, hgc_stream_t stream);
/* The same with a processing order of the target vertices (may be NULL), as
 * for hgc_accumulate_knn_slots: same bits, 0.49 -> 0.24 ms at N=150k, K=64,
 * F=64 on shuffled points. No counterpart in the reference. */
int hgc_push_knn_ordered(const float *d_weights, const float *d_feat, const int *d_idxs,
                         const int *d_inv_offsets, const int *d_inv_slots,
                         const int *d_vertex_order, float *d_out_feat,
                         int n_vert, int n_neigh, int n_feat, hgc_stream_t stream);

/* Gradients of hgc_push_knn. Replaces PushKnnGradOpFunctor
 * (modules/compiled/push_knn_grad_kernel.h, _kernel.cc:23-71):
 *   feat_grad[v,f] = sum_n grad[idx[v,n],f] * w[v,n]   (slot order, bit-identical),
 *   w_grad[v,n]    = sum_f grad[idx[v,n],f] * feat[v,f] (tree reduction over f),
 *   0 where idx[v,n] < 0. */
int hgc_push_knn_grad(const float *d_grad, const float *d_weights, const float *d_feat,
                      const int *d_idxs, float *d_feat_grad, float *d_w_grad,
                      int n_vert, int n_neigh, int n_feat, hgc_stream_t stream);

/* The elementwise glue of the AccumulateKnn wrapper (modules/accknn_op.py:52,
 * `tf.exp(-distsq)`) and of its gradient, one pass each: d_weights[i] =
 * exp(-d_distances[i]); d_distance_grad[i] = -(d_weight_grad[i] * d_weights[i]).
 * Arrays of n_values floats on 16-byte boundaries. */
int hgc_exp_neg(const float *d_distances, float *d_weights, long long n_values, hgc_stream_t stream);
int hgc_exp_neg_grad(const float *d_weight_grad, const float *d_weights, float *d_distance_grad,
                     long long n_values, hgc_stream_t stream);

/* Ascending sort of n 64-bit keys that differ pairwise (none of them all ones):
 * d_values[i] = the low value_bits bits of the i-th smallest key. The keys are
 * not checked: equal keys come out in an unspecified order relative to each
 * other (every value still appears exactly once, nothing faults), and a key of
 * all ones is taken for padding and may lose its place to real keys. The order of
 * the condensate selection (event, beta descending, position) is this sort; the
 * reference has no counterpart (binned_assign_to_condensates_kernel.cc:187-236
 * picks by a linear arg-max per condensation point). d_keys is overwritten.
 * n <= 2^20. stage: 0, or the number of keys a workgroup sorts in LDS at once
 * (a power of two up to 8192; smaller values only make it slower). */
size_t hgc_sort_distinct_keys_workspace_bytes(long long n);
int hgc_sort_distinct_keys(unsigned long long *d_keys, long long n, int value_bits, int *d_values,
                           void *workspace, size_t workspace_bytes, int stage, hgc_stream_t stream);

/* ------------------------------------------------------------------ */
/* Condensate assignment                                               */
/* ------------------------------------------------------------------ */

/* Greedy highest-beta-first condensate selection and hit assignment per event.
 * Replaces BinnedCondensatesFinderOpFunctor
 * (modules/compiled/binned_assign_to_condensates_kernel.h, _kernel.cc:23-241);
 * argument order follows the functor, sizes the reference derives from tensor
 * shapes are explicit. Arrays without suffix hold all hits in bin-sorted order,
 * *_h the high-beta subset in the same order.
 *   outputs: d_high_assigned_status_h [n_vert_h] (1 for condensate points),
 *   d_assignment [n_vert] (shower index inside the event, -1 noise),
 *   d_association [n_vert] (original index of the condensate point, -1 noise),
 *   d_n_condensates [num_rows+1] (cumulative), d_alpha_indices [n_vert_h]
 *   (original indices of the condensate points per event, -1 padded).
 *   d_condensates_assigned_h [n_vert_h] and d_assignment_min_distance [n_vert]
 *   (the latter only if !assign_by_max_beta) are caller scratch like in the
 *   reference. d_error (may be NULL) is set to 0: the loop that could stall in
 *   the reference (it throws std::runtime_error there) does not exist here.
 *   The two views of the hits must agree as the reference wrapper builds them:
 *   d_indices_to_filtered[i] = q exactly for the hit i that entry q of the *_h
 *   arrays was taken from (same coordinates and mask), -1 for the others. */
size_t hgc_binned_assign_to_condensates_workspace_bytes(int n_vert, int n_vert_h, int num_rows);
int hgc_binned_assign_to_condensates(int dimensions, int dimensions_binning,
                                     int *d_condensates_assigned_h,
                                     const float *d_ccoords_h, const float *d_dist_h,
                                     const float *d_beta_h, const int *d_no_condensation_mask_h,
                                     int *d_high_assigned_status_h,
                                     const int *d_original_indices_h, const int *d_row_splits_h,
                                     const float *d_ccoords, const float *d_dist,
                                     const int *d_no_condensation_mask,
                                     const int *d_indices_to_filtered,
                                     float *d_assignment_min_distance,
                                     int *d_assignment, int *d_association,
                                     int *d_n_condensates, int *d_alpha_indices,
                                     const int *d_bin_splits, const int *d_n_bins,
                                     const float *d_bin_widths, const int *d_row_splits,
                                     int num_rows, int assign_by_max_beta,
                                     int n_vert, int n_vert_h, int *d_error,
                                     void *workspace, size_t workspace_bytes,
                                     hgc_stream_t stream);

/* The whole wrapper modules/assign_condensate_op.py:210-373
 * (BuildAndAssignCondensatesBinned without keep_noise) in one call: coordinates
 * shifted to their column minima, grid of n_bins_scalar bins along the widest of
 * the first min(nbin_dims, n_coords) coordinates, bin assignment, stable sort
 * into bin order, local radii divided by distance_threshold, high-beta subset
 * (beta > beta_threshold or masked), assignment, results back in the caller's
 * order. Inputs in the caller's order: d_ccoords [n_vert, n_coords], d_betas,
 * d_dist [n_vert], d_no_condensation_mask [n_vert] or NULL, d_row_splits
 * [num_rows + 1]. Outputs: d_assignment, d_association [n_vert], d_is_cond
 * [n_vert] (one byte each), d_n_condensates [num_rows + 1] (cumulative) and
 * d_alpha_idx, which must have room for n_vert entries; its first
 * d_n_condensates[num_rows] ones are the condensation points of all events in
 * selection order. No host synchronisation (the caller reads
 * d_n_condensates[num_rows] to learn how many entries of d_alpha_idx count). */
size_t hgc_build_and_assign_condensates_workspace_bytes(int n_vert, int n_coords, int num_rows,
                                                        int n_bins_scalar, int nbin_dims);
int hgc_build_and_assign_condensates(const float *d_ccoords, const float *d_betas, const float *d_dist,
                                     const int *d_no_condensation_mask, const int *d_row_splits,
                                     int n_vert, int n_coords, int num_rows, float beta_threshold,
                                     float distance_threshold, int assign_by_max_beta, int nbin_dims,
                                     int n_bins_scalar, int *d_assignment, int *d_association,
                                     int *d_alpha_idx, unsigned char *d_is_cond, int *d_n_condensates,
                                     void *workspace, size_t workspace_bytes, hgc_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* HGCALML_AMD_H_ */
