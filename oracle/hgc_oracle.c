/*
 * CPU oracle for the HGCalML custom-op hot path.
 *
 * THIS FILE IS TEST INFRASTRUCTURE. It restates, in plain single-threaded C,
 * the arithmetic and control flow of the reference CPU kernels so that the HIP
 * kernels can be checked against it. It is never part of the shipped compute
 * path: only tests/, __graft_entry__.smoke() and the cpu_baseline leg of
 * bench.py may load it.
 *
 * Reference (paths relative to the HGCalML tree) each function follows:
 *   hgo_bin_by_coordinates        modules/compiled/bin_by_coordinates_kernel.cc:46-114
 *   hgo_shell_next / shell walker modules/compiled/binstepper.h:11-97
 *   hgo_binned_select_knn         modules/compiled/binned_select_knn_kernel.cc:19-196
 *   hgo_index_replacer            modules/compiled/index_replacer_kernel.cc:29-40
 *   hgo_accumulate_knn            modules/compiled/accumulate_knn_kernel.cc:48-81
 *   hgo_accumulate_knn_grad       modules/compiled/accumulate_knn_grad_kernel.cc:24-165
 *   hgo_select_knn_grad           modules/compiled/select_knn_grad_kernel.cu.cc:81-164
 *   hgo_push_knn                  modules/compiled/push_knn_kernel.cc:40-62
 *   hgo_push_knn_grad             modules/compiled/push_knn_grad_kernel.cc:23-71
 *   hgo_local_distance            modules/compiled/local_distance_kernel.cc:18-70
 *   hgo_box_* / hgo_assign_to_condensates
 *                                 modules/compiled/binstepper.h:100-165,
 *                                 modules/compiled/binned_assign_to_condensates_kernel.cc:23-241
 *
 * Parity status of each function (what pins it, see tests/test_oracle_pins.py):
 *   hgo_bin_by_coordinates   pinned: closed-form integer arithmetic, brute force.
 *   shell walker             pinned: shells partition the grid, no duplicates.
 *   hgo_binned_select_knn    neighbour SETS and distances pinned by an O(N^2)
 *                            brute force with the same serial fp32 sum;
 *                            the raw slot order and which member of an exactly
 *                            tied K-th boundary group survives are
 *                            "parity unpinned" (only the compiled reference,
 *                            which cannot be built here, could pin them).
 *   hgo_index_replacer       pinned: closed form.
 *   hgo_accumulate_knn       pinned: gather/multiply/mean/max composition.
 *   hgo_accumulate_knn_grad  pinned: autograd of that composition.
 *   hgo_select_knn_grad      pinned: float64 autograd of sum((x_i - x_k)^2).
 *   hgo_push_knn             pinned: ordered unbuffered scatter-add (bitwise).
 *   hgo_push_knn_grad        pinned: float64 autograd of that scatter-add.
 *   hgo_local_distance       pinned: the brute-force serial fp32 distance.
 *   hgo_assign_to_condensates pinned by a bin-free sequential greedy written from
 *                            the reference text, without and with a
 *                            no_condensation_mask (incl. masks on the first two
 *                            high-beta entries, which switch the pick order).
 *                            That both restate the reference's mask indexing
 *                            the same way is all that pins it: "parity
 *                            unpinned" against the compiled reference there.
 *
 * Build: gcc -O2 -ffp-contract=off -shared -fPIC (see oracle/Makefile).
 * All fp32 arithmetic is written as separate multiplies and adds, in the
 * source order of the reference, and must not be contracted into FMAs.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define HGO_MAX_BIN_DIMS 8

/* ------------------------------------------------------------------ */
/* bin_by_coordinates                                                  */
/* ------------------------------------------------------------------ */

/* Returns the number of points whose coordinate fell outside the grid (the
 * reference prints a message for each and falls back to bin 0 in that
 * dimension). binass/flat rows of points whose flat index overflows the
 * total are left untouched, as in the reference. */
int hgo_bin_by_coordinates(const float *coords, const int *row_splits,
                           const float *bin_width, const int *n_bins,
                           int *binass, int *flat, int *n_per_bin,
                           int n_vert, int n_coords, int n_rs,
                           int n_total_bins, int calc_n_per_bin)
{
    int n_bad = 0;
    for (int b = 0; b < n_total_bins; ++b)
        n_per_bin[b] = 0;

    const float bw = bin_width[0];
    for (int p = 0; p < n_vert; ++p) {
        int stride = 1;
        int cell = 0;
        /* last coordinate is the fastest running one */
        for (int c = n_coords - 1; c >= 0; --c) {
            int k = (int)(coords[p * n_coords + c] / bw);
            if (k < 0 || k >= n_bins[c]) {
                k = 0;
                ++n_bad;
            }
            binass[p * (n_coords + 1) + c + 1] = k;
            cell += k * stride;
            stride *= n_bins[c];
        }
        /* event index: number of leading row splits (from the 2nd on) that
         * are not beyond this point */
        int ev = 0;
        for (int r = 1; r < n_rs; ++r) {
            if (row_splits[r] > p)
                break;
            ++ev;
        }
        cell += ev * stride;
        if (cell >= n_total_bins)
            continue;
        binass[p * (n_coords + 1)] = ev;
        flat[p] = cell;
        if (calc_n_per_bin)
            n_per_bin[cell] += 1;
    }
    return n_bad;
}

/* ------------------------------------------------------------------ */
/* shell walker: surface bins of the cube of half-width d              */
/* ------------------------------------------------------------------ */

typedef struct {
    int ndim;
    int d;
    int64_t step;
    int64_t cube_cap;
    int total;
    int nb[HGO_MAX_BIN_DIMS];
    int centre[HGO_MAX_BIN_DIMS];
} hgo_shell;

static void hgo_shell_init(hgo_shell *s, int ndim, const int *n_bins, const int *centre)
{
    s->ndim = ndim;
    s->total = 1;
    for (int i = 0; i < ndim; ++i) {
        s->nb[i] = n_bins[i];
        s->centre[i] = centre[i];
        s->total *= n_bins[i];
    }
}

static void hgo_shell_set_d(hgo_shell *s, int d)
{
    s->d = d;
    s->cube_cap = 1;
    for (int i = 0; i < s->ndim; ++i)
        s->cube_cap *= 2 * d + 1;
    s->step = 0;
}

/* next valid surface bin (flat index inside one event's grid) or -1 */
static int hgo_shell_next(hgo_shell *s)
{
    const int w = 2 * s->d + 1;
    while (s->step < s->cube_cap) {
        int64_t rem = s->step++;
        int64_t mul = s->cube_cap;
        int off[HGO_MAX_BIN_DIMS];
        int surface = 0;
        /* first dimension is the most significant digit */
        for (int i = 0; i < s->ndim; ++i) {
            mul /= w;
            int digit = (int)(rem / mul);
            rem -= digit * mul;
            off[i] = digit - s->d;
            if (abs(off[i]) == s->d)
                surface = 1;
        }
        if (!surface)
            continue;
        int flat = 0, stride = 1, ok = 1;
        for (int i = s->ndim - 1; i >= 0; --i) {
            int k = s->centre[i] + off[i];
            if (k < 0 || k >= s->nb[i]) {
                ok = 0;
                break;
            }
            flat += k * stride;
            stride *= s->nb[i];
        }
        if (!ok || flat < 0 || flat >= s->total)
            continue;
        return flat;
    }
    return -1;
}

/* test hook: enumerate one shell into out (capacity cap); returns count */
int hgo_shell_enumerate(int ndim, const int *n_bins, const int *centre, int d,
                        int *out, int cap)
{
    hgo_shell s;
    hgo_shell_init(&s, ndim, n_bins, centre);
    hgo_shell_set_d(&s, d);
    int n = 0;
    for (;;) {
        int b = hgo_shell_next(&s);
        if (b < 0)
            break;
        if (n < cap)
            out[n] = b;
        ++n;
    }
    return n;
}

/* ------------------------------------------------------------------ */
/* binned_select_knn                                                   */
/* ------------------------------------------------------------------ */

static float hgo_distsq(const float *x, int i, int j, int n_coords)
{
    if (i == j)
        return 0.f;
    float acc = 0.f;
    for (int c = 0; c < n_coords; ++c) {
        float diff = x[i * n_coords + c] - x[j * n_coords + c];
        float sq = diff * diff;
        acc = acc + sq;
    }
    return acc;
}

/* slot of the largest distance among slots 1..K-1 (first one among equals) */
static int hgo_worst_slot(const float *row, int K, float *worst)
{
    *worst = 0.f;
    int slot = 0;
    for (int n = 1; n < K; ++n) {
        if (row[n] > *worst) {
            *worst = row[n];
            slot = n;
        }
    }
    return slot;
}

/* Inputs are in bin-sorted order. Returns a count of anomalies the reference
 * only prints (bin index beyond the boundary table). */
int hgo_binned_select_knn(const float *coords, const int *bin_idx,
                          const int *direction, const int *dim_bin_idx,
                          const int *bin_boundaries, const int *n_bins,
                          const float *bin_width,
                          int *indices, float *distances,
                          int n_vert, int K, int n_coords, int n_bin_dim,
                          int n_bboundaries, int tf_compat, int use_direction)
{
    int anomalies = 0;
    for (int i = 0; i < n_vert; ++i) {
        for (int n = 0; n < K; ++n) {
            indices[i * K + n] = (n == 0 || tf_compat) ? i : -1;
            distances[i * K + n] = 0.f;
        }
    }

    int cells_per_event = 1;
    for (int b = 0; b < n_bin_dim; ++b)
        cells_per_event *= n_bins[b];
    const float bw = bin_width[0];

    for (int i = 0; i < n_vert; ++i) {
        /* direction: 0 may only be a neighbour, 1 may only have neighbours,
         * 2 neither */
        if (use_direction && (direction[i] == 0 || direction[i] == 2))
            continue;

        int filled = 1;
        int worst_slot = 0;
        float worst = 0.f;
        int *irow = indices + (size_t)i * K;
        float *drow = distances + (size_t)i * K;

        const int event_base = cells_per_event * (bin_idx[i] / cells_per_event);

        hgo_shell walker;
        hgo_shell_init(&walker, n_bin_dim, n_bins,
                       dim_bin_idx + (size_t)i * (n_bin_dim + 1) + 1);

        for (int d = 0;; ++d) {
            hgo_shell_set_d(&walker, d);
            int any_bin = 0;
            for (;;) {
                int cell = hgo_shell_next(&walker);
                if (cell < 0)
                    break;
                cell += event_base;
                if (cell >= n_bboundaries - 1) {
                    ++anomalies;
                    continue;
                }
                const int lo = bin_boundaries[cell];
                const int hi = bin_boundaries[cell + 1];
                for (int j = lo; j < hi; ++j) {
                    if (j == i)
                        continue;
                    if (use_direction && (direction[j] == 1 || direction[j] == 2))
                        continue;
                    float dsq = hgo_distsq(coords, i, j, n_coords);
                    if (filled < K) {
                        irow[filled] = j;
                        drow[filled] = dsq;
                        if (dsq > worst) {
                            worst = dsq;
                            worst_slot = filled;
                        }
                        ++filled;
                        continue;
                    }
                    if (dsq < worst) {
                        irow[worst_slot] = j;
                        drow[worst_slot] = dsq;
                        worst_slot = hgo_worst_slot(drow, K, &worst);
                    }
                }
                any_bin = 1;
            }
            if (!any_bin)
                break;
            /* conservative stop: everything unseen is at least d bin widths
             * away in one binned coordinate; fp32, evaluated left to right */
            float reach = bw * (float)d;
            reach = reach * bw;
            reach = reach * (float)d;
            if (filled == K && reach > worst)
                break;
        }
    }
    return anomalies;
}

/* ------------------------------------------------------------------ */
/* index_replacer                                                      */
/* ------------------------------------------------------------------ */

/* out[i] is left untouched for indices beyond the table (the reference
 * prints and skips); returns how many there were */
int hgo_index_replacer(const int *to_be_replaced, const int *replacements,
                       int *out, int n, int n_replacements)
{
    int bad = 0;
    for (int i = 0; i < n; ++i) {
        int v = to_be_replaced[i];
        if (v < 0) {
            out[i] = v;
        } else if (v >= n_replacements) {
            ++bad;
        } else {
            out[i] = replacements[v];
        }
    }
    return bad;
}

/* ------------------------------------------------------------------ */
/* accumulate_knn forward                                              */
/* ------------------------------------------------------------------ */

void hgo_accumulate_knn(const float *weights, const float *features,
                        const int *indices, float *out, int *out_maxidx,
                        int n_vert, int K, int F, int mean_and_max)
{
    const int out_cols = mean_and_max ? 2 * F : F;
    for (int v = 0; v < n_vert; ++v) {
        for (int f = 0; f < F; ++f) {
            float sum = 0.f;
            float best = 0.f;
            int best_idx = 0;
            for (int n = 0; n < K; ++n) {
                int j = indices[(size_t)v * K + n];
                if (j < 0)
                    continue;
                float wf = features[(size_t)j * F + f] * weights[(size_t)v * K + n];
                sum = sum + wf;
                /* ">=": a later slot wins ties; slot 0 always seeds the max */
                if (mean_and_max && (wf >= best || n == 0)) {
                    best = wf;
                    best_idx = j;
                }
            }
            out[(size_t)v * out_cols + f] = sum / (float)K;
            if (mean_and_max) {
                out[(size_t)v * out_cols + F + f] = best;
                out_maxidx[(size_t)v * F + f] = best_idx;
            }
        }
    }
}

/* ------------------------------------------------------------------ */
/* accumulate_knn gradient                                             */
/* ------------------------------------------------------------------ */

void hgo_accumulate_knn_grad(const float *grad_out, const float *weights,
                             const float *features, const int *maxidx,
                             const int *indices,
                             float *grad_weights, float *grad_features,
                             int n_vert, int K, int F, int grad_cols,
                             int mean_and_max)
{
    memset(grad_features, 0, sizeof(float) * (size_t)n_vert * F);

    /* feature gradient: every (vertex, slot) pushes into its neighbour's row;
     * per target the additions happen in ascending (vertex, slot) order */
    for (int v = 0; v < n_vert; ++v) {
        for (int f = 0; f < F; ++f) {
            const float g_mean = grad_out[(size_t)v * grad_cols + f];
            float g_max = 0.f;
            int arg = -1;
            if (mean_and_max) {
                g_max = grad_out[(size_t)v * grad_cols + F + f];
                arg = maxidx[(size_t)v * F + f];
            }
            int self_pending = 1;
            for (int n = 0; n < K; ++n) {
                int m = indices[(size_t)v * K + n];
                if (m < 0)
                    continue;
                const float w = weights[(size_t)v * K + n];
                float part_mean = g_mean / (float)K;
                part_mean = part_mean * w;
                float part_max = 0.f;
                if (m == arg) {
                    if (m == v) {
                        if (self_pending) {
                            part_max = g_max * w;
                            self_pending = 0;
                        }
                    } else {
                        part_max = g_max * w;
                    }
                }
                float add = part_mean + part_max;
                grad_features[(size_t)m * F + f] = grad_features[(size_t)m * F + f] + add;
            }
        }
    }

    /* weight gradient */
    for (int m = 0; m < n_vert; ++m) {
        for (int l = 0; l < K; ++l) {
            int j = indices[(size_t)m * K + l];
            if (j < 0) {
                grad_weights[(size_t)m * K + l] = 0.f;
                continue;
            }
            float acc_mean = 0.f;
            float acc_max = 0.f;
            for (int f = 0; f < F; ++f) {
                float g = grad_out[(size_t)m * grad_cols + f];
                float x = features[(size_t)j * F + f];
                float t = g * x;
                t = t * 1.f;
                acc_mean = acc_mean + t;
                if (mean_and_max && j == maxidx[(size_t)m * F + f]) {
                    /* the reference's "count self once" flag is reset for
                     * every feature, so it never suppresses a term */
                    float gm = grad_out[(size_t)m * grad_cols + F + f];
                    float u = gm * x;
                    u = u * 1.f;
                    acc_max = acc_max + u;
                }
            }
            /* the 1/K factor is applied in double precision and rounded back */
            double scaled = (double)acc_mean * (1. / (double)(float)K);
            acc_mean = (float)scaled;
            grad_weights[(size_t)m * K + l] = acc_mean + acc_max;
        }
    }
}

/* ------------------------------------------------------------------ */
/* condensate assignment                                               */
/* ------------------------------------------------------------------ */

typedef struct {
    int ndim;
    int lo[HGO_MAX_BIN_DIMS];
    int width[HGO_MAX_BIN_DIMS];
    const int *n_bins;
    int n_combos;
    int cursor;
    int total;
} hgo_box;

static void hgo_box_set(hgo_box *b, int ndim, const float *lo, const float *hi,
                        float bin_width, const int *n_bins)
{
    b->ndim = ndim;
    b->n_bins = n_bins;
    b->n_combos = 1;
    b->cursor = 0;
    b->total = 1;
    for (int d = 0; d < ndim; ++d) {
        int first = (int)floorf(lo[d] / bin_width);
        int last = (int)ceilf(hi[d] / bin_width);
        b->lo[d] = first;
        b->width[d] = last - first + 1;
        b->n_combos *= b->width[d];
        b->total *= n_bins[d];
    }
}

/* next flat bin index of the box that lies inside [0,total), or -1. Per
 * dimension indices are NOT range checked (only the flat index is), exactly
 * like the reference. */
static int hgo_box_next(hgo_box *b)
{
    while (b->cursor < b->n_combos) {
        int flat = 0, stride = 1, div = 1;
        for (int d = b->ndim - 1; d >= 0; --d) {
            int k = b->lo[d] + (b->cursor / div) % b->width[d];
            flat += k * stride;
            stride *= b->n_bins[d];
            div *= b->width[d];
        }
        b->cursor += 1;
        if (flat >= 0 && flat < b->total)
            return flat;
    }
    return -1;
}

static void hgo_claim(int shower, int alpha /* global index into *_h arrays */,
                      int C, int B,
                      int *taken_h, const float *ccoords_h, const float *dist_h,
                      const int *mask_h, int *is_alpha_h, const int *orig_h,
                      const float *ccoords, const int *mask,
                      float *best_dsq, int *assignment, int *association,
                      const int *bin_splits, const int *n_bins, float bin_width,
                      const int *to_filtered, int by_max_beta)
{
    float centre[16];
    float lo[HGO_MAX_BIN_DIMS], hi[HGO_MAX_BIN_DIMS];
    float radius = dist_h[alpha];
    const float radius_sq = radius * radius;
    for (int c = 0; c < C; ++c)
        centre[c] = ccoords_h[(size_t)alpha * C + c];

    int solitary = 0;
    if (mask_h[alpha] > 0) {
        radius = 0.f;
        solitary = 1;
    }
    for (int d = 0; d < B; ++d) {
        lo[d] = centre[d] - radius;
        hi[d] = centre[d] + radius;
    }
    is_alpha_h[alpha] = 1;
    taken_h[alpha] = 1;

    hgo_box box;
    hgo_box_set(&box, B, lo, hi, bin_width, n_bins);
    for (;;) {
        int cell = hgo_box_next(&box);
        if (cell < 0)
            break;
        for (int p = bin_splits[cell]; p < bin_splits[cell + 1]; ++p) {
            if (by_max_beta && assignment[p] != -1)
                continue;
            float dsq = 0.f;
            for (int c = 0; c < C; ++c) {
                float a = centre[c] - ccoords[(size_t)p * C + c];
                float b = centre[c] - ccoords[(size_t)p * C + c];
                float sq = a * b;
                dsq = dsq + sq;
            }
            int inside = (dsq <= radius_sq && !solitary && mask[p] == 0) ||
                         (solitary && to_filtered[p] == alpha);
            if (!inside)
                continue;
            if (!by_max_beta) {
                float lhs = best_dsq[p] * radius_sq;
                if (!(lhs >= dsq))
                    continue;
                best_dsq[p] = dsq;
            }
            assignment[p] = shower;
            association[p] = orig_h[alpha];
            if (to_filtered[p] != -1)
                taken_h[to_filtered[p]] = 1;
        }
    }
}

/* Arrays without suffix are all hits in bin-sorted order; *_h are the
 * high-beta subset in the same order. best_dsq is scratch of n_vert floats
 * (only used when by_max_beta == 0). taken_h is scratch of n_vert_h ints.
 * Returns 0, or -1 if the greedy loop stops making progress (the reference
 * throws std::runtime_error there). */
int hgo_assign_to_condensates(int C, int B,
                              int *taken_h,
                              const float *ccoords_h, const float *dist_h,
                              const float *beta_h, const int *mask_h,
                              int *is_alpha_h, const int *orig_h,
                              const int *row_splits_h,
                              const float *ccoords, const int *mask,
                              const int *to_filtered,
                              float *best_dsq,
                              int *assignment, int *association,
                              int *n_condensates, int *alpha_indices,
                              const int *bin_splits, const int *n_bins,
                              const float *bin_widths,
                              const int *row_splits, int n_events,
                              int by_max_beta)
{
    int cells_per_event = 1;
    for (int d = 0; d < B; ++d)
        cells_per_event *= n_bins[d];
    n_condensates[0] = 0;
    int running = 0;

    for (int r = 0; r < n_events; ++r) {
        const int first = row_splits[r], last = row_splits[r + 1];
        const int first_h = row_splits_h[r], last_h = row_splits_h[r + 1];
        for (int q = first_h; q < last_h; ++q) {
            is_alpha_h[q] = 0;
            taken_h[q] = 0;
            alpha_indices[q] = -1;
        }
        for (int p = first; p < last; ++p) {
            assignment[p] = -1;
            association[p] = -1;
            if (!by_max_beta)
                best_dsq[p] = 10e20f;
        }

        int shower = 0;
        int previous = -1;
        for (;;) {
            float top = -1.f;
            int pick = -1;
            for (int q = first_h; q < last_h; ++q) {
                if (taken_h[q] != 0)
                    continue;
                /* the reference indexes the mask with the truth value of
                 * (q > 0), i.e. element 0 or 1 of mask_h */
                if (mask_h[q > 0 ? 1 : 0]) {
                    pick = q;
                    top = 0.f;
                    break;
                }
                if (beta_h[q] > top) {
                    top = beta_h[q];
                    pick = q;
                }
            }
            if (top == -1.f)
                break;
            if (pick == previous)
                return -1;
            previous = pick;

            hgo_claim(shower, pick, C, B, taken_h, ccoords_h, dist_h, mask_h,
                      is_alpha_h, orig_h, ccoords, mask, best_dsq,
                      assignment, association,
                      bin_splits + (size_t)cells_per_event * r, n_bins,
                      bin_widths[0], to_filtered, by_max_beta);

            alpha_indices[first_h + shower] = orig_h[pick];
            ++shower;
        }
        running += shower;
        n_condensates[r + 1] = running;
    }
    return 0;
}

/* ------------------------------------------------------------------ */
/* select_knn_grad: gradient of the kNN squared distances              */
/* ------------------------------------------------------------------ */

/* modules/compiled/select_knn_grad_kernel.cu.cc:81-164 (the reference's CPU
 * functor has an empty body, select_knn_grad_kernel.cc:23-41, so its device
 * kernels define the op). First every vertex collects -2 g (x_k - x_i) over
 * its own neighbours (accumulated in a float, each step evaluated in double as
 * the literal `2.` makes it), then every (vertex, slot) adds 2 g (x_m - x_i)
 * rounded to float into its neighbour m. The reference does the latter with
 * atomicAdd in no particular order; the order here is ascending (vertex,
 * slot), one of its possible outcomes. */
void hgo_select_knn_grad(const float *grad_dist, const int *indices,
                         const float *coords, float *grad_coords,
                         int n_vert, int K, int C)
{
    for (int i = 0; i < n_vert; ++i) {
        for (int c = 0; c < C; ++c) {
            const float xi = coords[(size_t)i * C + c];
            float self = 0.f;
            for (int n = 0; n < K; ++n) {
                int k = indices[(size_t)i * K + n];
                if (k < 0 || k >= n_vert)
                    continue;
                const float g = grad_dist[(size_t)i * K + n];
                const float xk = coords[(size_t)k * C + c];
                self -= 2. * g * (xk - xi);
            }
            grad_coords[(size_t)i * C + c] = self;
        }
    }
    for (int i = 0; i < n_vert; ++i) {
        for (int n = 0; n < K; ++n) {
            int m = indices[(size_t)i * K + n];
            if (m < 0 || m >= n_vert)
                continue;
            const float g = grad_dist[(size_t)i * K + n];
            for (int c = 0; c < C; ++c) {
                const float xi = coords[(size_t)i * C + c];
                const float xm = coords[(size_t)m * C + c];
                float add = 2. * g * (xm - xi);
                grad_coords[(size_t)m * C + c] += add;
            }
        }
    }
}

/* ------------------------------------------------------------------ */
/* push_knn forward and gradient                                       */
/* ------------------------------------------------------------------ */

/* modules/compiled/push_knn_kernel.cc:40-62 */
void hgo_push_knn(const float *weights, const float *features,
                  const int *indices, float *out,
                  int n_vert, int K, int F)
{
    memset(out, 0, sizeof(float) * (size_t)n_vert * F);
    for (int v = 0; v < n_vert; ++v) {
        for (int f = 0; f < F; ++f) {
            const float x = features[(size_t)v * F + f];
            for (int n = 0; n < K; ++n) {
                int m = indices[(size_t)v * K + n];
                if (m < 0)
                    continue;
                const float w = weights[(size_t)v * K + n];
                float term = x * w;
                out[(size_t)m * F + f] += term;
            }
        }
    }
}

/* modules/compiled/push_knn_grad_kernel.cc:23-71 */
void hgo_push_knn_grad(const float *grad, const float *weights,
                       const float *features, const int *indices,
                       float *feat_grad, float *w_grad,
                       int n_vert, int K, int F)
{
    for (int v = 0; v < n_vert; ++v) {
        for (int f = 0; f < F; ++f) {
            float acc = 0.f;
            for (int n = 0; n < K; ++n) {
                int m = indices[(size_t)v * K + n];
                if (m < 0)
                    continue;
                float term = grad[(size_t)m * F + f] * weights[(size_t)v * K + n];
                acc += term;
            }
            feat_grad[(size_t)v * F + f] = acc;
        }
    }
    for (int v = 0; v < n_vert; ++v) {
        for (int n = 0; n < K; ++n) {
            int m = indices[(size_t)v * K + n];
            if (m < 0) {
                w_grad[(size_t)v * K + n] = 0.f;
                continue;
            }
            float acc = 0.f;
            for (int f = 0; f < F; ++f) {
                float term = grad[(size_t)m * F + f] * features[(size_t)v * F + f];
                acc += term;
            }
            w_grad[(size_t)v * K + n] = acc;
        }
    }
}

/* ------------------------------------------------------------------ */
/* local_distance: squared distances to the listed neighbours          */
/* ------------------------------------------------------------------ */

/* modules/compiled/local_distance_kernel.cc:18-70: 0 for a missing neighbour
 * (index < 0) and for the vertex itself, else the serial fp32 sum of squared
 * coordinate differences */
void hgo_local_distance(const int *neigh_idxs, const float *coords,
                        float *distances, int n_coords, int n_out_vert,
                        int n_neigh)
{
    for (int i = 0; i < n_out_vert; ++i) {
        for (int n = 0; n < n_neigh; ++n) {
            const int j = neigh_idxs[(size_t)i * n_neigh + n];
            float dsq = 0.f;
            if (j >= 0 && j != i) {
                for (int c = 0; c < n_coords; ++c) {
                    float d = coords[(size_t)i * n_coords + c] - coords[(size_t)j * n_coords + c];
                    float sq = d * d;
                    dsq += sq;
                }
            }
            distances[(size_t)i * n_neigh + n] = dsq;
        }
    }
}
