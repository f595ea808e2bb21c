"""CPU oracle for the HGCalML custom-op hot path (TEST INFRASTRUCTURE ONLY).

The C part (``hgc_oracle.c``) restates the reference CPU kernels; this module
loads it with ctypes and restates, in numpy, the TensorFlow glue of the
reference's Python wrappers so that whole-op results can be compared:

  BinByCoordinates                  modules/bin_by_coordinates_op.py:15-89
  BinnedSelectKnn                   modules/binned_select_knn_op.py:33-104
  IndexReplacer                     modules/index_replacer_op.py:7-16
  AccumulateKnn / AccumulateLinKnn  modules/accknn_op.py:18-89
  BuildAndAssignCondensatesBinned   modules/assign_condensate_op.py:210-373
  select_knn_grad_kernel            modules/binned_select_knn_op.py:107-118 (the op it registers)
  PushKnn / push_knn_grad_kernel    modules/push_knn_op.py:10-36
  LocalDistance                     modules/local_distance_op.py:11-19
  NeighbourCovariance               modules/neighbour_covariance_op.py:8-62

Only tests/, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package. Nothing in ``hgcalml_amd`` does.

TensorFlow library numerics the glue depends on and that nothing in the
reference tree pins ("parity unpinned"): ``tf.math.pow`` for the default
``n_bins``, the tie order of ``tf.argsort`` (taken as stable here) and the
last-ulp value of ``tf.exp``.
"""
import ctypes
import math
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

_i32p = ctypes.POINTER(ctypes.c_int)
_f32p = ctypes.POINTER(ctypes.c_float)


def build(opt_level_0=False):
    """Compile the C restatement (gcc, seconds)."""
    target = "libhgc_oracle_O0.so" if opt_level_0 else "libhgc_oracle.so"
    subprocess.check_call(["make", "-s", "-C", _HERE, target])
    return os.path.join(_HERE, target)


def lib(opt_level_0=False):
    global _LIB
    if opt_level_0:
        path = os.path.join(_HERE, "libhgc_oracle_O0.so")
        if not os.path.exists(path):
            build(True)
        return ctypes.CDLL(path)
    if _LIB is None:
        path = os.path.join(_HERE, "libhgc_oracle.so")
        if not os.path.exists(path):
            build()
        _LIB = ctypes.CDLL(path)
    return _LIB


def _f(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a, a.ctypes.data_as(_f32p)


def _i(a):
    a = np.ascontiguousarray(a, dtype=np.int32)
    return a, a.ctypes.data_as(_i32p)


# ---------------------------------------------------------------------------
# raw kernels (same argument meaning as the reference functors)
# ---------------------------------------------------------------------------

def bin_by_coordinates_kernel(coords, row_splits, bin_width, n_bins, calc_n_per_bin=True):
    coords, pc = _f(coords)
    row_splits, prs = _i(row_splits)
    bin_width, pbw = _f(np.reshape(bin_width, [1]))
    n_bins, pnb = _i(n_bins)
    n_vert, n_coords = coords.shape
    total = int(np.prod(n_bins.astype(np.int64))) * (len(row_splits) - 1)
    binass = np.zeros((n_vert, n_coords + 1), np.int32)
    flat = np.zeros(n_vert, np.int32)
    nper = np.zeros(total, np.int32)
    bad = lib().hgo_bin_by_coordinates(pc, prs, pbw, pnb,
                                       binass.ctypes.data_as(_i32p), flat.ctypes.data_as(_i32p),
                                       nper.ctypes.data_as(_i32p), n_vert, n_coords, len(row_splits),
                                       total, int(calc_n_per_bin))
    return binass, flat, nper, bad


def shell_enumerate(n_bins, centre, d):
    n_bins, pnb = _i(n_bins)
    centre, pce = _i(centre)
    cap = (2 * d + 1) ** len(n_bins)
    out = np.zeros(cap, np.int32)
    n = lib().hgo_shell_enumerate(len(n_bins), pnb, pce, int(d), out.ctypes.data_as(_i32p), cap)
    return out[:n]


def binned_select_knn_kernel(K, coords, bin_idx, dim_bin_idx, bin_boundaries, n_bins, bin_width,
                             tf_compatible=False, direction=None, opt_level_0=False):
    coords, pc = _f(coords)
    bin_idx, pbi = _i(bin_idx)
    dim_bin_idx, pdb = _i(dim_bin_idx)
    bin_boundaries, pbb = _i(bin_boundaries)
    n_bins, pnb = _i(n_bins)
    bin_width, pbw = _f(np.reshape(bin_width, [1]))
    use_dir = direction is not None
    direction, pdir = _i(direction if use_dir else np.zeros(1, np.int32))
    n_vert, n_coords = coords.shape
    idx = np.empty((n_vert, K), np.int32)
    dist = np.empty((n_vert, K), np.float32)
    lib(opt_level_0).hgo_binned_select_knn(pc, pbi, pdir, pdb, pbb, pnb, pbw,
                                           idx.ctypes.data_as(_i32p), dist.ctypes.data_as(_f32p),
                                           n_vert, int(K), n_coords, len(n_bins), len(bin_boundaries),
                                           int(tf_compatible), int(use_dir))
    return idx, dist


def index_replacer_kernel(to_be_replaced, replacements):
    tbr, ptbr = _i(to_be_replaced)
    rep, prep = _i(replacements)
    out = np.zeros(tbr.shape, np.int32)
    lib().hgo_index_replacer(ptbr, prep, out.ctypes.data_as(_i32p), tbr.size, rep.size)
    return out


def accumulate_knn_kernel(weights, features, indices, mean_and_max=True, opt_level_0=False):
    w, pw = _f(weights)
    x, px = _f(features)
    idx, pidx = _i(indices)
    n_vert, K = idx.shape
    F = x.shape[1]
    out = np.zeros((n_vert, 2 * F if mean_and_max else F), np.float32)
    maxidx = np.zeros((n_vert, F), np.int32)
    lib(opt_level_0).hgo_accumulate_knn(pw, px, pidx, out.ctypes.data_as(_f32p),
                                        maxidx.ctypes.data_as(_i32p), n_vert, K, F, int(mean_and_max))
    return out, maxidx


def accumulate_knn_grad_kernel(grad_out, weights, features, indices, maxidx, opt_level_0=False):
    g, pg = _f(grad_out)
    w, pw = _f(weights)
    x, px = _f(features)
    idx, pidx = _i(indices)
    mi, pmi = _i(maxidx)
    n_vert, K = idx.shape
    F = x.shape[1]
    mean_and_max = g.shape[1] > F
    gw = np.zeros((n_vert, K), np.float32)
    gx = np.zeros((n_vert, F), np.float32)
    lib(opt_level_0).hgo_accumulate_knn_grad(pg, pw, px, pmi, pidx, gw.ctypes.data_as(_f32p),
                                             gx.ctypes.data_as(_f32p), n_vert, K, F, g.shape[1],
                                             int(mean_and_max))
    return gw, gx


def select_knn_grad_kernel(grad_dist, indices, coords):
    g, pg = _f(grad_dist)
    idx, pidx = _i(indices)
    x, px = _f(coords)
    out = np.zeros_like(x)
    lib().hgo_select_knn_grad(pg, pidx, px, out.ctypes.data_as(_f32p), idx.shape[0], idx.shape[1], x.shape[1])
    return out


def push_knn_kernel(weights, features, indices):
    w, pw = _f(weights)
    x, px = _f(features)
    idx, pidx = _i(indices)
    out = np.zeros_like(x)
    lib().hgo_push_knn(pw, px, pidx, out.ctypes.data_as(_f32p), idx.shape[0], idx.shape[1], x.shape[1])
    return out


def push_knn_grad_kernel(grad, weights, features, indices):
    """(weight_grad, feature_grad), the output order of modules/compiled/push_knn_grad_module.cc:12-13"""
    g, pg = _f(grad)
    w, pw = _f(weights)
    x, px = _f(features)
    idx, pidx = _i(indices)
    fgrad = np.zeros_like(x)
    wgrad = np.zeros_like(w)
    lib().hgo_push_knn_grad(pg, pw, px, pidx, fgrad.ctypes.data_as(_f32p), wgrad.ctypes.data_as(_f32p),
                            idx.shape[0], idx.shape[1], x.shape[1])
    return wgrad, fgrad


def local_distance_kernel(coords, neigh_idxs):
    x, px = _f(coords)
    idx, pidx = _i(neigh_idxs)
    out = np.zeros(idx.shape, np.float32)
    lib().hgo_local_distance(pidx, px, out.ctypes.data_as(_f32p), x.shape[1], idx.shape[0], idx.shape[1])
    return out


def assign_to_condensates_kernel(ccoords, dist, beta, mask, bin_splits, to_filtered, orig_h,
                                 row_splits, n_bins, bin_width, ccoords_h, dist_h, beta_h, mask_h,
                                 row_splits_h, assign_by_max_beta, opt_level_0=False):
    cc, pcc = _f(ccoords)
    _, _ = _f(dist)
    msk, pmsk = _i(mask)
    bs, pbs = _i(bin_splits)
    tf_, ptf = _i(to_filtered)
    oh, poh = _i(orig_h)
    rs, prs = _i(row_splits)
    nb, pnb = _i(n_bins)
    bw, pbw = _f(np.reshape(bin_width, [1]))
    cch, pcch = _f(ccoords_h)
    dh, pdh = _f(dist_h)
    bh, pbh = _f(beta_h)
    # the reference reads element 1 of the high-beta mask unconditionally
    mh = np.zeros(max(2, np.size(mask_h)), np.int32)
    mh[:np.size(mask_h)] = np.reshape(mask_h, [-1])
    pmh = mh.ctypes.data_as(_i32p)
    rsh, prsh = _i(row_splits_h)
    n, C = cc.shape
    nh = bh.size
    taken = np.zeros(max(nh, 1), np.int32)
    is_alpha = np.zeros(max(nh, 1), np.int32)
    alpha = np.zeros(max(nh, 1), np.int32)
    best = np.zeros(max(n, 1), np.float32)
    assignment = np.zeros(n, np.int32)
    association = np.zeros(n, np.int32)
    ncond = np.zeros(len(rs), np.int32)
    rc = lib(opt_level_0).hgo_assign_to_condensates(
        C, len(nb), taken.ctypes.data_as(_i32p), pcch, pdh, pbh, pmh, is_alpha.ctypes.data_as(_i32p),
        poh, prsh, pcc, pmsk, ptf, best.ctypes.data_as(_f32p), assignment.ctypes.data_as(_i32p),
        association.ctypes.data_as(_i32p), ncond.ctypes.data_as(_i32p), alpha.ctypes.data_as(_i32p),
        pbs, pnb, pbw, prs, len(rs) - 1, int(assign_by_max_beta))
    if rc != 0:
        raise RuntimeError("Error progressing to next highest beta")
    return is_alpha[:nh], assignment, alpha[:nh], association, ncond


# ---------------------------------------------------------------------------
# wrapper glue, numpy restatement
# ---------------------------------------------------------------------------

def BinByCoordinates(coordinates, row_splits, bin_width=None, n_bins=None, calc_n_per_bin=True,
                     pre_normalized=False):
    x = np.asarray(coordinates, np.float32)
    if not np.all(np.isfinite(x)):
        raise ValueError("BinByCoordinates: input coordinates not finite")
    if not pre_normalized:
        x = x - x.min(axis=0, keepdims=True)
    dmax = x.max(axis=0)
    dmax = np.where(x.min(axis=0) == dmax, dmax + np.float32(1.), dmax) + np.float32(1e-3)
    dmax = np.where(np.isfinite(dmax), dmax, np.float32(1.)).astype(np.float32)
    if bin_width is None:
        assert n_bins is not None
        bin_width = np.max(dmax / np.float32(n_bins)).astype(np.float32).reshape(1)
        n_bins = None
    if n_bins is None:
        nb = dmax / np.asarray(bin_width, np.float32)
        nb = nb + np.float32(1.)
        n_bins = nb.astype(np.int32)
    bin_width = np.asarray(bin_width, np.float32).reshape(1)
    binass, flat, nper, _ = bin_by_coordinates_kernel(x, row_splits, bin_width, n_bins, calc_n_per_bin)
    if calc_n_per_bin:
        return binass, flat, n_bins, bin_width, nper
    return binass, flat, n_bins, bin_width


def default_knn_n_bins(first_event_size, K, max_bin_dims):
    """modules/binned_select_knn_op.py:59-63 (float32 pow, truncation, clamp to [5,30])"""
    v = np.power(np.float32(first_event_size) / np.float32(K / 32), np.float32(1 / max_bin_dims))
    return int(min(30, max(5, int(np.int32(v)))))


def BinnedSelectKnn(K, coords, row_splits, direction=None, n_bins=None, max_bin_dims=3,
                    tf_compatible=False, max_radius=None, raw_slot_order=True, opt_level_0=False):
    """Reference wrapper, then (only if ``max_radius`` > 0) the radius mask of
    modules/compiled/select_knn_kernel.cc:158,244-245: neighbours with
    d^2 > r^2 become padding ((-1, 0.0), or (self, 0.0) in tf_compatible mode). The reference wrapper itself ignores
    ``max_radius``; pass ``None`` to get exactly what it returns."""
    coords = np.asarray(coords, np.float32)
    row_splits = np.asarray(row_splits, np.int32)
    assert row_splits[-1] == coords.shape[0]
    max_bin_dims = min(max_bin_dims, coords.shape[1])
    if n_bins is None:
        n_bins = default_knn_n_bins(int(row_splits[1]), K, max_bin_dims)
    dbinning, binning, nb, bin_width, nper = BinByCoordinates(coords[:, :max_bin_dims], row_splits,
                                                             n_bins=n_bins)
    sorting = np.argsort(binning, kind="stable").astype(np.int32)
    scoords = coords[sorting]
    sbinning = binning[sorting]
    sdbinning = dbinning[sorting]
    sdir = None if direction is None else np.asarray(direction, np.int32)[sorting]
    bin_boundaries = np.concatenate([np.zeros(1, np.int32), np.cumsum(nper, dtype=np.int32)])
    idx_s, dist_s = binned_select_knn_kernel(K, scoords, sbinning, sdbinning, bin_boundaries, nb,
                                             bin_width, tf_compatible, sdir, opt_level_0)
    idx_r = index_replacer_kernel(idx_s, sorting)
    idx = np.zeros_like(idx_r)
    dist = np.zeros_like(dist_s)
    idx[sorting] = idx_r
    dist[sorting] = dist_s
    dist = np.where(idx < 0, np.float32(0.), dist)
    if max_radius is not None and max_radius > 0:
        r = np.float32(max_radius)
        rsq = np.float32(r * r)
        outside = dist > rsq
        outside[:, 0] = False
        # a neighbour beyond the radius is never filled in, so its slot keeps the
        # default: -1, or the vertex itself in tf_compatible mode (select_knn_kernel.cc:61-84)
        pad = np.arange(idx.shape[0], dtype=np.int32)[:, None] if tf_compatible else np.int32(-1)
        idx = np.where(outside, pad, idx)
        dist = np.where(outside, np.float32(0.), dist)
    return idx, dist


def canonical_knn(idx, dist):
    """Slot 0 kept; the other slots ordered by ascending (d^2, index) with the
    padding at the tail. Used to compare neighbour sets."""
    idx = np.asarray(idx)
    dist = np.asarray(dist)
    n, K = idx.shape
    if K <= 1:
        return idx.copy(), dist.copy()
    # padding is -1, or a repeated self reference in tf_compatible mode
    pad = (idx[:, 1:] < 0) | (idx[:, 1:] == idx[:, :1])
    dkey = np.where(pad, np.float32(np.inf), dist[:, 1:])
    ikey = np.where(pad, np.iinfo(np.int32).max, idx[:, 1:])
    order = np.lexsort((ikey, dkey), axis=1)
    ci = np.take_along_axis(idx[:, 1:], order, axis=1)
    cd = np.take_along_axis(dist[:, 1:], order, axis=1)
    return (np.concatenate([idx[:, :1], ci], axis=1), np.concatenate([dist[:, :1], cd], axis=1))


def IndexReplacer(to_be_replaced, replacements):
    return index_replacer_kernel(to_be_replaced, replacements)


def AccumulateLinKnn(weights, features, indices, mean_and_max=True):
    return accumulate_knn_kernel(weights, features, indices, mean_and_max)


def AccumulateKnn(distances, features, indices, mean_and_max=True):
    w = np.exp(-np.asarray(distances, np.float32)).astype(np.float32)
    return accumulate_knn_kernel(w, features, indices, mean_and_max)


def AccumulateKnnSumw(distances, features, indices, mean_and_max=False, linear=False):
    """modules/GravNetLayersRagged.py:35-62: weighted mean normalised by the
    accumulated weight (a column of ones rides along), divide_no_nan"""
    F = features.shape[1]
    x = np.concatenate([features, np.ones_like(features[:, :1])], axis=1).astype(np.float32)
    f, midx = (AccumulateLinKnn if linear else AccumulateKnn)(distances, x, indices, mean_and_max)
    norm = f[:, F:F + 1]
    with np.errstate(divide="ignore", invalid="ignore"):
        fmean = np.where(norm == 0, np.float32(0), f[:, :F] / norm).astype(np.float32)
    if mean_and_max:
        fmean = np.concatenate([fmean, f[:, F + 1:-1]], axis=1)
    return fmean, midx


def LocalDistance(coords, neighbour_idxs):
    return local_distance_kernel(coords, neighbour_idxs)


def NeighbourCovariance(coordinates, distsq, features, n_idxs):
    """modules/neighbour_covariance_op.py:8-62: feature-weighted mean and covariance
    of the neighbours' coordinates, three mean-only accumulations; returns
    (cov [N, F, C*C], mean_C [N, F, C])"""
    coordinates = np.asarray(coordinates, np.float32)
    features = (1.0 / (1.0 + np.exp(-np.asarray(features, np.float64)))).astype(np.float32) + np.float32(1e-3)
    n, nF = features.shape
    nC = coordinates.shape[1]
    nKf = np.float32(distsq.shape[1])

    def no_nan_div(a, b):
        with np.errstate(divide="ignore", invalid="ignore"):
            return np.where(b == 0, np.float32(0), a / b).astype(np.float32)
    sum_F = AccumulateKnn(distsq, features, n_idxs, mean_and_max=False)[0] * nKf
    FC = (coordinates[:, None, :] * features[:, :, None]).astype(np.float32).reshape(n, nF * nC)
    sum_FC = AccumulateKnn(distsq, FC, n_idxs, mean_and_max=False)[0] * nKf
    mean_C = no_nan_div(sum_FC.reshape(n, nF, nC), sum_F[:, :, None] + np.float32(1e-3))
    centered = (coordinates[:, None, :] - mean_C).astype(np.float32)
    cov = (centered[:, :, :, None] * centered[:, :, None, :]).astype(np.float32).reshape(n, nF, nC * nC)
    cov = (cov * features[:, :, None]).astype(np.float32).reshape(n, nF * nC * nC)
    cov = AccumulateKnn(distsq, cov, n_idxs, mean_and_max=False)[0] * nKf
    cov = no_nan_div(cov.reshape(n, nF, nC * nC), sum_F[:, :, None] + np.float32(1e-3))
    return cov, mean_C


def PushKnn(w, f, nidx):
    return push_knn_kernel(w, f, nidx)


def AccumulateKnnGrad(grad_out, distances, features, indices, maxidx, linear=False):
    """Gradients w.r.t. (distances-or-weights, features) as TF autodiff chains
    them through modules/accknn_op.py:52,71-89."""
    d = np.asarray(distances, np.float32)
    w = d if linear else np.exp(-d).astype(np.float32)
    gw, gx = accumulate_knn_grad_kernel(grad_out, w, features, indices, maxidx)
    if linear:
        return gw, gx
    return (-(w * gw)).astype(np.float32), gx


def merge_noise_as_indiv_cp(assignment, asso_idx, alpha_idx, is_cond, n_condensates, row_splits):
    """modules/assign_condensate_op.py:9-44 (the keep_noise post-pass) on flat arrays.
    The reference numbers the noise hits of an event with a cumulative sum over ALL
    hits minus the previous event's running maximum (`cumsum_ragged`, :9-13), gives
    noise hit number j the shower index j-1, lifts the event's real showers by the
    event's noise count, lists `noise indices ++ condensation points` per event and
    recounts the condensation points per event from the merged flags. Events
    without hits are outside what it defines (reduce_max of an empty row)."""
    a = np.asarray(assignment, np.int32).reshape(-1)
    asso_idx = np.asarray(asso_idx, np.int32)
    alpha_idx = np.asarray(alpha_idx, np.int32)
    cond = np.asarray(is_cond, bool).reshape(-1)
    ncond = np.asarray(n_condensates, np.int32)
    rs = np.asarray(row_splits, np.int64)
    n = len(a)
    noise = a < 0
    running = np.cumsum(noise.astype(np.int32))                     # tf.cumsum over the flat values
    at_event_end = np.array([running[rs[e + 1] - 1] for e in range(len(rs) - 1)], np.int32)
    carried = np.concatenate([np.zeros(1, np.int32), at_event_end[:-1]])
    x = running - np.repeat(carried, np.diff(rs))
    x = np.where(noise, x, 0)
    n_noise = np.array([x[rs[e]:rs[e + 1]].max() for e in range(len(rs) - 1)], np.int32)
    new_assignment = np.where(noise, x - 1, a + np.repeat(n_noise, np.diff(rs))).astype(np.int32)
    allrange = np.arange(n, dtype=np.int32)
    merged = [np.concatenate([allrange[rs[e]:rs[e + 1]][noise[rs[e]:rs[e + 1]]], alpha_idx[ncond[e]:ncond[e + 1]]])
              for e in range(len(rs) - 1)]
    new_alpha = np.concatenate(merged).astype(np.int32) if merged else np.zeros(0, np.int32)
    new_cond = np.where(asso_idx < 0, True, cond)
    new_asso = np.where(asso_idx < 0, allrange, asso_idx).astype(np.int32)
    per_event = np.array([new_cond[rs[e]:rs[e + 1]].sum() for e in range(len(rs) - 1)], np.int32)
    new_ncond = np.concatenate([ncond[0:1], np.cumsum(per_event, dtype=np.int32)]).astype(np.int32)
    return new_assignment[:, None], new_asso, new_alpha, new_cond[:, None], new_ncond


def BuildAndAssignCondensatesBinned(ccoords, betas, dist, row_splits, beta_threshold,
                                    no_condensation_mask=None, distance_threshold=1.,
                                    assign_by_max_beta=False, nbin_dims=3, keep_noise=False,
                                    opt_level_0=False, return_kernel_inputs=False):
    assert 1 <= nbin_dims <= 6
    assert 0. <= beta_threshold <= 1.
    assert distance_threshold > 0.
    ccoords = np.asarray(ccoords, np.float32)
    betas = np.asarray(betas, np.float32).reshape(-1)
    row_splits = np.asarray(row_splits, np.int32)
    n = ccoords.shape[0]
    n_events = len(row_splits) - 1
    dist = (np.asarray(dist, np.float32).reshape(-1) / np.float32(distance_threshold)).astype(np.float32)
    mask = (np.zeros(n, np.int32) if no_condensation_mask is None
            else np.asarray(no_condensation_mask, np.int32).reshape(-1))

    n_total = int(row_splits[-1] - row_splits[0])
    n_bins_sc = max(4, min(int(math.ceil(math.pow(n_total / 5, 1 / 3))), 25))
    cc = ccoords - ccoords.min(axis=0, keepdims=True)
    _, bins_flat, n_bins, bin_width = BinByCoordinates(cc[:, :min(cc.shape[1], nbin_dims)], row_splits,
                                                       n_bins=n_bins_sc, calc_n_per_bin=False,
                                                       pre_normalized=True)
    sorting = np.argsort(bins_flat, kind="stable").astype(np.int32)
    back = np.argsort(sorting, kind="stable")
    cc = cc[sorting]
    betas_s = betas[sorting]
    dist_s = dist[sorting]
    mask_s = mask[sorting]
    bins_s = bins_flat[sorting]
    total_bins = int(np.prod(n_bins.astype(np.int64))) * n_events
    bin_splits = np.concatenate([np.zeros(1, np.int64),
                                 np.cumsum(np.bincount(bins_s, minlength=total_bins))]).astype(np.int32)
    high = (betas_s > np.float32(beta_threshold)) | (mask_s > 0)
    event_of = np.searchsorted(row_splits[1:], np.arange(n), side="right")
    rs_h = np.concatenate([np.zeros(1, np.int64),
                           np.cumsum(np.bincount(event_of[high], minlength=n_events))]).astype(np.int32)
    to_filtered = np.full(n, -1, np.int32)
    to_filtered[high] = np.arange(int(high.sum()), dtype=np.int32)
    kernel_inputs = dict(ccoords=cc, dist=dist_s, beta=betas_s, mask=mask_s, bin_splits=bin_splits,
                         to_filtered=to_filtered, orig_h=sorting[high], row_splits=row_splits,
                         n_bins=n_bins, bin_width=bin_width, ccoords_h=cc[high], dist_h=dist_s[high],
                         beta_h=betas_s[high], mask_h=mask_s[high], row_splits_h=rs_h,
                         assign_by_max_beta=assign_by_max_beta)
    _, assignment, alpha, asso, ncond = assign_to_condensates_kernel(opt_level_0=opt_level_0,
                                                                     **kernel_inputs)
    assignment = assignment[back]
    asso = asso[back]
    alpha_idx = alpha[alpha != -1]
    is_cond = np.zeros(n, bool)
    is_cond[alpha_idx] = True
    out = (assignment[:, None], asso, alpha_idx, is_cond[:, None], ncond)
    if keep_noise:
        out = merge_noise_as_indiv_cp(*out, row_splits)
    if return_kernel_inputs:
        return out, kernel_inputs
    return out
