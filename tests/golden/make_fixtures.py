#!/usr/bin/env python3
"""Writes the small input/output vectors under tests/golden/ (run from the repository root:
``python tests/golden/make_fixtures.py``).

The expected outputs come from the CPU oracle (``oracle/``), whose functions are pinned by
tests/test_oracle_pins.py against brute force, closed forms and float64 autograd. The reference's own
kernels cannot be built in this image (they need the TensorFlow and CUDA runtime headers) and its test
tree holds no numeric vectors for these ops, so these files are a frozen copy of this repository's own
oracle: regression fixtures. They pin nothing independently of the oracle (tests/test_oracle_pins.py does
that); they catch drift of the oracle and of the GPU path between commits. Seeds are fixed; the
arrays of a second run are identical.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(1, os.path.dirname(HERE))  # tests/workloads.py

import oracle  # noqa: E402


def g1_binning():
    rng = np.random.default_rng(101)
    coords = (rng.random((64, 3), dtype=np.float32) * np.float32(4.0)).astype(np.float32)
    coords[5] = [1.0, 2.0, 0.5]          # exactly on bin edges for bin_width 0.5
    coords[9] = [9.0, 0.1, 0.1]          # outside the grid in dimension 0: falls back to bin 0 there
    rs = np.array([0, 30, 64], np.int32)
    bw = np.array([0.5], np.float32)
    nb = np.array([8, 8, 8], np.int32)
    binass, flat, nper, n_bad = oracle.bin_by_coordinates_kernel(coords, rs, bw, nb)
    return dict(coords=coords, row_splits=rs, bin_width=bw, n_bins=nb, binass=binass, flat=flat, nper=nper,
                n_bad=np.int32(n_bad))


def g2_knn():
    import workloads
    cfg = workloads.cfg2(scale=512 / 150000, seed=102)
    coords = cfg["coords"][:512].copy()
    rs = np.array([0, 200, 512], np.int32)
    out = dict(coords=coords, row_splits=rs)
    direction = np.random.default_rng(103).integers(0, 5, 512).astype(np.int32)
    out["direction"] = direction
    for K in (4, 16, 64):
        idx, dist = oracle.canonical_knn(*oracle.BinnedSelectKnn(K, coords, rs, n_bins=5))
        out["idx_K%d" % K], out["dist_K%d" % K] = idx, dist
    idx, dist = oracle.canonical_knn(*oracle.BinnedSelectKnn(16, coords, rs, direction=direction, n_bins=5))
    out["idx_dir"], out["dist_dir"] = idx, dist
    idx, dist = oracle.canonical_knn(*oracle.BinnedSelectKnn(16, coords, rs, n_bins=5, tf_compatible=True))
    out["idx_tfc"], out["dist_tfc"] = idx, dist
    # an event with fewer points than K
    rs_small = np.array([0, 10, 512], np.int32)
    idx, dist = oracle.canonical_knn(*oracle.BinnedSelectKnn(16, coords, rs_small, n_bins=5))
    out["row_splits_small"], out["idx_small"], out["dist_small"] = rs_small, idx, dist
    return out


def g3_accumulate():
    rng = np.random.default_rng(104)
    n, K = 128, 8
    out = {}
    for F in (3, 32):
        x = rng.standard_normal((n, F)).astype(np.float32)
        idx = np.stack([np.concatenate([[v], rng.permutation(np.delete(np.arange(n), v))[:K - 1]])
                        for v in range(n)]).astype(np.int32)
        idx[10:30, 5:] = -1
        idx[40, 0] = -1
        idx[50, 3:] = 50
        w = np.exp(-rng.random((n, K), dtype=np.float32)).astype(np.float32)
        w[60, 2] = w[60, 6]
        x[idx[60, 2]] = x[idx[60, 6]]      # exact ties in w*x between two slots
        g = rng.standard_normal((n, 2 * F)).astype(np.float32)
        res, arg = oracle.AccumulateLinKnn(w, x, idx)
        res1, _ = oracle.AccumulateLinKnn(w, x, idx, mean_and_max=False)
        gw, gx = oracle.accumulate_knn_grad_kernel(g, w, x, idx, arg)
        gw1, gx1 = oracle.accumulate_knn_grad_kernel(g[:, :F].copy(), w, x, idx, arg)
        for k, v in dict(x=x, idx=idx, w=w, g=g, out=res, arg=arg, out_mean=res1, gw=gw, gx=gx, gw_mean=gw1,
                         gx_mean=gx1).items():
            out["F%d_%s" % (F, k)] = v
    return out


def g5_condensates():
    import workloads
    cfg = workloads.cfg5(scale=1000 / 62500, seed=105, n_events=2)
    out = dict(ccoords=cfg["ccoords"], betas=cfg["betas"], dist=cfg["dist"], row_splits=cfg["row_splits"])
    for mode in (True, False):
        for t_b in (1e-5, 0.1, 0.9999):
            res = oracle.BuildAndAssignCondensatesBinned(cfg["ccoords"], cfg["betas"], cfg["dist"], cfg["row_splits"],
                                                         t_b, assign_by_max_beta=mode)
            for name, v in zip(("assignment", "asso", "alpha", "is_cond", "ncond"), res):
                out["%s_%s_tb%g" % (name, "maxbeta" if mode else "mindist", t_b)] = np.asarray(v)
    zeros = np.zeros_like(cfg["ccoords"])
    res = oracle.BuildAndAssignCondensatesBinned(zeros, cfg["betas"], cfg["dist"], cfg["row_splits"], 0.1,
                                                 assign_by_max_beta=True)
    for name, v in zip(("assignment", "asso", "alpha", "is_cond", "ncond"), res):
        out["%s_degenerate" % name] = np.asarray(v)
    return out


def g6_small_ops():
    rng = np.random.default_rng(106)
    tbr = rng.integers(-1, 40, size=(50, 4)).astype(np.int32)
    rep = rng.permutation(40).astype(np.int32)
    n, K, C, F = 96, 6, 3, 5
    x = rng.standard_normal((n, C)).astype(np.float32)
    feat = rng.standard_normal((n, F)).astype(np.float32)
    idx = np.stack([np.concatenate([[v], rng.permutation(np.delete(np.arange(n), v))[:K - 1]])
                    for v in range(n)]).astype(np.int32)
    idx[3:9, 3:] = -1
    g = rng.standard_normal((n, K)).astype(np.float32)
    w = (rng.random((n, K)) + 0.1).astype(np.float32)
    gf = rng.standard_normal((n, F)).astype(np.float32)
    wgrad, fgrad = oracle.push_knn_grad_kernel(gf, w, feat, idx)
    return dict(tbr=tbr, rep=rep, replaced=oracle.IndexReplacer(tbr, rep), coords=x, idx=idx, grad_dist=g,
                grad_coords=oracle.select_knn_grad_kernel(g, idx, x), w=w, feat=feat, pushed=oracle.PushKnn(w, feat, idx),
                grad_pushed=gf, push_wgrad=wgrad, push_fgrad=fgrad)


FIXTURES = dict(g1_binning=g1_binning, g2_knn=g2_knn, g3_accumulate=g3_accumulate, g5_condensates=g5_condensates,
                g6_small_ops=g6_small_ops)


def main():
    for name, fn in FIXTURES.items():
        path = os.path.join(HERE, name + ".npz")
        np.savez_compressed(path, **fn())
        print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
