"""Pins the CPU oracle (oracle/) against independent formulations.

The reference tree holds no golden vectors for these ops and its kernels cannot
be built in this image, so each oracle function is checked against what the
mathematics fixes: brute force, closed forms, invariants and hand-computed tiny
cases chosen so that a wrong sign, index, tie rule or summation order fails.
"""
import numpy as np
import pytest

import workloads


from helpers import brute_knn_row, check_knn_rows, serial_distsq  # noqa: E402,F401


# ------------------------------------------------------------------ binning

def test_bin_kernel_matches_closed_form(oracle):
    rng = np.random.default_rng(1)
    n = 64
    coords = (rng.random((n, 3), dtype=np.float32) * np.float32(3.0)).astype(np.float32)
    bw = np.array([0.5], np.float32)
    nb = np.array([6, 7, 6], np.int32)
    coords[5] = [1.0, 1.5, 2.5]          # exactly on bin edges
    coords[9, 1] = 3.6                   # index 7 -> beyond n_bins[1] -> falls back to 0
    coords[11, 0] = -0.7                 # negative index -> 0
    rs = np.array([0, 20, 20, 64], np.int32)   # with an empty event
    binass, flat, nper, bad = oracle.bin_by_coordinates_kernel(coords, rs, bw, nb)
    assert bad == 2
    k = np.trunc(coords / bw[0]).astype(np.int64)
    k[(k < 0) | (k >= nb[None, :])] = 0
    ev = np.array([0] * 20 + [2] * 44)
    want_flat = ((ev * nb[0] + k[:, 0]) * nb[1] + k[:, 1]) * nb[2] + k[:, 2]
    assert (flat == want_flat).all()
    assert (binass[:, 0] == ev).all() and (binass[:, 1:] == k).all()
    assert (binass[5] == [0, 2, 3, 5]).all()
    assert (nper == np.bincount(want_flat, minlength=6 * 7 * 6 * 3)).all() and nper.sum() == n


def test_bin_wrapper_formulas(oracle):
    rng = np.random.default_rng(2)
    x = (rng.random((500, 3), dtype=np.float32) * np.array([4., 2., 1.], np.float32)
         + np.array([-3., 5., 0.], np.float32)).astype(np.float32)
    rs = np.array([0, 200, 500], np.int32)
    binass, flat, nb, bw, nper = oracle.BinByCoordinates(x, rs, n_bins=10)
    ext = (x - x.min(0)).max(0).astype(np.float32) + np.float32(1e-3)
    assert bw.shape == (1,) and bw[0] == np.max(ext / np.float32(10))
    assert (nb == (ext / bw[0] + np.float32(1)).astype(np.int32)).all()
    assert nb.max() in (10, 11) and (nb >= 1).all()
    assert nper.shape == (int(np.prod(nb)) * 2,) and nper.sum() == 500
    # every point lies inside its bin (up to the fp32 rounding of the divide)
    shifted = x - x.min(0)
    assert (np.abs(shifted / bw[0] - binass[:, 1:] - 0.5) <= 0.5 + 1e-4).all()
    # a degenerate dimension gets extent 1 + 1e-3
    x[:, 2] = 7.0
    _, _, nb2, bw2, _ = oracle.BinByCoordinates(x, rs, n_bins=10)
    assert nb2[2] == int(np.float32(1.001) / bw2[0] + np.float32(1))
    # bin_width given instead
    _, _, nb3, bw3, _ = oracle.BinByCoordinates(x, rs, bin_width=np.array([0.25], np.float32))
    assert bw3[0] == np.float32(0.25) and nb3[0] == int(ext[0] / np.float32(0.25) + 1)


# ------------------------------------------------------------------ shells

@pytest.mark.parametrize("nb", [(4, 5), (3, 4, 5), (6, 2, 3), (2, 3, 2, 3), (2, 2, 3, 2, 2)])
def test_shells_partition_grid(oracle, nb):
    rng = np.random.default_rng(3)
    nb = np.array(nb, np.int32)
    total = int(np.prod(nb))
    for _ in range(4):
        centre = np.array([rng.integers(0, b) for b in nb], np.int32)
        seen = []
        for d in range(int(nb.max()) + 1):
            cells = oracle.shell_enumerate(nb, centre, d)
            unr = np.array(np.unravel_index(cells, nb)).T.reshape(-1, len(nb))
            assert (np.abs(unr - centre[None, :]).max(axis=1) == d).all()
            # dimension 0 is the most significant digit: the flat index rises
            assert (np.diff(cells) > 0).all()
            seen.append(cells)
        seen = np.concatenate(seen)
        assert len(seen) == total and len(np.unique(seen)) == total
        assert len(oracle.shell_enumerate(nb, centre, int(nb.max()) + 1)) == 0


# ------------------------------------------------------------------ kNN

def test_knn_sets_vs_brute_force_uniform(oracle):
    cfg = workloads.cfg1(scale=0.1)  # 2000 points, K=16
    coords = cfg["coords"]
    rs = np.array([0, 700, 2000], np.int32)
    idx, dist = oracle.BinnedSelectKnn(16, coords, rs, n_bins=8)
    ties = check_knn_rows(oracle, idx, dist, coords, rs, 16, np.arange(2000))
    assert ties == 0
    # slot order of the reference algorithm is generally not distance sorted
    assert (np.diff(dist[:, 1:], axis=1) < 0).any()


def test_knn_sets_vs_brute_force_clustered_4d(oracle):
    cfg = workloads.cfg2(scale=0.04)  # 6000 points, 4-D distance over 3 binned dims
    coords = cfg["coords"]
    rs = np.array([0, 2500, 6000], np.int32)
    idx, dist = oracle.BinnedSelectKnn(64, coords, rs, n_bins=12)
    rows = np.random.default_rng(4).choice(6000, 600, replace=False)
    assert check_knn_rows(oracle, idx, dist, coords, rs, 64, rows) == 0


def test_knn_small_event_padding_direction_and_tf_compat(oracle):
    rng = np.random.default_rng(5)
    coords = rng.standard_normal((330, 3)).astype(np.float32)
    rs = np.array([0, 7, 7, 30, 330], np.int32)  # 7 < K, empty, 23 < K, 300
    K = 24
    for tfc in (False, True):
        idx, dist = oracle.BinnedSelectKnn(K, coords, rs, n_bins=5, tf_compatible=tfc)
        check_knn_rows(oracle, idx, dist, coords, rs, K, np.arange(330), tf_compatible=tfc)
    direction = rng.integers(0, 4, size=330).astype(np.int32)
    idx, dist = oracle.BinnedSelectKnn(K, coords, rs, n_bins=5, direction=direction)
    check_knn_rows(oracle, idx, dist, coords, rs, K, np.arange(330), direction=direction)
    # radius mask (select_knn rule: keep d^2 <= r^2)
    idx, dist = oracle.BinnedSelectKnn(K, coords, rs, n_bins=5, max_radius=0.6)
    ci, cd = oracle.canonical_knn(idx, dist)
    check_knn_rows(oracle, ci, cd, coords, rs, K, np.arange(330), radius=0.6)
    assert (ci[:, 1:] < 0).any() and (np.diff((ci[:, 1:] < 0).astype(int), axis=1) >= 0).all()


def test_knn_lattice_ties_are_valid_sets(oracle):
    g = np.arange(8, dtype=np.float32)
    coords = np.stack(np.meshgrid(g, g, g, indexing="ij"), -1).reshape(-1, 3)
    rs = np.array([0, 512], np.int32)
    idx, dist = oracle.BinnedSelectKnn(8, coords, rs, n_bins=5)
    ties = check_knn_rows(oracle, idx, dist, coords, rs, 8, np.arange(512))
    assert ties > 100  # the lattice makes most K-th boundaries exact ties


def test_default_n_bins_formula(oracle):
    assert oracle.default_knn_n_bins(20000, 16, 3) == 30
    assert oracle.default_knn_n_bins(150000, 64, 3) == 30
    assert oracle.default_knn_n_bins(1000, 32, 3) == 10   # 1000^(1/3) = 10 (float32 pow)
    assert oracle.default_knn_n_bins(100, 64, 3) == 5     # clamp below
    assert oracle.default_knn_n_bins(4000, 32, 2) == 30   # sqrt(4000) = 63 -> clamp


# ------------------------------------------------------------------ index replacer

def test_index_replacer(oracle):
    rep = np.array([10, 11, 12, 13], np.int32)
    tbr = np.array([[0, 3, -1], [2, -5, 7]], np.int32)
    out = oracle.IndexReplacer(tbr, rep)
    assert (out == [[10, 13, -1], [12, -5, 0]]).all()  # 7 is out of range: left at the zero init


# ------------------------------------------------------------------ accumulate forward

def np_accumulate(w, x, idx, mean_and_max=True):
    """gather -> multiply -> slot-serial fp32 sum / K, and max with the
    reference's rules, vectorised over (vertex, feature)."""
    n, K = idx.shape
    F = x.shape[1]
    s = np.zeros((n, F), np.float32)
    best = np.zeros((n, F), np.float32)
    arg = np.zeros((n, F), np.int32)
    for k in range(K):
        j = idx[:, k]
        ok = (j >= 0)[:, None]
        wf = (x[np.maximum(j, 0)] * w[:, k:k + 1]).astype(np.float32)
        s = np.where(ok, (s + wf).astype(np.float32), s)
        take = ok & ((wf >= best) | (k == 0))
        best = np.where(take, wf, best)
        arg = np.where(take, j[:, None], arg)
    mean = (s / np.float32(K)).astype(np.float32)
    return (np.concatenate([mean, best], 1), arg) if mean_and_max else (mean, arg)


def test_accumulate_hand_cases(oracle):
    x = np.array([[1., -2.], [3., 4.], [-5., 0.5]], np.float32)
    idx = np.array([[0, 1, 2], [1, 2, -1], [-1, 0, 1]], np.int32)
    w = np.array([[1., .5, .25], [2., 1., 9.], [7., 1., 1.]], np.float32)
    out, arg = oracle.AccumulateLinKnn(w, x, idx)
    # vertex 0: wf = [1,-2],[1.5,2],[-1.25,.125]; mean = sum/3 ; max: slot 0 seeds, then >=
    assert np.allclose(out[0], [1.25 / 3, 0.125 / 3, 1.5, 2.0])
    assert (arg[0] == [1, 1]).all()
    # vertex 1: slots (1,w2) (2,w1) pad: wf=[6,8],[-5,.5]; divides by K=3, not by 2
    assert np.allclose(out[1], [1. / 3, 8.5 / 3, 6., 8.])
    assert (arg[1] == [1, 1]).all()
    # vertex 2: slot 0 is padding -> max floored at 0 with index 0 unless something >= 0 comes
    # wf slot1 = [1,-2], slot2 = [3,4]
    assert np.allclose(out[2], [4. / 3, 2. / 3, 3., 4.])
    assert (arg[2] == [1, 1]).all()
    # all-negative contributions with slot 0 padded: max stays 0, index 0
    x2 = -np.abs(x)
    out2, arg2 = oracle.AccumulateLinKnn(w, x2, idx)
    assert (out2[2, 2:] == 0).all() and (arg2[2] == 0).all()
    # exact tie: the later slot wins
    x3 = np.array([[2.], [2.], [2.]], np.float32)
    out3, arg3 = oracle.AccumulateLinKnn(np.ones((3, 3), np.float32), x3, np.array([[0, 1, 2]] * 3, np.int32))
    assert (arg3 == 2).all() and (out3[:, 1] == 2).all()
    # mean only
    out4, _ = oracle.AccumulateLinKnn(w, x, idx, mean_and_max=False)
    assert out4.shape == (3, 2) and np.allclose(out4, out[:, :2])


@pytest.mark.parametrize("F", [3, 32])
def test_accumulate_vs_numpy_composition(oracle, F):
    rng = np.random.default_rng(6)
    n, K = 128, 8
    x = rng.standard_normal((n, F)).astype(np.float32)
    idx = np.stack([rng.permutation(n)[:K] for _ in range(n)]).astype(np.int32)
    idx[:, 0] = np.arange(n)
    idx[10:30, 5:] = -1           # -1 tail
    idx[40, 0] = -1               # slot 0 missing
    idx[50, 3:] = 50              # duplicated-self padding
    d = rng.random((n, K), dtype=np.float32)
    for mm in (True, False):
        out, arg = oracle.AccumulateKnn(d, x, idx, mean_and_max=mm)
        w = np.exp(-d).astype(np.float32)
        ref, rarg = np_accumulate(w, x, idx, mm)
        assert (out.view(np.int32) == ref.view(np.int32)).all()
        if mm:
            assert (arg == rarg).all()


# ------------------------------------------------------------------ accumulate gradient

def test_accumulate_grad_vs_autograd(oracle):
    import torch
    rng = np.random.default_rng(7)
    n, K, F = 96, 8, 5
    x = rng.standard_normal((n, F)).astype(np.float32)
    # unique neighbours per row (self only in slot 0), as the op's contract asks
    idx = np.stack([np.concatenate([[v], rng.permutation(np.delete(np.arange(n), v))[:K - 1]])
                    for v in range(n)]).astype(np.int32)
    idx[5:20, 6:] = -1
    w = (rng.random((n, K)) + 0.1).astype(np.float32)
    g = rng.standard_normal((n, 2 * F)).astype(np.float32)
    out, arg = oracle.AccumulateLinKnn(w, x, idx)
    gw, gx = oracle.accumulate_knn_grad_kernel(g, w, x, idx, arg)

    tw = torch.tensor(w, dtype=torch.float64, requires_grad=True)
    tx = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    tidx = torch.tensor(idx, dtype=torch.int64)
    valid = (tidx >= 0)
    gath = tx[tidx.clamp(min=0)] * tw[:, :, None]
    gath_mean = torch.where(valid[:, :, None], gath, torch.zeros_like(gath))
    mean = gath_mean.sum(1) / K
    gath_max = torch.where(valid[:, :, None], gath, torch.full_like(gath, -1e30))
    mx = gath_max.max(1).values
    assert np.allclose(torch.cat([mean, mx], 1).detach().numpy(), out, rtol=1e-5, atol=1e-6)
    (torch.cat([mean, mx], 1) * torch.tensor(g, dtype=torch.float64)).sum().backward()
    assert np.allclose(gw, tw.grad.numpy(), rtol=1e-5, atol=1e-5)
    assert np.allclose(gx, tx.grad.numpy(), rtol=1e-5, atol=1e-5)
    # mean-only mode is detected from the gradient width
    gw1, gx1 = oracle.accumulate_knn_grad_kernel(g[:, :F], w, x, idx, arg)
    tw.grad = None
    tx.grad = None
    gath = tx[tidx.clamp(min=0)] * tw[:, :, None]
    mean = torch.where(valid[:, :, None], gath, torch.zeros_like(gath)).sum(1) / K
    (mean * torch.tensor(g[:, :F], dtype=torch.float64)).sum().backward()
    assert np.allclose(gw1, tw.grad.numpy(), rtol=1e-5, atol=1e-5)
    assert np.allclose(gx1, tx.grad.numpy(), rtol=1e-5, atol=1e-5)


def test_accumulate_knn_grad_chain_through_exp_vs_autograd(oracle):
    """oracle.AccumulateKnnGrad (the wrapper's gradient w.r.t. the DISTANCES, chained through
    w = exp(-d) as TF autodiff does, modules/accknn_op.py:52,71-89) against float64 autograd of
    the whole composition exp -> gather -> mean|max; a missing minus sign, a missing factor w or a
    gradient taken w.r.t. w instead of d each change the result by O(1)."""
    import torch
    rng = np.random.default_rng(17)
    n, K, F = 80, 7, 4
    x = rng.standard_normal((n, F)).astype(np.float32)
    idx = np.stack([np.concatenate([[v], rng.permutation(np.delete(np.arange(n), v))[:K - 1]])
                    for v in range(n)]).astype(np.int32)
    idx[5:20, 5:] = -1
    d = (rng.random((n, K)) * 2.0).astype(np.float32)
    g = rng.standard_normal((n, 2 * F)).astype(np.float32)
    out, arg = oracle.AccumulateKnn(d, x, idx)
    gd, gx = oracle.AccumulateKnnGrad(g, d, x, idx, arg)

    td = torch.tensor(d, dtype=torch.float64, requires_grad=True)
    tx = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    tidx = torch.tensor(idx, dtype=torch.int64)
    valid = (tidx >= 0)[:, :, None]
    gath = tx[tidx.clamp(min=0)] * torch.exp(-td)[:, :, None]
    mean = torch.where(valid, gath, torch.zeros_like(gath)).sum(1) / K
    mx = torch.where(valid, gath, torch.full_like(gath, -1e30)).max(1).values
    comp = torch.cat([mean, mx], 1)
    assert np.allclose(comp.detach().numpy(), out, rtol=1e-5, atol=1e-6)
    (comp * torch.tensor(g, dtype=torch.float64)).sum().backward()
    assert np.allclose(gd, td.grad.numpy(), rtol=1e-5, atol=1e-6)
    assert np.allclose(gx, tx.grad.numpy(), rtol=1e-5, atol=1e-5)
    assert np.abs(td.grad.numpy()).max() > 0.1            # the comparison is not vacuous
    # linear=True hands the weights through untouched: gradient w.r.t. the weights themselves
    gw_lin, _ = oracle.AccumulateKnnGrad(g, np.exp(-d).astype(np.float32), x, idx, arg, linear=True)
    assert np.allclose(-(np.exp(-d.astype(np.float64)) * gw_lin), td.grad.numpy(), rtol=1e-5, atol=1e-6)


def test_accumulate_grad_summation_order_and_self_rule(oracle):
    """Feature gradient = ordered scatter of ((g/K)*w + max part); the ordered
    unbuffered numpy scatter reproduces the ascending (vertex, slot) order."""
    rng = np.random.default_rng(8)
    n, K, F = 64, 6, 4
    x = rng.standard_normal((n, F)).astype(np.float32)
    idx = np.stack([rng.permutation(n)[:K] for _ in range(n)]).astype(np.int32)
    idx[:, 0] = np.arange(n)
    idx[7, 3:] = 7      # repeated self: max part may be counted once only
    x[7] = 50.0         # make self the arg-max of vertex 7
    idx[9, 4:] = -1
    w = (rng.random((n, K)) + 0.5).astype(np.float32)
    g = rng.standard_normal((n, 2 * F)).astype(np.float32)
    _, arg = oracle.AccumulateLinKnn(w, x, idx)
    assert (arg[7] == 7).all()
    gw, gx = oracle.accumulate_knn_grad_kernel(g, w, x, idx, arg)

    ref = np.zeros((n, F), np.float32)
    gm = (g[:, :F] / np.float32(K)).astype(np.float32)
    for v in range(n):
        first_self = True
        for k in range(K):
            m = idx[v, k]
            if m < 0:
                continue
            add = (gm[v] * w[v, k]).astype(np.float32)
            hit = arg[v] == m
            if m == v:
                hit = hit & first_self
                first_self = False if (arg[v] == m).any() else first_self
            add = (add + np.where(hit, (g[v, F:] * w[v, k]).astype(np.float32), np.float32(0))).astype(np.float32)
            ref[m] = (ref[m] + add).astype(np.float32)
    assert (ref.view(np.int32) == gx.view(np.int32)).all()
    # weight gradient of the repeated-self slots: every slot gets the max part
    j = 7
    want = np.float32(0)
    acc_m = np.float32(0)
    acc_x = np.float32(0)
    for f in range(F):
        acc_m = np.float32(acc_m + np.float32(g[j, f] * x[j, f]))
        acc_x = np.float32(acc_x + np.float32(g[j, F + f] * x[j, f]))
    want = np.float32(np.float32(np.float64(acc_m) * (1.0 / K)) + acc_x)
    assert (gw[7, [0, 3, 4, 5]] == want).all()
    assert (gw[9, 4:] == 0).all()


# ------------------------------------------------------------------ condensates

def stable_bin_positions(oracle, cfg):
    """position of every hit in the wrapper's stable bin order (what breaks ties between equal betas)"""
    cc = cfg["ccoords"].astype(np.float32)
    n = len(cc)
    cc = cc - cc.min(0, keepdims=True)
    n_bins_sc = max(4, min(int(np.ceil((n / 5) ** (1 / 3))), 25))
    _, flat, _, _ = oracle.BinByCoordinates(cc[:, :3], cfg["row_splits"], n_bins=n_bins_sc, calc_n_per_bin=False,
                                            pre_normalized=True)
    pos = np.empty(n, np.int64)
    pos[np.argsort(flat, kind="stable")] = np.arange(n)
    return pos


def bin_free_greedy(oracle, cfg, by_max_beta, mask=None):
    """The reference's loop without bins, written from its text
    (binned_assign_to_condensates_kernel.cc:23-125 claim, :180-226 pick): every pick scans the
    unclaimed high-beta hits in position order; the no_condensation_mask of the high-beta subset
    is indexed with the truth value of (index > 0), and an entry that is set there ends the scan at
    the first unclaimed hit. A masked pick claims only itself; a masked hit is claimed by nobody else."""
    cc = cfg["ccoords"].astype(np.float32)
    beta = cfg["betas"].reshape(-1)
    rad = (cfg["dist"].reshape(-1) / np.float32(cfg["distance_threshold"])).astype(np.float32)
    rs = cfg["row_splits"]
    n = len(beta)
    mask = np.zeros(n, np.int32) if mask is None else np.asarray(mask).reshape(-1).astype(np.int32)
    cc = cc - cc.min(0, keepdims=True)
    pos = stable_bin_positions(oracle, cfg)
    is_high = (beta > np.float32(cfg["beta_threshold"])) | (mask > 0)
    # the filtered arrays: high-beta hits in position order, events one after the other
    filtered = np.concatenate([
        (np.arange(rs[e], rs[e + 1])[is_high[rs[e]:rs[e + 1]]])[np.argsort(pos[rs[e]:rs[e + 1]][is_high[rs[e]:rs[e + 1]]],
                                                                              kind="stable")]
        for e in range(len(rs) - 1)]).astype(np.int64)
    mask_h = mask[filtered]
    assignment = np.full(n, -1, np.int32)
    asso = np.full(n, -1, np.int32)
    alphas, ncond = [], [0]
    q0 = 0
    for e in range(len(rs) - 1):
        lo, hi = rs[e], rs[e + 1]
        mine = filtered[(filtered >= lo) & (filtered < hi)]    # this event's entries, global index q0 + i
        taken = np.zeros(len(mine), bool)
        claimed = np.zeros(n, bool)
        best = np.full(n, np.float32(10e20), np.float32)
        shower = 0
        while True:
            biggest, pick = np.float32(-1), -1
            for i in np.nonzero(~taken)[0]:
                q = q0 + i
                if q < len(mask_h) and (1 if q > 0 else 0) < len(mask_h) and mask_h[1 if q > 0 else 0]:
                    pick, biggest = i, np.float32(0)
                    break
                if beta[mine[i]] > biggest:
                    biggest, pick = beta[mine[i]], i
            if biggest == np.float32(-1):
                break
            a = mine[pick]
            taken[pick] = True
            d = np.zeros(hi - lo, np.float32)
            for c in range(cc.shape[1]):
                t = (cc[a, c] - cc[lo:hi, c]).astype(np.float32)
                d = (d + (t * t).astype(np.float32)).astype(np.float32)
            rsq = np.float32(rad[a] * rad[a])
            if mask[a] > 0:
                inside = np.arange(lo, hi) == a
            else:
                inside = (d <= rsq) & (mask[lo:hi] == 0)
            if by_max_beta:
                claim = inside & (assignment[lo:hi] == -1)
            else:
                claim = inside & ((best[lo:hi] * rsq).astype(np.float32) >= d)
                best[lo:hi] = np.where(claim, d, best[lo:hi])
            assignment[lo:hi] = np.where(claim, shower, assignment[lo:hi])
            asso[lo:hi] = np.where(claim, a, asso[lo:hi])
            claimed[lo:hi] |= claim
            taken |= claimed[mine]
            alphas.append(a)
            shower += 1
        ncond.append(ncond[-1] + shower)
        q0 += len(mine)
    return assignment, asso, np.array(alphas, np.int32), np.array(ncond, np.int32)


# ------------------------------------------------------------------ ops next to the accumulation

def neighbour_case(rng, n, K, with_holes=True):
    idx = np.stack([np.concatenate([[v], rng.permutation(np.delete(np.arange(n), v))[:K - 1]])
                    for v in range(n)]).astype(np.int32)
    if with_holes:
        idx[3:9, K // 2:] = -1
        idx[11, :] = -1
    return idx


def test_select_knn_grad_vs_autograd(oracle):
    """d(sum g_ik |x_i - x_k|^2)/dx by float64 autograd; a wrong sign, a dropped
    self or neighbour term, or a swapped index each change the result by O(1)"""
    import torch
    rng = np.random.default_rng(31)
    n, K, C = 200, 7, 4
    x = rng.standard_normal((n, C)).astype(np.float32)
    idx = neighbour_case(rng, n, K)
    g = rng.standard_normal((n, K)).astype(np.float32)
    got = oracle.select_knn_grad_kernel(g, idx, x)
    tx = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    tidx = torch.tensor(idx, dtype=torch.int64)
    d2 = ((tx[:, None, :] - tx[tidx.clamp(min=0)]) ** 2).sum(2)
    d2 = torch.where(tidx >= 0, d2, torch.zeros_like(d2))
    (d2 * torch.tensor(g, dtype=torch.float64)).sum().backward()
    scale = np.abs(tx.grad.numpy()).max()
    assert np.abs(got - tx.grad.numpy()).max() <= 1e-5 * scale
    # a vertex nobody names and without neighbours gets exactly zero
    lonely = np.setdiff1d(np.arange(n), idx[idx >= 0])
    for v in lonely:
        if (idx[v] < 0).all():
            assert (got[v] == 0).all()
    # out-of-range indices are skipped like -1
    idx2 = idx.copy()
    idx2[20, 2] = n + 5
    idx3 = idx.copy()
    idx3[20, 2] = -1
    assert (oracle.select_knn_grad_kernel(g, idx2, x) == oracle.select_knn_grad_kernel(g, idx3, x)).all()


def test_push_knn_vs_ordered_scatter_and_autograd(oracle):
    import torch
    rng = np.random.default_rng(32)
    n, K, F = 150, 6, 5
    idx = neighbour_case(rng, n, K)
    w = (rng.random((n, K)) + 0.1).astype(np.float32)
    x = rng.standard_normal((n, F)).astype(np.float32)
    out = oracle.PushKnn(w, x, idx)
    # unbuffered scatter-add in ascending (vertex, slot) order: same bits
    ref = np.zeros((n, F), np.float32)
    valid = idx >= 0
    terms = (x[:, None, :] * w[:, :, None]).astype(np.float32)
    np.add.at(ref, idx[valid], terms[valid])
    assert (ref.view(np.int32) == out.view(np.int32)).all()
    # the reference's own slow composition (modules/push_knn_op.py:38-66) in float64
    tw = torch.tensor(w, dtype=torch.float64, requires_grad=True)
    tx = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    tidx = torch.tensor(idx, dtype=torch.int64)
    contrib = tx[:, None, :] * tw[:, :, None]
    contrib = torch.where((tidx >= 0)[:, :, None], contrib, torch.zeros_like(contrib))
    tout = torch.zeros((n, F), dtype=torch.float64).index_add(0, tidx.clamp(min=0).reshape(-1), contrib.reshape(-1, F))
    assert np.allclose(out, tout.detach().numpy(), rtol=1e-5, atol=1e-6)
    g = rng.standard_normal((n, F)).astype(np.float32)
    (tout * torch.tensor(g, dtype=torch.float64)).sum().backward()
    wgrad, fgrad = oracle.push_knn_grad_kernel(g, w, x, idx)
    assert np.allclose(wgrad, tw.grad.numpy(), rtol=1e-5, atol=1e-5)
    assert np.allclose(fgrad, tx.grad.numpy(), rtol=1e-5, atol=1e-5)
    assert (wgrad[idx < 0] == 0).all()


def test_accumulate_sumw_composition(oracle):
    """weighted mean over the accumulated weight: equals sum(w x)/sum(w) per vertex"""
    rng = np.random.default_rng(33)
    n, K, F = 80, 5, 3
    idx = neighbour_case(rng, n, K)
    w = (rng.random((n, K)) + 0.1).astype(np.float32)
    x = rng.standard_normal((n, F)).astype(np.float32)
    for mm in (False, True):
        out, _ = oracle.AccumulateKnnSumw(w, x, idx, mean_and_max=mm, linear=True)
        valid = (idx >= 0)[:, :, None]
        wx = np.where(valid, x[np.maximum(idx, 0)].astype(np.float64) * w[:, :, None], 0.)
        sw = np.where(idx >= 0, w, 0.).astype(np.float64).sum(1, keepdims=True)
        want = np.divide(wx.sum(1), sw, out=np.zeros((n, F)), where=sw != 0)
        assert out.shape == (n, 2 * F if mm else F)
        assert np.allclose(out[:, :F], want, rtol=1e-5, atol=1e-6)
        assert (out[11] == 0).all()   # no neighbours at all: divide_no_nan
        if mm:
            full, _ = oracle.AccumulateLinKnn(w, x, idx)
            assert (out[:, F:] == full[:, F:]).all()


def test_local_distance_vs_brute_force(oracle):
    from helpers import serial_distsq
    rng = np.random.default_rng(34)
    n, K, C = 120, 6, 5
    x = rng.standard_normal((n, C)).astype(np.float32)
    idx = neighbour_case(rng, n, K)
    got = oracle.LocalDistance(x, idx)
    for v in range(n):
        for k in range(K):
            j = idx[v, k]
            want = np.float32(0) if (j < 0 or j == v) else serial_distsq(x[j:j + 1], x[v])[0]
            assert got[v, k].view(np.int32) == np.float32(want).view(np.int32)
    # fewer index rows than coordinates
    assert (oracle.LocalDistance(x, idx[:50]) == got[:50]).all()


def test_neighbour_covariance_vs_float64_formula(oracle):
    rng = np.random.default_rng(35)
    n, K, C, F = 90, 5, 3, 4
    x = rng.standard_normal((n, C)).astype(np.float32)
    feat = rng.standard_normal((n, F)).astype(np.float32)
    idx = neighbour_case(rng, n, K)
    d2 = rng.random((n, K), dtype=np.float32)
    cov, mean_c = oracle.NeighbourCovariance(x, d2, feat, idx)
    assert cov.shape == (n, F, C * C) and mean_c.shape == (n, F, C)
    fs = 1.0 / (1.0 + np.exp(-feat.astype(np.float64))) + 1e-3
    w = np.where(idx >= 0, np.exp(-d2.astype(np.float64)), 0.0)            # [n, K]
    j = np.maximum(idx, 0)
    sum_f = (w[:, :, None] * fs[j]).sum(1)                                  # [n, F]
    sum_fc = (w[:, :, None, None] * fs[j][:, :, :, None] * x.astype(np.float64)[j][:, :, None, :]).sum(1)
    want_mean = sum_fc / (sum_f[:, :, None] + 1e-3)
    assert np.allclose(mean_c, want_mean, rtol=1e-4, atol=1e-6)
    cen = x.astype(np.float64)[:, None, :] - want_mean                     # per vertex, [n, F, C]
    outer = (cen[:, :, :, None] * cen[:, :, None, :]).reshape(n, F, C * C) * fs[:, :, None]
    want_cov = (w[:, :, None, None] * outer[j]).sum(1) / (sum_f[:, :, None] + 1e-3)
    assert np.allclose(cov, want_cov, rtol=1e-4, atol=1e-6)


@pytest.mark.parametrize("by_max_beta", [True, False])
@pytest.mark.parametrize("t_d", [0.5, 0.15])
def test_condensates_vs_bin_free_greedy(oracle, by_max_beta, t_d):
    cfg = workloads.cfg5(scale=0.024, n_events=3)   # 3 x 1500 hits, many 0.999 beta ties
    cfg["dist"] = (cfg["dist"] * 0 + t_d).astype(np.float32)
    # per-hit radii, not just a constant
    rng = np.random.default_rng(9)
    cfg["dist"] = (cfg["dist"] * rng.uniform(0.6, 1.4, size=cfg["dist"].shape)).astype(np.float32)
    b = cfg["betas"].reshape(-1)
    assert (np.bincount((b * 1000).astype(int))[999] > 5)  # clipped ties are present
    assignment, asso, alpha, is_cond, ncond = oracle.BuildAndAssignCondensatesBinned(
        cfg["ccoords"], cfg["betas"], cfg["dist"], cfg["row_splits"], cfg["beta_threshold"],
        assign_by_max_beta=by_max_beta)
    r_assignment, r_asso, r_alpha, r_ncond = bin_free_greedy(oracle, cfg, by_max_beta)
    assert (ncond == r_ncond).all()
    assert (alpha == r_alpha).all()
    assert (assignment[:, 0] == r_assignment).all()
    assert (asso == r_asso).all()
    # invariants of the reference wrapper / tests
    assert (asso[alpha] == alpha).all()
    assert is_cond.sum() == len(alpha) and is_cond[alpha, 0].all()
    rs = cfg["row_splits"]
    per_event_max = np.array([assignment[rs[e]:rs[e + 1]].max() + 1 for e in range(len(rs) - 1)])
    assert (ncond == np.concatenate([[0], np.cumsum(per_event_max)])).all()
    for e in range(len(rs) - 1):
        assert (assignment[alpha[ncond[e]:ncond[e + 1]], 0] == np.arange(ncond[e + 1] - ncond[e])).all()


@pytest.mark.parametrize("by_max_beta", [True, False])
@pytest.mark.parametrize("case", ["sparse", "first", "second", "first two", "dense"])
def test_condensates_with_mask_vs_bin_free_greedy(oracle, by_max_beta, case):
    """no_condensation_mask: sparse and dense random masks, and masks on the first / second entry of
    the high-beta subset, which switch the reference's pick loop to position order (its index
    expression `mask_h[offset + i > 0]`)"""
    cfg = workloads.cfg5(scale=0.016, n_events=3)   # 3 x 1000 hits
    rng = np.random.default_rng(12)
    cfg["dist"] = (0.3 * rng.uniform(0.6, 1.4, size=cfg["dist"].shape)).astype(np.float32)
    n = len(cfg["betas"])
    pos = stable_bin_positions(oracle, cfg)
    high = cfg["betas"].reshape(-1) > np.float32(cfg["beta_threshold"])
    first_two = np.argsort(np.where(high[:cfg["row_splits"][1]], pos[:cfg["row_splits"][1]], n))[:2]
    mask = np.zeros(n, np.int32)
    if case == "sparse":
        mask[rng.random(n) < 0.02] = 1
        mask[first_two] = 0
    elif case == "dense":
        mask[rng.random(n) < 0.4] = 1
    elif case == "first":
        mask[first_two[0]] = 1
    elif case == "second":
        mask[first_two[1]] = 1
    else:
        mask[first_two] = 1
    assignment, asso, alpha, is_cond, ncond = oracle.BuildAndAssignCondensatesBinned(
        cfg["ccoords"], cfg["betas"], cfg["dist"], cfg["row_splits"], cfg["beta_threshold"],
        no_condensation_mask=mask[:, None], assign_by_max_beta=by_max_beta)
    r_assignment, r_asso, r_alpha, r_ncond = bin_free_greedy(oracle, cfg, by_max_beta, mask=mask)
    assert (ncond == r_ncond).all()
    assert (alpha == r_alpha).all()
    assert (assignment[:, 0] == r_assignment).all()
    assert (asso == r_asso).all()
    # a masked hit is its own condensation point
    masked = np.nonzero(mask)[0]
    assert (asso[masked] == masked).all() and is_cond[masked, 0].all()


@pytest.mark.parametrize("t_b", [1e-5, 0.1, 0.9999])
def test_condensates_degenerate_coordinates_and_thresholds(oracle, t_b):
    """4x3 grid x 2 events and all-zero coordinates (the structural cases of the
    reference's tests/unit/condensate.py:40-128)."""
    rng = np.random.default_rng(10)
    gx, gy = np.meshgrid(np.linspace(0, 10, 4), np.linspace(0, 10, 3))
    x = np.concatenate([np.stack([gx, gy], -1).reshape(-1, 2)] * 2).astype(np.float32)
    beta = rng.random((24, 1)).astype(np.float32)
    rs = np.array([0, 12, 24], np.int32)
    for coords in (x, 0 * x):
        a, asso, alpha, is_cond, ncond = oracle.BuildAndAssignCondensatesBinned(
            coords, beta, np.ones_like(beta), rs, t_b, assign_by_max_beta=False)
        high = beta[:, 0] > np.float32(t_b)
        if coords.any():
            # grid spacing 3.33 / 5 > radius 1: every high-beta hit is its own condensate
            assert set(alpha.tolist()) == set(np.nonzero(high)[0].tolist())
            assert (asso[high] == np.nonzero(high)[0]).all() and (asso[~high] == -1).all()
        else:
            # everything on one spot: one condensate per event that has any high-beta hit
            for e in range(2):
                h = np.nonzero(high[rs[e]:rs[e + 1]])[0] + rs[e]
                n_e = ncond[e + 1] - ncond[e]
                assert n_e == (1 if len(h) else 0)
                if len(h):
                    top = h[np.argmax(beta[h, 0])]
                    assert (asso[rs[e]:rs[e + 1]] == top).all()
        assert (a[alpha, 0] >= 0).all()


# ------------------------------------------------------------------ condensates: hand-computed cases

from condensate_cases import CASES as HAND_CASES  # noqa: E402


@pytest.mark.parametrize("case", HAND_CASES, ids=[c["name"] for c in HAND_CASES])
def test_condensates_hand_computed(oracle, case):
    """literal expectations (tests/condensate_cases.py): the min-distance claim rule
    `best * r^2 >= d^2` where a plain arg-min, "the first coverer keeps it" and the reference all
    differ, per-hit radii, a claimed high-beta hit that changes hands, and the pick loop's mask
    indexing with entry 0 / entry 1 / a later entry set, in one and in two events"""
    a, s, alpha, is_cond, ncond = oracle.BuildAndAssignCondensatesBinned(
        case["ccoords"], case["betas"], case["dist"], case["row_splits"], case["beta_threshold"],
        no_condensation_mask=case["mask"], assign_by_max_beta=case["assign_by_max_beta"])
    assert a[:, 0].tolist() == case["assignment"].tolist()
    assert s.tolist() == case["asso"].tolist()
    assert alpha.tolist() == case["alpha"].tolist()
    assert ncond.tolist() == case["ncond"].tolist()
    want_cond = np.zeros(len(s), bool)
    want_cond[case["alpha"]] = True
    assert is_cond[:, 0].tolist() == want_cond.tolist()


# ------------------------------------------------------------------ keep_noise post-pass

def merge_noise_per_event_loop(assignment, asso, alpha, is_cond, ncond, rs):
    """modules/assign_condensate_op.py:16-44 event by event with plain lists: noise hit number j of an
    event (ascending hit index) becomes shower j, the event's real showers move up by its noise count,
    its list of condensation points is its noise hits followed by its original points, every noise hit
    is its own condensation point and association target, and the counts are recounted"""
    new_a, new_alpha, new_n = [], [], [int(ncond[0])]
    new_asso, new_cond = list(asso), [bool(c) for c in is_cond[:, 0]]
    for e in range(len(rs) - 1):
        hits = range(rs[e], rs[e + 1])
        noise_hits = [i for i in hits if assignment[i, 0] < 0]
        seen = 0
        for i in hits:
            if assignment[i, 0] < 0:
                new_a.append(seen)
                seen += 1
                new_asso[i] = i
                new_cond[i] = True
            else:
                new_a.append(int(assignment[i, 0]) + len(noise_hits))
        new_alpha += noise_hits + [int(v) for v in alpha[ncond[e]:ncond[e + 1]]]
        new_n.append(new_n[-1] + sum(new_cond[i] for i in hits))
    return new_a, new_asso, new_alpha, new_cond, new_n


def test_keep_noise_vs_per_event_loop(oracle):
    rng = np.random.default_rng(61)
    # three events: mixed, without any noise, all noise
    rs = np.array([0, 9, 14, 20], np.int32)
    assignment = np.array([1, -1, 0, -1, -1, 2, 0, 1, -1,   0, 1, 1, 0, 2,   -1, -1, -1, -1, -1, -1], np.int32)[:, None]
    ncond = np.array([0, 3, 6, 6], np.int32)
    alpha = np.array([2, 0, 5,   9, 10, 13], np.int32)          # shower s of event e is led by alpha[ncond[e] + s]
    asso = np.full(20, -1, np.int32)
    for e in range(3):
        for i in range(rs[e], rs[e + 1]):
            if assignment[i, 0] >= 0:
                asso[i] = alpha[ncond[e] + assignment[i, 0]]
    is_cond = np.zeros((20, 1), bool)
    is_cond[alpha, 0] = True
    got = oracle.merge_noise_as_indiv_cp(assignment, asso, alpha, is_cond, ncond, rs)
    want = merge_noise_per_event_loop(assignment, asso, alpha, is_cond, ncond, rs)
    assert got[0][:, 0].tolist() == want[0]
    assert got[1].tolist() == want[1]
    assert got[2].tolist() == want[2]
    assert got[3][:, 0].tolist() == want[3]
    assert got[4].tolist() == want[4]
    # spelled out for the first event: noise hits 1, 3, 4, 8 -> showers 0..3, real showers 0, 1, 2 -> 4, 5, 6
    assert got[0][:9, 0].tolist() == [5, 0, 4, 1, 2, 6, 4, 5, 3]
    assert got[2][:7].tolist() == [1, 3, 4, 8, 2, 0, 5]
    assert got[4].tolist() == [0, 7, 10, 16]
    assert got[1][:9].tolist() == [0, 1, 2, 3, 4, 5, 2, 0, 8]
    # random events through the whole wrapper
    cfg = workloads.cfg5(scale=0.004, n_events=3)
    args = (cfg["ccoords"], cfg["betas"], cfg["dist"], cfg["row_splits"], 0.4)
    plain = oracle.BuildAndAssignCondensatesBinned(*args, assign_by_max_beta=True)
    kept = oracle.BuildAndAssignCondensatesBinned(*args, assign_by_max_beta=True, keep_noise=True)
    want = merge_noise_per_event_loop(*plain, cfg["row_splits"])
    assert (plain[0] < 0).any()
    assert kept[0][:, 0].tolist() == want[0] and kept[1].tolist() == want[1] and kept[2].tolist() == want[2]
    assert kept[3][:, 0].tolist() == want[3] and kept[4].tolist() == want[4]
    del rng
