"""Seeded sweep over random shapes and option combinations: every op of the path
on the GPU against the oracle (kNN options incl. radius x tf_compatible x
direction, ragged events, lattice ties; accumulate forward / gradient / PushKnn /
distance gradient over the resulting tables; condensates with per-hit radii, masks,
ties and 1-9 coordinates)."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def t(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def bits(a):
    return np.ascontiguousarray(a).view(np.int32)


@pytest.mark.parametrize("seed", range(24))
def test_random_configuration(oracle, seed):
    from hgcalml_amd import (AccumulateLinKnn, BinnedSelectKnn, BuildAndAssignCondensatesBinned, LocalDistance,
                             PushKnn, ops)
    import workloads
    rng = np.random.default_rng(1000 + seed)
    n = int(rng.integers(50, 5000))
    C = int(rng.integers(2, 7))
    B = int(min(C, rng.integers(2, 5)))
    K = int(rng.choice([1, 2, 5, 16, 33, 64, 65, 100]))
    n_ev = int(rng.integers(1, 5))
    rs = np.concatenate([[0], np.sort(rng.integers(0, n + 1, n_ev - 1)), [n]]).astype(np.int32)
    kind = int(rng.integers(0, 3))
    coords = (rng.random((n, C), dtype=np.float32) if kind == 0 else
              rng.standard_normal((n, C)).astype(np.float32) if kind == 1 else
              rng.integers(0, 6, (n, C)).astype(np.float32))       # lattice: many exact distance ties
    nb = int(rng.integers(3, 20))
    radius = None if rng.random() < 0.6 else float(rng.random() * 0.5 + 0.05)
    direction = None if rng.random() < 0.7 else rng.integers(0, 5, n).astype(np.int32)
    tfc = bool(rng.random() < 0.3)
    idx, dist = BinnedSelectKnn(K, t(coords), t(rs), direction=None if direction is None else t(direction),
                                n_bins=nb, max_bin_dims=B, tf_compatible=tfc, max_radius=radius)
    ri, rd = oracle.canonical_knn(*oracle.BinnedSelectKnn(K, coords, rs, direction=direction, n_bins=nb,
                                                          max_bin_dims=B, tf_compatible=tfc, max_radius=radius))
    gi, gd = idx.cpu().numpy(), dist.cpu().numpy()
    if kind == 2:
        # which member of an exactly tied K-th group survives is open; the distances are not
        assert (np.sort(bits(gd), 1) == np.sort(bits(rd), 1)).all()
    else:
        # random floats: rows may differ from the oracle's only where the K-th boundary is an exact tie
        # (which member of the tied group survives is open), and such a row is still a valid kNN set
        differ = np.nonzero((gi != ri).any(1) | (bits(gd) != bits(rd)).any(1))[0]
        assert len(differ) <= max(2, n // 500), differ[:10]
        if len(differ):
            from helpers import check_knn_rows
            assert check_knn_rows(oracle, gi, gd, coords, rs, K, differ, direction=direction, tf_compatible=tfc,
                                  radius=radius) == len(differ)

    if kind != 2 and K >= 2:      # the accumulation needs rows of distinct neighbours
        F = int(rng.choice([3, 8, 32, 64, 96, 128, 192, 256]))
        x = rng.standard_normal((n, F)).astype(np.float32)
        w = np.exp(-10 * gd).astype(np.float32)
        g = rng.standard_normal((n, 2 * F)).astype(np.float32)
        inv = ops.inverse_neighbour_index(idx)
        for mm in (True, False):
            ro, ra = oracle.AccumulateLinKnn(w, x, gi, mm)
            out, arg, slots = torch.ops.hgcalml.accumulate_knn_slots(t(w), t(x), idx, 0, mm)
            assert (bits(out.cpu().numpy()) == bits(ro)).all()
            if mm:
                assert (arg.cpu().numpy() == ra).all()
            gg = g if mm else g[:, :F].copy()
            rgw, rgx = oracle.accumulate_knn_grad_kernel(gg, w, x, gi, ra)
            # the gather fed by per-slot hit records in half of the configurations (it applies up to 128 features)
            import hgcalml_amd.globals as gl
            gl.acc_grad_hit_records = bool(seed % 2)
            try:
                gw, gx = torch.ops.hgcalml.accumulate_knn_grad_slots(t(gg), t(w), t(x), idx, arg, slots, *inv)
            finally:
                gl.acc_grad_hit_records = None
            assert (bits(gx.cpu().numpy()) == bits(rgx)).all()
            gm = np.abs(gg[:, :F]) / K + (np.abs(gg[:, F:]) if mm else 0)
            scale = (np.abs(x[np.maximum(gi, 0)]) * gm[:, None, :]).sum(-1)
            assert (np.abs(gw.cpu().numpy() - rgw) <= 1e-5 * scale + 1e-30).all()
        assert (bits(PushKnn(t(w), t(x), idx).cpu().numpy()) == bits(oracle.PushKnn(w, x, gi))).all()
        gdist = rng.standard_normal((n, K)).astype(np.float32)
        got = torch.ops.hgcalml.select_knn_grad(t(gdist), idx, dist, t(coords))
        assert (bits(got.cpu().numpy()) == bits(oracle.select_knn_grad_kernel(gdist, gi, coords))).all()
        assert (bits(LocalDistance(t(coords), idx).cpu().numpy()) == bits(oracle.LocalDistance(coords, gi))).all()

    c5 = workloads.cfg5(scale=float(rng.random() * 0.03 + 0.002), seed=2000 + seed, n_events=int(rng.integers(1, 4)))
    tb = float(rng.choice([1e-5, 0.05, 0.3, 0.9]))
    mode = bool(rng.integers(0, 2))
    radii = (c5["dist"] * (rng.random(c5["dist"].shape, dtype=np.float32) + 0.5)).astype(np.float32)
    got = BuildAndAssignCondensatesBinned(t(c5["ccoords"]), t(c5["betas"]), t(radii), t(c5["row_splits"]), tb,
                                          assign_by_max_beta=mode)
    ref = oracle.BuildAndAssignCondensatesBinned(c5["ccoords"], c5["betas"], radii, c5["row_splits"], tb,
                                                 assign_by_max_beta=mode)
    for a, b in zip(got, ref):
        assert (a.cpu().numpy() == b).all()


@pytest.mark.parametrize("seed", range(12))
def test_random_knn_long_lists_and_dense_blobs(oracle, seed):
    """neighbour lists of several runs of 64 (K > 65) and points crowded into a
    few bins; rows that differ from the oracle must be exact ties at the K-th
    boundary (a dense blob produces a few)"""
    from helpers import check_knn_rows
    from hgcalml_amd import BinnedSelectKnn
    rng = np.random.default_rng(3000 + seed)
    n = int(rng.integers(400, 7000))
    C = int(rng.integers(2, 6))
    K = int(rng.choice([66, 129, 130, 200, 300]))
    n_ev = int(rng.integers(1, 3))
    rs = np.concatenate([[0], np.sort(rng.integers(0, n + 1, n_ev - 1)), [n]]).astype(np.int32)
    kind = int(rng.integers(0, 3))
    coords = (rng.random((n, C), dtype=np.float32) if kind == 0 else
              rng.standard_normal((n, C)).astype(np.float32) if kind == 1 else
              np.concatenate([0.5 + 0.01 * rng.standard_normal((n - n // 5, C)),
                              rng.random((n // 5, C))]).astype(np.float32)[rng.permutation(n)])
    nb = int(rng.integers(3, 16))
    radius = None if rng.random() < 0.7 else float(rng.random() * 0.5 + 0.05)
    idx, dist = BinnedSelectKnn(K, t(coords), t(rs), n_bins=nb, max_radius=radius)
    ri, rd = oracle.canonical_knn(*oracle.BinnedSelectKnn(K, coords, rs, n_bins=nb, max_radius=radius))
    gi, gd = idx.cpu().numpy(), dist.cpu().numpy()
    differ = np.nonzero((gi != ri).any(1) | (bits(gd) != bits(rd)).any(1))[0]
    kw = {} if radius is None else {"radius": radius}
    assert check_knn_rows(oracle, gi, gd, coords, rs, K, differ, **kw) == len(differ)
    assert len(differ) <= n // 100


@pytest.mark.parametrize("seed", range(40))
def test_random_condensates(oracle, seed):
    """condensate assignment over random sizes, 1-9 coordinates, 1-4 binned dimensions, uniform /
    normal / lattice / clustered hits, beta with ties, radii from tiny to half the extent (per hit
    or common), distance thresholds, sparse to full no_condensation_mask, both assignment modes"""
    from hgcalml_amd import BuildAndAssignCondensatesBinned
    rng = np.random.default_rng(5000 + seed)
    n = int(rng.choice([rng.integers(1, 60), rng.integers(60, 3000), rng.integers(3000, 40000)]))
    C = int(rng.integers(1, 10))
    nbin_dims = int(rng.integers(1, 5))
    n_ev = int(rng.integers(1, 6))
    rs = np.concatenate([[0], np.sort(rng.integers(0, n + 1, n_ev - 1)), [n]]).astype(np.int32)
    kind = int(rng.integers(0, 4))
    if kind == 0:
        x = rng.random((n, C), dtype=np.float32)
    elif kind == 1:
        x = rng.standard_normal((n, C)).astype(np.float32)
    elif kind == 2:
        x = rng.integers(0, 4, (n, C)).astype(np.float32)  # distance ties, coincident hits
    else:
        k = max(1, n // 50)
        centres = rng.random((k, C)) * 2 - 1
        x = (centres[rng.integers(0, k, n)] + 0.03 * rng.standard_normal((n, C))).astype(np.float32)
    beta_kind = int(rng.integers(0, 3))
    if beta_kind == 0:
        beta = rng.random((n, 1), dtype=np.float32)
    elif beta_kind == 1:
        beta = (rng.integers(0, 8, (n, 1)) / 8).astype(np.float32)
    else:
        beta = np.clip(rng.beta(0.5, 2, (n, 1)) + 0.5 * (rng.random((n, 1)) < 0.3), 0, 0.999).astype(np.float32)
    # radii relative to the extent: the reference's box walk counts its cells in an int
    extent = max(1e-3, float((x.max(0) - x.min(0)).max()))
    scale = float(rng.choice([0.001, 0.02, 0.1, 0.2, 0.3, 0.5])) * extent
    dist = (scale * (0.5 + rng.random((n, 1)))).astype(np.float32)
    if rng.random() < 0.3:
        dist[:] = scale
    threshold = float(rng.choice([0.5, 1.0, 0.7, 2.0]))
    t_b = float(rng.choice([0.0, 1e-5, 0.1, 0.5, 0.95]))
    mask = None
    if rng.random() < 0.5:
        mask = (rng.random((n, 1)) < float(rng.choice([0.001, 0.02, 0.3, 1.0]))).astype(np.int32)
    kw = dict(distance_threshold=threshold, assign_by_max_beta=bool(rng.integers(0, 2)), nbin_dims=nbin_dims)
    ref = oracle.BuildAndAssignCondensatesBinned(x, beta, dist, rs, t_b, no_condensation_mask=mask, **kw)
    got = BuildAndAssignCondensatesBinned(t(x), t(beta), t(dist), t(rs), t_b,
                                          no_condensation_mask=None if mask is None else t(mask), **kw)
    for name, a, b in zip(("assignment", "association", "alpha_idx", "is_cond", "n_condensates"), got, ref):
        a = a.cpu().numpy()
        assert a.shape == b.shape, name
        assert (a == b).all(), name
