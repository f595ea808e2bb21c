"""Seeded sweep over random shapes and option combinations: every op of the path
on the GPU against the oracle (kNN options incl. radius x tf_compatible x
direction, ragged events, lattice ties; accumulate forward / gradient / PushKnn /
distance gradient over the resulting tables; condensates with per-hit radii)."""
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
                             PushKnn, ops, workloads)
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
        assert (gi == ri).all() and (bits(gd) == bits(rd)).all()

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
            gw, gx = torch.ops.hgcalml.accumulate_knn_grad_slots(t(gg), t(w), t(x), idx, arg, slots, *inv)
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
