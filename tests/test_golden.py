"""The committed vectors under tests/golden/ (written by tests/golden/make_fixtures.py).

CPU: the oracle still reproduces every stored array bit for bit (a change of the oracle shows up here).
GPU: the HIP path, through the C ABI and the wrappers, reproduces the stored outputs from the stored inputs.
"""
import importlib.util
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    with np.load(os.path.join(GOLDEN, name + ".npz"), allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def same(a, b):
    a, b = np.asarray(a), np.asarray(b)
    if a.shape != b.shape or a.dtype != b.dtype:
        return False
    if a.dtype.kind == "f":
        return bool((a.view(np.int32) == b.view(np.int32)).all())
    return bool((a == b).all())


def test_oracle_reproduces_the_fixtures(oracle):
    spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(GOLDEN, "make_fixtures.py"))
    mk = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mk)
    for name, fn in mk.FIXTURES.items():
        stored, fresh = load(name), fn()
        assert sorted(stored) == sorted(fresh), name
        for k in stored:
            assert same(stored[k], fresh[k]), (name, k)


# ------------------------------------------------------------------ GPU

@pytest.fixture
def hip_ops():
    from hgcalml_amd import ops  # registers torch.ops.hgcalml.*
    return ops


def t(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")


@pytest.mark.gpu
def test_gpu_binning_fixture(hip_ops):
    import torch
    g = load("g1_binning")
    total = int(np.prod(g["n_bins"])) * (len(g["row_splits"]) - 1)
    binass, flat, nper = torch.ops.hgcalml.bin_by_coordinates(t(g["coords"]), t(g["row_splits"]), t(g["bin_width"]),
                                                              t(g["n_bins"]), total, True)
    assert same(binass.cpu().numpy(), g["binass"]) and same(flat.cpu().numpy(), g["flat"])
    assert same(nper.cpu().numpy(), g["nper"])


@pytest.mark.gpu
def test_gpu_knn_fixture(hip_ops):
    from hgcalml_amd import BinnedSelectKnn
    g = load("g2_knn")
    co, rs = t(g["coords"]), t(g["row_splits"])
    for K in (4, 16, 64):
        idx, dist = BinnedSelectKnn(K, co, rs, n_bins=5)
        assert same(idx.cpu().numpy(), g["idx_K%d" % K]) and same(dist.detach().cpu().numpy(), g["dist_K%d" % K])
    idx, dist = BinnedSelectKnn(16, co, rs, direction=t(g["direction"]), n_bins=5)
    assert same(idx.cpu().numpy(), g["idx_dir"]) and same(dist.cpu().numpy(), g["dist_dir"])
    idx, dist = BinnedSelectKnn(16, co, rs, n_bins=5, tf_compatible=True)
    assert same(idx.cpu().numpy(), g["idx_tfc"]) and same(dist.cpu().numpy(), g["dist_tfc"])
    idx, dist = BinnedSelectKnn(16, co, t(g["row_splits_small"]), n_bins=5)
    assert same(idx.cpu().numpy(), g["idx_small"]) and same(dist.cpu().numpy(), g["dist_small"])


@pytest.mark.gpu
@pytest.mark.parametrize("F", [3, 32])
def test_gpu_accumulate_fixture(hip_ops, F):
    import torch
    ops = hip_ops
    g = {k[len("F%d_" % F):]: v for k, v in load("g3_accumulate").items() if k.startswith("F%d_" % F)}
    w, x, idx, grad = t(g["w"]), t(g["x"]), t(g["idx"]), t(g["g"])
    out, arg = torch.ops.hgcalml.accumulate_knn(w, x, idx, 0, True)
    assert same(out.cpu().numpy(), g["out"]) and same(arg.cpu().numpy(), g["arg"])
    out1, _ = torch.ops.hgcalml.accumulate_knn(w, x, idx, 0, False)
    assert same(out1.cpu().numpy(), g["out_mean"])
    inv = ops.inverse_neighbour_index(idx)
    K = idx.shape[1]
    for gr, want_w, want_x in ((grad, g["gw"], g["gx"]), (grad[:, :F].contiguous(), g["gw_mean"], g["gx_mean"])):
        gw, gx = torch.ops.hgcalml.accumulate_knn_grad(gr, w, x, idx, arg, *inv)
        assert same(gx.cpu().numpy(), want_x)
        # weight gradient: tree reduction over the features, 1e-5 relative to the sum of |terms|
        gm = np.abs(g["g"][:, :F]) / K + (np.abs(g["g"][:, F:]) if gr.shape[1] > F else 0)
        scale = (np.abs(g["x"][np.maximum(g["idx"], 0)]) * gm[:, None, :]).sum(-1)
        assert (np.abs(gw.cpu().numpy() - want_w) <= 1e-5 * scale + 1e-30).all()


@pytest.mark.gpu
def test_gpu_condensate_fixture(hip_ops):
    from hgcalml_amd import BuildAndAssignCondensatesBinned
    g = load("g5_condensates")
    args = [t(g[k]) for k in ("ccoords", "betas", "dist", "row_splits")]
    names = ("assignment", "asso", "alpha", "is_cond", "ncond")
    for mode in (True, False):
        for t_b in (1e-5, 0.1, 0.9999):
            got = BuildAndAssignCondensatesBinned(*args, t_b, assign_by_max_beta=mode)
            for name, v in zip(names, got):
                want = g["%s_%s_tb%g" % (name, "maxbeta" if mode else "mindist", t_b)]
                assert (v.cpu().numpy() == want).all(), (name, mode, t_b)
    got = BuildAndAssignCondensatesBinned(t(np.zeros_like(g["ccoords"])), *args[1:], 0.1, assign_by_max_beta=True)
    for name, v in zip(names, got):
        assert (v.cpu().numpy() == g["%s_degenerate" % name]).all(), name


@pytest.mark.gpu
def test_gpu_small_ops_fixture(hip_ops):
    import torch
    g = load("g6_small_ops")
    assert same(torch.ops.hgcalml.index_replacer(t(g["tbr"]), t(g["rep"])).cpu().numpy(), g["replaced"])
    gc = torch.ops.hgcalml.select_knn_grad(t(g["grad_dist"]), t(g["idx"]), t(np.zeros_like(g["grad_dist"])), t(g["coords"]))
    assert same(gc.cpu().numpy(), g["grad_coords"])
    pushed = torch.ops.hgcalml.push_knn(t(g["w"]), t(g["feat"]), t(g["idx"]))
    assert same(pushed.cpu().numpy(), g["pushed"])
    wgrad, fgrad = torch.ops.hgcalml.push_knn_grad(t(g["grad_pushed"]), t(g["w"]), t(g["feat"]), t(g["idx"]))
    assert same(fgrad.cpu().numpy(), g["push_fgrad"])
    scale = (np.abs(g["grad_pushed"][np.maximum(g["idx"], 0)]) * np.abs(g["feat"])[:, None, :]).sum(-1)
    assert (np.abs(wgrad.cpu().numpy() - g["push_wgrad"]) <= 1e-5 * scale + 1e-30).all()
