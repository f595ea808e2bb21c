"""Bad DATA (as opposed to bad arguments): the kernels keep the reference's fallbacks and report
through a device status word; the wrappers act on it while hgcalml_amd.globals.debug_checks is set.
Reference reactions: modules/compiled/bin_by_coordinates_kernel.cc:75-78,
binned_select_knn_kernel.cc:146-149, index_replacer_kernel.cc:35-38 (print and continue),
modules/bin_by_coordinates_op.py:46 (check_numerics raises),
modules/assign_condensate_op.py:334-343 (count relation)."""
import warnings

import numpy as np
import pytest
import torch


# ------------------------------------------------------------------ host side (no GPU)

def test_flag_values_match_the_header():
    import os
    import re
    from hgcalml_amd import ops
    header = open(os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include",
                               "hgcalml_amd.h")).read()
    flags = dict(re.findall(r"HGC_FLAG_(\w+) = (\d+)", header))
    assert {k: int(v) for k, v in flags.items()} == {
        "COORDINATE_OUT_OF_GRID": ops.FLAG_COORDINATE_OUT_OF_GRID,
        "COORDINATE_NOT_FINITE": ops.FLAG_COORDINATE_NOT_FINITE,
        "BIN_BEYOND_TABLE": ops.FLAG_BIN_BEYOND_TABLE,
        "REPLACEMENT_OUT_OF_RANGE": ops.FLAG_REPLACEMENT_OUT_OF_RANGE,
        "SHELL_TOO_WIDE": ops.FLAG_SHELL_TOO_WIDE}


def test_reactions_to_flags():
    from hgcalml_amd import ops
    with warnings.catch_warnings():
        warnings.simplefilter("error")
        ops.report_data_flags(0, "op")                     # nothing met: silent
    with pytest.raises(ValueError, match="NaN or Inf"):
        ops.report_data_flags(ops.FLAG_COORDINATE_NOT_FINITE | ops.FLAG_COORDINATE_OUT_OF_GRID, "op")
    for flag, text in ((ops.FLAG_COORDINATE_OUT_OF_GRID, "bin 0"), (ops.FLAG_BIN_BEYOND_TABLE, "bin boundaries"),
                       (ops.FLAG_REPLACEMENT_OUT_OF_RANGE, "replacements"), (ops.FLAG_SHELL_TOO_WIDE, "too fine")):
        with pytest.warns(ops.DataWarning, match=text):
            ops.report_data_flags(flag, "op")


def test_condensate_count_relation_on_host_tensors():
    from hgcalml_amd.assign_condensate_op import check_condensate_counts
    a = torch.tensor([0, 1, -1, 1, -1, -1, -1, 2, 0, 1], dtype=torch.int32)[:, None]
    rs = torch.tensor([0, 4, 4, 7, 10], dtype=torch.int32)     # with an empty event and one of noise only
    check_condensate_counts(a, torch.tensor([0, 2, 2, 2, 5], dtype=torch.int32), rs)
    with pytest.raises(RuntimeError, match="does not match"):
        check_condensate_counts(a, torch.tensor([0, 2, 2, 3, 5], dtype=torch.int32), rs)


def test_status_word_off_means_no_call_and_no_sync(monkeypatch):
    from hgcalml_amd import globals as gl
    from hgcalml_amd import ops
    calls = []
    monkeypatch.setattr(ops.lib, "hgc_set_status_word", lambda *a: calls.append(a) or 0)
    assert gl.debug_checks is False
    with ops.data_checks("op", "cpu"):
        pass
    assert calls == []


# ------------------------------------------------------------------ on the GPU: one case per flag

DEV = "cuda:0"


@pytest.fixture
def debug_checks():
    from hgcalml_amd import globals as gl
    gl.debug_checks = True
    yield
    gl.debug_checks = False


def _status_after(call):
    """flags a raw library call leaves in a fresh status word"""
    from hgcalml_amd._lib import check, lib, p
    word = torch.zeros(1, dtype=torch.int32, device=DEV)
    check(lib.hgc_set_status_word(p(word)))
    try:
        call()
    finally:
        check(lib.hgc_set_status_word(None))
    torch.cuda.synchronize()
    return int(word.item())


@pytest.mark.gpu
def test_out_of_grid_coordinate_is_flagged_and_lands_in_bin_0(oracle, debug_checks):
    from hgcalml_amd import ops
    x = np.array([[0.1, 0.1], [0.9, 0.5], [7.0, 0.2], [0.3, -4.0]], np.float32)   # two points outside a 2 x 2 grid
    rs = np.array([0, 4], np.int32)
    bw, nb = np.array([0.5], np.float32), np.array([2, 2], np.int32)
    with pytest.warns(ops.DataWarning, match="bin 0"):
        binass, flat, _ = torch.ops.hgcalml.bin_by_coordinates(torch.from_numpy(x).to(DEV), torch.from_numpy(rs).to(DEV),
                                                               torch.from_numpy(bw).to(DEV), torch.from_numpy(nb).to(DEV),
                                                               4, True)
    ref_binass, ref_flat, _, bad = oracle.bin_by_coordinates_kernel(x, rs, bw, nb)
    assert bad == 2 and (binass.cpu().numpy() == ref_binass).all() and (flat.cpu().numpy() == ref_flat).all()
    assert binass.cpu().tolist() == [[0, 0, 0], [0, 1, 1], [0, 0, 0], [0, 0, 0]]


@pytest.mark.gpu
def test_non_finite_coordinates_are_refused_on_the_pipelines(debug_checks):
    from hgcalml_amd import BinnedSelectKnn, BuildAndAssignCondensatesBinned
    rng = np.random.default_rng(3)
    x = rng.random((500, 4)).astype(np.float32)
    rs = torch.tensor([0, 500], dtype=torch.int32)
    for bad in (np.nan, np.inf):
        y = x.copy()
        y[123, 1] = bad
        with pytest.raises(ValueError, match="NaN or Inf"):
            BinnedSelectKnn(8, torch.from_numpy(y).to(DEV), rs, n_bins=5)
        with pytest.raises(ValueError, match="NaN or Inf"):
            BuildAndAssignCondensatesBinned(torch.from_numpy(y).to(DEV), torch.rand(500, 1, device=DEV),
                                            torch.full((500, 1), 0.1, device=DEV), rs.to(DEV), 0.1)
    # binning as the reference does leaves the fourth coordinate out, and so does its check;
    # the library's own grid bins (and checks) it too
    from hgcalml_amd import globals as gl
    y = x.copy()
    y[7, 3] = np.inf
    gl.knn_callers_grid = True
    try:
        BinnedSelectKnn(8, torch.from_numpy(y).to(DEV), rs, n_bins=5)
    finally:
        gl.knn_callers_grid = False
    with pytest.raises(ValueError, match="NaN or Inf"):
        BinnedSelectKnn(8, torch.from_numpy(y).to(DEV), rs, n_bins=5)
    # clean data passes, including the condensate count relation
    BuildAndAssignCondensatesBinned(torch.from_numpy(x).to(DEV), torch.rand(500, 1, device=DEV),
                                    torch.full((500, 1), 0.1, device=DEV), rs.to(DEV), 0.1, keep_noise=True)


@pytest.mark.gpu
def test_bin_beyond_the_boundary_table_is_flagged_and_skipped(oracle):
    """the op on a boundary table that is one event too short: the reference prints 'idx out of
    range' and skips those bins; here the points of the missing event keep their defaults"""
    from hgcalml_amd import ops
    from hgcalml_amd._lib import check, lib, p, stream
    rng = np.random.default_rng(4)
    x = rng.random((300, 3)).astype(np.float32)
    rs = np.array([0, 150, 300], np.int32)
    dbin, flat, nb, bw, nper = oracle.BinByCoordinates(x, rs, n_bins=4)
    order = np.argsort(flat, kind="stable")
    bounds = np.concatenate([[0], np.cumsum(nper)]).astype(np.int32)
    cells = int(np.prod(nb))
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(DEV)  # noqa: E731
    args = [t(x[order]), t(flat[order]), t(dbin[order]), t(nb), t(bw)]
    idx = torch.empty((300, 6), dtype=torch.int32, device=DEV)
    dist = torch.empty((300, 6), dtype=torch.float32, device=DEV)

    def run(table):
        tb = t(table)
        check(lib.hgc_binned_select_knn(p(args[0]), p(args[1]), None, p(args[2]), p(tb), p(args[3]), p(args[4]), p(idx),
                                        p(dist), 300, 6, 3, 3, len(table), 0, 0, stream()))
    assert _status_after(lambda: run(bounds)) == 0
    whole = idx.clone()
    assert _status_after(lambda: run(bounds[:cells + 1])) == ops.FLAG_BIN_BEYOND_TABLE
    assert torch.equal(idx[:150], whole[:150])                      # first event untouched
    assert (idx[150:, 1:] == -1).all() and (idx[150:, 0] == torch.arange(150, 300, device=DEV)).all()


@pytest.mark.gpu
def test_replacement_out_of_range_is_flagged_and_left_alone(debug_checks):
    from hgcalml_amd import IndexReplacer, ops
    tbr = torch.tensor([[0, 2, -1], [5, 1, 9]], dtype=torch.int32, device=DEV)
    rep = torch.tensor([10, 11, 12], dtype=torch.int32, device=DEV)
    with pytest.warns(ops.DataWarning, match="replacements"):
        out = IndexReplacer(tbr, rep)
    assert out.cpu().tolist() == [[10, 12, -1], [0, 11, 0]]          # untouched entries keep the zero fill
    with warnings.catch_warnings():
        warnings.simplefilter("error")
        IndexReplacer(tbr[:1], rep)


@pytest.mark.gpu
def test_too_fine_grid_is_refused_or_flagged():
    """5 binned dimensions, 48 bins each: the grid has 49^4 > 2^22 rows of bins, more than a shell of the walk may have"""
    from hgcalml_amd import BinnedSelectKnn
    from hgcalml_amd import globals as gl
    x = torch.rand((200, 5), device=DEV)
    rs = torch.tensor([0, 200], dtype=torch.int32)
    gl.knn_callers_grid = True          # bin exactly as asked
    try:
        with pytest.raises(ValueError, match="too fine"):
            BinnedSelectKnn(4, x, rs, n_bins=48, max_bin_dims=5)
        idx, _ = BinnedSelectKnn(4, x, rs, n_bins=20, max_bin_dims=5)
    finally:
        gl.knn_callers_grid = False
    assert (idx[:, 0].cpu() == torch.arange(200)).all() and (idx >= 0).all()
    # on the library's own grid the same request is simply answered
    idx2, _ = BinnedSelectKnn(4, x, rs, n_bins=48, max_bin_dims=5)
    assert torch.equal(idx, idx2)
