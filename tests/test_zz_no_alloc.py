"""The allocation-free kNN entry point (scratch inside the library's device image)
against hgc_binned_select_knn_pipeline, through the C ABI. Collected last on
purpose: a failure here must not hide the other tests under `pytest -x`."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _both(coords, row_splits, K, n_bins, direction=None, max_radius=-1.0):
    """(idx, dist) of the workspace entry point and of the static-scratch one on the same inputs"""
    import torch
    from hgcalml_amd._lib import check, lib, p, stream, workspace
    dev = "cuda:0"
    c = torch.from_numpy(coords).to(dev)
    rs = torch.from_numpy(row_splits).to(dev)
    d = None if direction is None else torch.from_numpy(direction).to(dev)
    n, C = coords.shape
    out = []
    for static in (False, True):
        idx = torch.full((n, K), -7, dtype=torch.int32, device=dev)
        dist = torch.full((n, K), -7.0, dtype=torch.float32, device=dev)
        order = torch.empty((n,), dtype=torch.int32, device=dev)
        if static:
            # neither torch's allocator nor the device as a whole (hipMemGetInfo: a hipMalloc inside the
            # library would show here) may lose memory over the call; the scratch array's address is
            # looked up on the first call per device, so that call is made before the measurement
            torch.cuda.synchronize()
            if not _both.warmed:
                check(lib.hgc_binned_select_knn_pipeline_static(p(c), p(rs), p(d), n, C, len(row_splits), K, n_bins, 3,
                                                                0, float(max_radius), p(idx), p(dist), p(order), stream()))
                torch.cuda.synchronize()
                _both.warmed = True
            before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
            check(lib.hgc_binned_select_knn_pipeline_static(p(c), p(rs), p(d), n, C, len(row_splits), K, n_bins, 3, 0,
                                                            float(max_radius), p(idx), p(dist), p(order), stream()))
            torch.cuda.synchronize()
            assert torch.cuda.memory_allocated() == before and torch.cuda.mem_get_info()[0] == free_before
        else:
            ws = workspace(lib.hgc_binned_select_knn_pipeline_workspace_bytes(n, C, len(row_splits), n_bins, 3,
                                                                              int(d is not None)), dev)
            check(lib.hgc_binned_select_knn_pipeline(p(c), p(rs), p(d), n, C, len(row_splits), K, n_bins, 3, 0,
                                                     float(max_radius), p(idx), p(dist), p(order), p(ws), ws.numel(),
                                                     stream()))
        torch.cuda.synchronize()
        assert sorted(order.cpu().tolist()) == list(range(n))
        out.append((idx.cpu().numpy(), dist.cpu().numpy()))
    return out


_both.warmed = False


def test_static_scratch_knn_matches_workspace_knn_twice():
    import workloads
    # first call: cfg2-like event at 60k hits in two events; second call: a smaller, different problem
    # (fewer points, other K, direction flags, a radius) that finds the first call's contents in the scratch
    big = workloads.cfg2(scale=0.4)["coords"]
    rs_big = np.array([0, 25000, len(big)], np.int32)
    small = workloads.cfg2(scale=0.03, seed=77)["coords"][:, :3].copy()
    rs_small = np.array([0, len(small)], np.int32)
    direction = np.random.default_rng(5).integers(0, 4, len(small)).astype(np.int32)
    for coords, rs, K, nb, dirn, radius in ((big, rs_big, 32, 30, None, -1.0), (small, rs_small, 12, 9, direction, 0.2)):
        (ri, rd), (si, sd) = _both(coords, rs, K, nb, dirn, radius)
        assert (si == ri).all()
        assert (sd.view(np.int32) == rd.view(np.int32)).all()
        assert (ri[:, 0] == np.arange(len(coords))).all()


def test_static_scratch_refuses_what_does_not_fit():
    import torch
    from hgcalml_amd._lib import lib, p, stream
    n, C, K = 1_000_000, 4, 8
    assert lib.hgc_binned_select_knn_pipeline_workspace_bytes(n, C, 2, 30, 3, 0) > (32 << 20)
    c = torch.zeros((n, C), device="cuda:0")
    rs = torch.tensor([0, n], dtype=torch.int32, device="cuda:0")
    idx = torch.empty((n, K), dtype=torch.int32, device="cuda:0")
    dist = torch.empty((n, K), dtype=torch.float32, device="cuda:0")
    rc = lib.hgc_binned_select_knn_pipeline_static(p(c), p(rs), None, n, C, 2, K, 30, 3, 0, -1.0, p(idx), p(dist), None,
                                                   stream())
    assert rc == -2 and b"scratch" in lib.hgc_last_error()
