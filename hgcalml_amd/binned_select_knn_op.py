"""`BinnedSelectKnn` — same call signature and results as
modules/binned_select_knn_op.py:33-104 of the reference, on torch tensors.

The whole pipeline (bounding box, binning, stable sort into bin order, search,
un-sort) runs on the GPU without a host synchronisation when `n_bins` is given.
"""
import torch

from . import globals as gl
from . import ops


def _BinnedSelectKnn(K, coords, bin_idx, dim_bin_idx, bin_boundaries, n_bins, bin_width, tf_compatible=False,
                     direction=None):
    """the op only (modules/binned_select_knn_op.py:9-30): inputs in bin order"""
    use_direction = direction is not None
    if direction is None:
        direction = torch.empty((0,), dtype=torch.int32, device=coords.device)
    return torch.ops.hgcalml.binned_select_knn(coords, bin_idx, dim_bin_idx, bin_boundaries, n_bins, bin_width,
                                               direction, int(K), bool(tf_compatible), use_direction)


class _BinnedSelectKnnFn(torch.autograd.Function):
    """the op with its registered gradient SelectKnnGrad
    (modules/binned_select_knn_op.py:107-118): distances are differentiable
    w.r.t. the coordinates, indices are not"""

    @staticmethod
    def forward(ctx, coords, rs_dev, dir_dev, K, n_bins, max_bin_dims, tf_compatible, max_radius):
        idx, dist = ops.binned_select_knn_pipeline(coords, rs_dev, dir_dev, K, n_bins, max_bin_dims, tf_compatible,
                                                   max_radius)
        ctx.save_for_backward(coords, idx, dist)
        ctx.mark_non_differentiable(idx)
        return idx, dist

    @staticmethod
    def backward(ctx, _grad_idx, grad_dist):
        coords, idx, dist = ctx.saved_tensors
        grad_coords = torch.ops.hgcalml.select_knn_grad(grad_dist.contiguous(), idx, dist, coords)
        return grad_coords, None, None, None, None, None, None, None


def default_n_bins(first_event_size, K, max_bin_dims):
    # float32 pow, truncation, clamp to [5, 30] (modules/binned_select_knn_op.py:59-63)
    v = torch.pow(torch.tensor(float(first_event_size), dtype=torch.float32) / torch.tensor(K / 32, dtype=torch.float32),
                  torch.tensor(1 / max_bin_dims, dtype=torch.float32))
    return int(min(30, max(5, int(v.to(torch.int32)))))


def BinnedSelectKnn(K, coords, row_splits, direction=None, n_bins=None, max_bin_dims=3, tf_compatible=False,
                    max_radius=None, name=""):
    """K nearest neighbours (including the point itself in slot 0) inside each event.

    direction, if provided: 0 can only be neighbour, 1 can only have neighbours,
    2 neither, anything else both.

    max_radius, if > 0: neighbours farther than max_radius are dropped (the
    reference accepts the argument and ignores it).

    Returns (indices [N,K] int32, squared distances [N,K] float32) in the order
    and index space of the input; slots 1.. are sorted by ascending
    (distance, index), missing neighbours are (-1, 0.0) at the tail.
    """
    coords = coords.to(torch.float32).contiguous()
    dev = coords.device
    n, n_coords = coords.shape
    row_splits = row_splits.to(torch.int32)
    if row_splits.is_cuda:
        rs_dev = row_splits.contiguous()
        rs_host = None
    else:
        rs_host = row_splits
        rs_dev = row_splits.to(dev).contiguous()
        if int(rs_host[-1]) != n:
            raise ValueError("BinnedSelectKnn: row_splits[-1] must equal the number of points")
    n_events = rs_dev.numel() - 1
    max_bin_dims = min(max_bin_dims, n_coords)

    if n_bins is None:
        if gl.knn_callers_grid:
            first = int(rs_host[1]) if rs_host is not None else int(rs_dev[1])
            n_bins = default_n_bins(first, K, max_bin_dims)
        else:
            n_bins = 30  # the library searches on a grid of its own: no read of the first event's size
    n_bins = int(n_bins)
    if n == 0:
        return (torch.empty((0, K), dtype=torch.int32, device=dev),
                torch.empty((0, K), dtype=torch.float32, device=dev))

    if max_bin_dims < 2:
        raise ValueError("BinnedSelectKnnOp expects at least 2 binning dimensions.")
    dir_dev = None if direction is None else direction.to(device=dev, dtype=torch.int32).contiguous()
    if not gl.knn_ops_use_tf_gradients:
        return _BinnedSelectKnnFn.apply(coords, rs_dev, dir_dev, int(K), n_bins, max_bin_dims, bool(tf_compatible),
                                        max_radius)
    idx, dist = ops.binned_select_knn_pipeline(coords, rs_dev, dir_dev, int(K), n_bins, max_bin_dims,
                                               bool(tf_compatible), max_radius)

    # differentiable re-computation of the distances (modules/binned_select_knn_op.py:97-104)
    safe = idx.clamp(min=0).to(torch.int64)
    ncoords = coords[safe]
    ncoords = torch.where((idx < 0)[..., None], torch.zeros_like(ncoords), ncoords)
    distsq = ((ncoords[:, 0:1, :] - ncoords) ** 2).sum(dim=2)
    distsq = torch.where(idx < 0, torch.zeros_like(distsq), distsq)
    return idx, distsq
