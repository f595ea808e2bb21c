"""`LocalDistance` — same call signature and results as
modules/local_distance_op.py:11-40 of the reference: squared distances from
every vertex to the neighbours an index table lists (0 for -1 and for the
vertex itself), differentiable w.r.t. the coordinates through SelectKnnGrad.
"""
import torch

from . import ops  # noqa: F401  (registers torch.ops.hgcalml.*)


class _LocalDistanceFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, coords, neighbour_idxs):
        dist = torch.ops.hgcalml.local_distance(coords, neighbour_idxs)
        ctx.save_for_backward(coords, neighbour_idxs, dist)
        return dist

    @staticmethod
    def backward(ctx, dstgrad):
        coords, idx, dist = ctx.saved_tensors
        if idx.shape[0] != coords.shape[0]:
            raise RuntimeError("LocalDistance gradient needs one row of neighbour indices per vertex")
        return torch.ops.hgcalml.select_knn_grad(dstgrad.contiguous(), idx, dist, coords), None


def LocalDistance(coords, neighbour_idxs):
    return _LocalDistanceFn.apply(coords, neighbour_idxs)
