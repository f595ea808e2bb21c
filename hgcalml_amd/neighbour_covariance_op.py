"""`NeighbourCovariance` -- call signature and results of modules/neighbour_covariance_op.py:8-62
of the reference: for every vertex and feature the feature-weighted mean of its neighbours'
coordinates, and the sum of the neighbours' weighted outer products of their coordinates, each
neighbour centred on its own mean (returns ``(cov [N, F, C*C], mean [N, F, C])``).

Forward: two kernels over the neighbour table (`hgc_neighbour_covariance`) that gather
feature rows, coordinates and means and form the C*C products in registers; the reference's
route through matrices of F*C and F*C*C columns is never materialised.

Backward: stated fallback -- the outputs are rebuilt as a differentiable composition of the
package's accumulation op and torch autograd runs through that. The composition is arranged
for one pass less than a literal transcription would take: the weights' sum and the
weighted coordinate sums share one accumulation over [a | a*x], the second accumulation runs over
the F*C*(C+1)/2 distinct products only.
"""
import torch

from . import ops
from ._lib import check, f32, i32, lib, p, require_device, stream
from .accknn_op import AccumulateKnn

_EPS = 1e-3


def _activated(features):
    return torch.sigmoid(features) + _EPS


def _safe_ratio(num, den):
    zero = den == 0
    return torch.where(zero, torch.zeros_like(num), num / torch.where(zero, torch.ones_like(den), den))


def _moments_by_accumulation(coordinates, distsq, features, n_idxs):
    """(cov, mean) out of two mean-only accumulations; differentiable w.r.t. the three float inputs"""
    a = _activated(features)                                           # [N, F]
    n, n_f = a.shape
    n_c = coordinates.shape[1]
    k = float(distsq.shape[1])
    first = torch.cat([a, (a.unsqueeze(2) * coordinates.unsqueeze(1)).reshape(n, n_f * n_c)], dim=1)
    acc = AccumulateKnn(distsq, first, n_idxs, mean_and_max=False)[0] * k
    total = acc[:, :n_f].unsqueeze(2) + _EPS                            # [N, F, 1]
    mean = _safe_ratio(acc[:, n_f:].reshape(n, n_f, n_c), total)
    offset = coordinates.unsqueeze(1) - mean                           # every vertex about its own mean
    rows, cols = torch.tril_indices(n_c, n_c, device=coordinates.device)
    lower = offset[:, :, rows] * offset[:, :, cols] * a.unsqueeze(2)   # [N, F, C(C+1)/2]
    acc2 = AccumulateKnn(distsq, lower.reshape(n, -1), n_idxs, mean_and_max=False)[0] * k
    tri = _safe_ratio(acc2.reshape(n, n_f, -1), total)
    full = tri.new_zeros((n, n_f, n_c, n_c))
    full[:, :, rows, cols] = tri
    full[:, :, cols, rows] = tri
    return full.reshape(n, n_f, n_c * n_c), mean


class _CovarianceFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, coordinates, distsq, features, n_idxs):
        dev = require_device(coordinates, distsq, features, n_idxs)
        x, d, idx = f32(coordinates), f32(distsq), i32(n_idxs)
        a = _activated(f32(features)).contiguous()
        if x.dim() != 2 or a.dim() != 2 or idx.dim() != 2 or d.shape != idx.shape or \
                not (x.shape[0] == a.shape[0] == idx.shape[0]):
            raise ValueError("NeighbourCovariance expects coordinates [N,C], distsq and n_idxs [N,K], features [N,F]")
        n, c = x.shape
        n_f, k = a.shape[1], idx.shape[1]
        w = ops.exp_neg(d)
        cov = torch.empty((n, n_f, c * c), dtype=torch.float32, device=dev)
        mean = torch.empty((n, n_f, c), dtype=torch.float32, device=dev)
        total = torch.empty((n, n_f), dtype=torch.float32, device=dev)
        check(lib.hgc_neighbour_covariance(p(x), p(w), p(a), p(idx), p(ops.vertex_order_of(n_idxs)), p(cov), p(mean),
                                           p(total), n, c, n_f, k, stream()))
        ctx.save_for_backward(coordinates, distsq, features, n_idxs)
        return cov, mean

    @staticmethod
    def backward(ctx, grad_cov, grad_mean):
        coordinates, distsq, features, n_idxs = ctx.saved_tensors
        needs = ctx.needs_input_grad[:3]
        leaves = [t.detach().requires_grad_(need) for t, need in zip((coordinates, distsq, features), needs)]
        with torch.enable_grad():
            cov, mean = _moments_by_accumulation(leaves[0], leaves[1], leaves[2], n_idxs)
        wanted = [t for t, need in zip(leaves, needs) if need]
        grads = iter(torch.autograd.grad([cov, mean], wanted, [grad_cov, grad_mean], allow_unused=True))
        return tuple(next(grads) if need else None for need in needs) + (None,)


def NeighbourCovariance(coordinates, distsq, features, n_idxs):
    """returns (cov [N, F, C*C], mean_C [N, F, C]); feed features without activation"""
    if coordinates.shape[1] > 6:  # the kernels are built for up to six coordinates
        return _moments_by_accumulation(coordinates, distsq, features, n_idxs)
    return _CovarianceFn.apply(coordinates, distsq, features, n_idxs)
