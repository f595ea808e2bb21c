"""`AccumulateKnn` / `AccumulateLinKnn` — same call signatures and results as
modules/accknn_op.py:18-89 of the reference, on torch tensors, differentiable
w.r.t. distances/weights and features.

Indices must be unique in each row, except for repeated self references used
as padding; -1 entries are skipped (padding at the end of the row).
"""
import torch

from . import globals as gl
from . import ops


class _AccumulateFn(torch.autograd.Function):
    """op + registered gradient (modules/accknn_op.py:71-89)"""

    @staticmethod
    def forward(ctx, weights, features, indices, mean_and_max):
        out, maxidx, slots = torch.ops.hgcalml.accumulate_knn_slots(weights, features, indices, 0, mean_and_max)
        ctx.save_for_backward(weights, features, indices, maxidx, slots)
        ctx.indices_ref = indices
        ctx.mark_non_differentiable(maxidx)
        return out, maxidx

    @staticmethod
    def backward(ctx, grad_out, _grad_maxidx):
        weights, features, indices, maxidx, slots = ctx.saved_tensors
        inv_off, inv_slots = ops.cached_inverse_neighbour_index(ctx.indices_ref)
        gw, gx = torch.ops.hgcalml.accumulate_knn_grad_slots(grad_out.contiguous(), weights, features, indices,
                                                             maxidx, slots, inv_off, inv_slots)
        return gw, gx, None, None


class _AccumulateExpFn(torch.autograd.Function):
    """AccumulateKnn as one op each way: exp(-distances) is taken inside the accumulation kernel
    (modules/accknn_op.py:52 + :71-89), the gradient w.r.t. the distances is -(gw * w)"""

    @staticmethod
    def forward(ctx, distances, features, indices, mean_and_max):
        out, maxidx, slots, weights = torch.ops.hgcalml.accumulate_knn_exp_slots(distances, features, indices, 0,
                                                                                 mean_and_max)
        ctx.save_for_backward(weights, features, indices, maxidx, slots)
        ctx.indices_ref = indices
        ctx.mark_non_differentiable(maxidx)
        return out, maxidx

    @staticmethod
    def backward(ctx, grad_out, _grad_maxidx):
        weights, features, indices, maxidx, slots = ctx.saved_tensors
        inv_off, inv_slots = ops.cached_inverse_neighbour_index(ctx.indices_ref)
        gw, gx = torch.ops.hgcalml.accumulate_knn_grad_slots(grad_out.contiguous(), weights, features, indices,
                                                             maxidx, slots, inv_off, inv_slots)
        return ops.exp_neg_grad(gw, weights), gx, None, None


class _ExpNegFn(torch.autograd.Function):
    """weights = exp(-distances) (modules/accknn_op.py:52) and its chain rule, one kernel each"""

    @staticmethod
    def forward(ctx, distances):
        weights = ops.exp_neg(distances)
        ctx.save_for_backward(weights)
        return weights

    @staticmethod
    def backward(ctx, grad_weights):
        weights, = ctx.saved_tensors
        return ops.exp_neg_grad(grad_weights.contiguous(), weights)


def _torch_composition(weights, features, indices, mean_and_max):
    # the reference's pure-TF path (modules/accknn_op.py:27-36): padded slots
    # contribute 0 to the mean and to the max
    w = weights.unsqueeze(2)
    safe = indices.clamp(min=0).to(torch.int64)
    nfeat = features[safe]
    nfeat = torch.where((indices < 0)[..., None], torch.zeros_like(nfeat), nfeat)
    wfeat = w * nfeat
    fout = wfeat.mean(dim=1)
    if mean_and_max:
        fout = torch.cat([fout, wfeat.max(dim=1).values], dim=1)
    return fout, None


def AccumulateLinKnn(weights, features, indices, mean_and_max=True, force_tf=False):
    """Accumulates neighbour features with linear weights (not exp(-w) as AccumulateKnn)."""
    if (not gl.acc_ops_use_tf_gradients) and (not force_tf):
        return _AccumulateFn.apply(weights, features, indices, bool(mean_and_max))
    return _torch_composition(weights, features, indices, mean_and_max)


def AccumulateKnn(distances, features, indices, mean_and_max=True, force_tf=False):
    """Weighted mean (and max) of neighbour features with weights exp(-distances).

    Returns (out [N, 2F] (mean | max) or [N, F], arg-max neighbour index [N, F]).
    """
    if (not gl.acc_ops_use_tf_gradients) and (not force_tf):
        if distances.dtype == torch.float32:
            return _AccumulateExpFn.apply(distances, features, indices, bool(mean_and_max))
        return _AccumulateFn.apply(torch.exp(-distances), features, indices, bool(mean_and_max))
    return _torch_composition(torch.exp(-distances), features, indices, mean_and_max)


def _sumw(acc, x, features, indices, mean_and_max):
    # modules/GravNetLayersRagged.py:35-62: a column of ones rides along and
    # collects the accumulated weight; divide_no_nan
    origshape = features.shape[1]
    features = torch.cat([features, torch.ones_like(features[:, 0:1])], dim=1)
    f, midx = acc(x, features, indices, mean_and_max=mean_and_max)
    fmean = f[:, :origshape]
    fnorm = f[:, origshape:origshape + 1]
    # tf.math.divide_no_nan: 0 where the accumulated weight is 0, and a zero gradient there too
    # (dividing by the raw denominator would send 0/0 = NaN into the backward pass)
    empty = fnorm == 0
    fmean = torch.where(empty, torch.zeros_like(fmean), fmean / torch.where(empty, torch.ones_like(fnorm), fnorm))
    if mean_and_max:
        fmean = torch.cat([fmean, f[:, origshape + 1:-1]], dim=1)
    return fmean, midx


def AccumulateKnnSumw(distances, features, indices, mean_and_max=False):
    return _sumw(AccumulateKnn, distances, features, indices, mean_and_max)


def AccumulateLinKnnSumw(weights, features, indices, mean_and_max=False):
    return _sumw(AccumulateLinKnn, weights, features, indices, mean_and_max)
