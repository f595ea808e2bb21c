"""`PushKnn` — same call signature and results as modules/push_knn_op.py:10-36
of the reference, on torch tensors, differentiable w.r.t. weights and features.

Pushes (sums) w[v, n] * f[v] into row nidx[v, n]; -1 means no neighbour. A
self index is a neighbour like any other.
"""
import torch

from . import ops  # noqa: F401  (registers torch.ops.hgcalml.*)


class _PushKnnFn(torch.autograd.Function):
    """op + registered gradient (modules/push_knn_op.py:21-36)"""

    @staticmethod
    def forward(ctx, w, f, nidx):
        ctx.save_for_backward(w, f, nidx)
        return torch.ops.hgcalml.push_knn(w, f, nidx)

    @staticmethod
    def backward(ctx, grad):
        w, f, nidx = ctx.saved_tensors
        wgrad, fgrad = torch.ops.hgcalml.push_knn_grad(grad.contiguous(), w, f, nidx)
        return wgrad, fgrad, None


def PushKnn(w, f, nidx):
    return _PushKnnFn.apply(w, f, nidx)
