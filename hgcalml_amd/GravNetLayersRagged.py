"""`RaggedGravNet` — the GravNet block that sits directly on top of the custom-op
path (modules/GravNetLayersRagged.py:3095-3283 of the reference), as a
``torch.nn.Module``: learned coordinates -> BinnedSelectKnn -> AccumulateKnn of
the propagated features with weights exp(-10 d^2) -> output transform.

Only the exact kNN is built (the reference asserts the same,
GravNetLayersRagged.py:3135). Gradients flow through the accumulated features
(AccumulateKnnGrad), through the distances into the coordinates (SelectKnnGrad)
and through the dense layers (torch).
"""
import torch
from torch import nn

from . import ops
from .accknn_op import AccumulateKnn, AccumulateKnnSumw
from .binned_select_knn_op import BinnedSelectKnn


def eye_init_(weight, mean=0.0, stddev=0.1, eye_scaling=1.0):
    """identity + normal noise (modules/Initializers.py:4-26); `weight` is
    [out, in] as torch stores it, the identity is laid on the [in, out] view"""
    with torch.no_grad():
        weight.normal_(mean, stddev)
        n_out, n_in = weight.shape
        weight += torch.eye(n_in, n_out, dtype=weight.dtype, device=weight.device).t() * eye_scaling
    return weight


class _TallLinearFn(torch.autograd.Function):
    """y = x W^T + b for x of very many rows. The weight gradient g^T x reduces over those rows
    into a small matrix; as one GEMM it runs on a handful of workgroups (0.35-0.44 ms for 150k rows
    of 64-192 columns), as a batch of 64 row slices added up afterwards it takes 0.07-0.11 ms."""

    SLICES = 64

    @staticmethod
    def forward(ctx, x, weight, bias):
        ctx.save_for_backward(x, weight)
        ctx.has_bias = bias is not None
        return torch.nn.functional.linear(x, weight, bias)

    @staticmethod
    def backward(ctx, g):
        x, weight = ctx.saved_tensors
        g = g.contiguous()
        grad_x = g @ weight if ctx.needs_input_grad[0] else None
        grad_w = None
        if ctx.needs_input_grad[1]:
            n, s = x.shape[0], _TallLinearFn.SLICES
            whole = n // s * s
            if whole >= 64 * s:
                grad_w = torch.bmm(g[:whole].view(s, -1, g.shape[1]).transpose(1, 2),
                                   x[:whole].view(s, -1, x.shape[1])).sum(0)
                if whole < n:
                    grad_w = grad_w + g[whole:].t() @ x[whole:]
            else:
                grad_w = g.t() @ x
        grad_b = g.sum(0) if ctx.has_bias and ctx.needs_input_grad[2] else None
        return grad_x, grad_w, grad_b


class TallLinear(nn.Linear):
    """nn.Linear whose weight gradient is formed slice-wise (see _TallLinearFn); same parameters and results
    up to the summation order of that gradient"""

    def forward(self, x):
        if x.dim() == 2 and x.is_contiguous():
            return _TallLinearFn.apply(x, self.weight, self.bias)
        return super().forward(x)


_ACTIVATIONS = {None: nn.Identity, "linear": nn.Identity, "relu": nn.ReLU, "elu": nn.ELU, "tanh": nn.Tanh,
                "sigmoid": nn.Sigmoid, "selu": nn.SELU, "gelu": nn.GELU}


class RaggedGravNet(nn.Module):
    """call(x [N, F_in], row_splits [R+1]) -> (features [N, n_filters], coordinates
    [N, n_dimensions], neighbour indices, squared distances); the last two with
    the self entry in slot 0 if return_self (then n_neighbours+1 wide)."""

    def __init__(self, in_features, n_neighbours, n_dimensions, n_filters, n_propagate, return_self=True,
                 sumwnorm=False, feature_activation="relu", coord_initialiser_noise=1e-2, n_knn_bins=None):
        super().__init__()
        assert n_neighbours > 1
        self.n_neighbours = n_neighbours
        self.n_dimensions = n_dimensions
        self.n_filters = n_filters
        self.n_propagate = n_propagate
        self.return_self = return_self
        self.sumwnorm = sumwnorm
        self.n_knn_bins = n_knn_bins
        self.input_feature_transform = TallLinear(in_features, n_propagate)
        self.feature_activation = _ACTIVATIONS[feature_activation]()
        self.input_spatial_transform = TallLinear(in_features, n_dimensions, bias=False)
        eye_init_(self.input_spatial_transform.weight, 0.0, coord_initialiser_noise)
        self.output_feature_transform = TallLinear(2 * n_propagate + in_features, n_filters)
        # bookkeeping of the reference (GravNetLayersRagged.py:3180-3193); the exact kNN does not use it
        self.register_buffer("dynamic_radius", torch.tensor(1.0))

    def update_dynamic_radius(self, dist):
        if not self.training:
            return
        with torch.no_grad():
            lindist = torch.sqrt(dist)
            update = lindist.max() * 1.05
            mean_dist = lindist.mean()
            low_update = torch.clamp(update, max=2.0)
            update = torch.where(low_update > 2.0 * mean_dist, low_update, 2.0 * mean_dist) + 1e-3
            self.dynamic_radius += 0.05 * (update - self.dynamic_radius)

    def compute_neighbours_and_distancesq(self, coordinates, row_splits):
        idx, dist = BinnedSelectKnn(self.n_neighbours + 1, coordinates, row_splits, max_radius=-1.0,
                                    tf_compatible=False, n_bins=self.n_knn_bins)
        dist = torch.where(idx < 0, torch.zeros_like(dist), dist)
        self.update_dynamic_radius(dist.detach())
        # the table without its self column, as tensors of their own; it lists the
        # same vertices row by row, so the kNN's processing order applies to it too
        nidx, ndist = idx[:, 1:].contiguous(), dist[:, 1:].contiguous()
        ops.share_vertex_order(idx, nidx)
        ops.declare_without_first_column(nidx, idx)
        if self.return_self:
            return nidx, ndist, idx, dist
        return nidx, ndist, None, None

    def collect_neighbours(self, features, neighbour_indices, distancesq):
        acc = AccumulateKnnSumw if self.sumwnorm else AccumulateKnn
        f, _ = acc(10.0 * distancesq, features, neighbour_indices, mean_and_max=True)
        return f

    def create_output_features(self, x, neighbour_indices, distancesq):
        features = self.feature_activation(self.input_feature_transform(x))
        prev_feat = features
        features = self.collect_neighbours(features, neighbour_indices, distancesq)
        features = features.reshape(-1, prev_feat.shape[1] * 2)
        features = features - prev_feat.repeat(1, 2)
        return torch.relu(self.output_feature_transform(torch.cat([features, x], dim=-1)))

    def forward(self, x, row_splits):
        assert x.dim() == 2 and row_splits.dim() == 1
        coordinates = self.input_spatial_transform(x)
        neighbour_indices, distancesq, sidx, sdist = self.compute_neighbours_and_distancesq(coordinates, row_splits)
        outfeats = self.create_output_features(x, neighbour_indices, distancesq)
        if self.return_self:
            neighbour_indices, distancesq = sidx, sdist
        return outfeats, coordinates, neighbour_indices, distancesq
