"""`NeighbourCovariance` — same call signature and results as
modules/neighbour_covariance_op.py:8-62 of the reference: feature-weighted mean
and covariance of the neighbours' coordinates, built from three mean-only
neighbour accumulations (differentiable through them).
"""
import torch

from .accknn_op import AccumulateKnn


def _divide_no_nan(a, b):
    return torch.where(b == 0, torch.zeros_like(a), a / b)


def NeighbourCovariance(coordinates, distsq, features, n_idxs):
    """returns (cov [N, F, C*C], mean_C [N, F, C]); feed features without activation"""
    features = torch.sigmoid(features) + 1e-3  # make sure they are in a good range
    nF = features.shape[1]
    nC = coordinates.shape[1]
    nKf = float(distsq.shape[1])
    # the accumulations divide by K, which is undone here
    sum_F = AccumulateKnn(distsq, features, n_idxs, mean_and_max=False)[0] * nKf
    FC = (coordinates.unsqueeze(1) * features.unsqueeze(2)).reshape(-1, nF * nC)
    sum_FC = AccumulateKnn(distsq, FC, n_idxs, mean_and_max=False)[0] * nKf
    mean_C = _divide_no_nan(sum_FC.reshape(-1, nF, nC), sum_F.unsqueeze(2) + 1e-3)
    centered_C = coordinates.unsqueeze(1) - mean_C
    cov = (centered_C.unsqueeze(3) * centered_C.unsqueeze(2)).reshape(-1, nF, nC ** 2)
    cov = (cov * features.unsqueeze(2)).reshape(-1, nF * nC ** 2)
    cov = AccumulateKnn(distsq, cov, n_idxs, mean_and_max=False)[0] * nKf
    cov = _divide_no_nan(cov.reshape(-1, nF, nC ** 2), sum_F.unsqueeze(2) + 1e-3)
    return cov, mean_C
