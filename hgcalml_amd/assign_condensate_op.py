"""`BuildAndAssignCondensatesBinned` — same call signature and return tuple as
modules/assign_condensate_op.py:210-373 of the reference, on torch tensors.
Unlike the reference (whose kernel is CPU only) everything runs on the GPU."""
import math

import torch

from . import ops
from .bin_by_coordinates_op import BinByCoordinates


def merge_noise_as_indiv_cp(assignment, asso_idx, alpha_idx, is_cond, n_condensates, row_splits):
    """Every noise hit becomes a condensation point of its own, numbered before
    the real ones inside each event (modules/assign_condensate_op.py:16-44)."""
    dev = assignment.device
    n = assignment.shape[0]
    rs = row_splits.to(device=dev, dtype=torch.int64)
    n_events = rs.numel() - 1
    a = assignment[:, 0].to(torch.int64)
    noise = a < 0
    event_of = torch.searchsorted(rs[1:].contiguous(), torch.arange(n, device=dev), right=True)
    csum = torch.cumsum(noise.to(torch.int64), 0)
    before_event = torch.cat([torch.zeros(1, dtype=torch.int64, device=dev), csum])[rs[:-1]]
    rank = csum - before_event[event_of]                      # 1-based rank among the event's noise hits
    n_noise = torch.zeros(n_events, dtype=torch.int64, device=dev).scatter_add_(0, event_of, noise.to(torch.int64))
    new_assignment = torch.where(noise, rank - 1, a + n_noise[event_of]).to(torch.int32)

    allrange = torch.arange(n, device=dev, dtype=torch.int32)
    ncond = n_condensates.to(torch.int64)
    # per event: noise hit indices first, then the condensate points
    noise_idx = allrange[noise]
    noise_ev = event_of[noise]
    alpha_ev = torch.searchsorted(ncond[1:].contiguous(), torch.arange(alpha_idx.numel(), device=dev), right=True)
    merged = torch.cat([noise_idx, alpha_idx.to(torch.int32)])
    key = torch.cat([noise_ev * 2, alpha_ev * 2 + 1])
    order = torch.sort(key, stable=True).indices
    new_alpha = merged[order]

    new_is_cond = torch.where(asso_idx < 0, torch.ones_like(is_cond[:, 0]), is_cond[:, 0])
    new_asso = torch.where(asso_idx < 0, allrange, asso_idx)
    per_event = torch.zeros(n_events, dtype=torch.int64, device=dev).scatter_add_(0, event_of,
                                                                                 new_is_cond.to(torch.int64))
    new_ncond = torch.cat([n_condensates[0:1].to(torch.int32), torch.cumsum(per_event, 0).to(torch.int32)])
    return new_assignment[:, None], new_asso, new_alpha, new_is_cond[:, None], new_ncond


def BuildAndAssignCondensatesBinned(ccoords, betas, dist, row_splits, beta_threshold, no_condensation_mask=None,
                                    distance_threshold=1., assign_by_max_beta=False, nbin_dims=3, keep_noise=False):
    """
    :param ccoords: [nvert, ndim] clustering coordinates
    :param betas: [nvert, 1]
    :param dist: [nvert, 1] local distance thresholds
    :param row_splits: [nevents+1]
    :param beta_threshold: minimum beta of a condensation point
    :param no_condensation_mask: 1 for each hit that must become its own condensation point
    :param assign_by_max_beta: True: the higher-beta point takes every unassigned hit in its radius;
                               False: a hit goes to the point it is (relatively) closest to
    :param keep_noise: noise hits become one condensation point each
    :return: (assignment [nvert,1], association [nvert], alpha_idx [ncond], is_cond [nvert,1] bool,
              n_condensates [nevents+1])
    """
    assert 1 <= nbin_dims <= 6
    assert 0. <= beta_threshold <= 1.
    assert distance_threshold > 0.
    ccoords = ccoords.to(torch.float32)
    dev = ccoords.device
    n = ccoords.shape[0]
    row_splits = row_splits.to(device=dev, dtype=torch.int32).contiguous()
    num_rows = row_splits.numel() - 1

    dist = (dist.to(torch.float32) / distance_threshold).reshape(-1)
    betas = betas.to(torch.float32).reshape(-1)
    if no_condensation_mask is None:
        mask = torch.zeros((n,), dtype=torch.int32, device=dev)
    else:
        mask = no_condensation_mask.to(device=dev, dtype=torch.int32).reshape(-1)

    n_bins_sc = max(4, min(int(math.ceil(math.pow(n / 5, 1 / 3))), 25))
    ccoords = (ccoords - ccoords.min(dim=0, keepdim=True).values).contiguous()
    n_bin_dims = min(ccoords.shape[1], nbin_dims)

    # binning of the first n_bin_dims columns (pre-normalised), stable sort into bin order
    _shift, bin_width, n_bins = ops.bin_setup(ccoords, n_bin_dims, True, n_bins=n_bins_sc)
    cells_bound = (n_bins_sc + 1) ** n_bin_dims * num_rows
    _, bins_flat, _ = ops.bin_points(ccoords, n_bin_dims, None, row_splits, bin_width, n_bins, cells_bound, False)
    sorting, bin_splits = ops.sort_by_bin(bins_flat, cells_bound)

    ccoords_s = ops.gather_rows(ccoords, sorting)
    betas_s = ops.gather_rows(betas.contiguous(), sorting)
    dist_s = ops.gather_rows(dist.contiguous(), sorting)
    mask_s = ops.gather_rows(mask.contiguous(), sorting)
    bins_s = ops.gather_rows(bins_flat, sorting)

    # high-beta subset, same order
    high = (betas_s > beta_threshold) | (mask_s > 0)
    csum = torch.cumsum(high.to(torch.int32), 0, dtype=torch.int32)
    to_filtered = torch.where(high, csum - 1, torch.full_like(csum, -1))
    csum0 = torch.cat([torch.zeros(1, dtype=torch.int32, device=dev), csum])
    row_splits_h = csum0[row_splits.to(torch.int64)].contiguous()
    sel = torch.nonzero(high).reshape(-1)
    ccoords_h = ccoords_s[sel]
    betas_h = betas_s[sel]
    dist_h = dist_s[sel]
    mask_h = mask_s[sel]
    orig_h = sorting[sel]

    _, assignment_s, alpha, asso_s, n_condensates = torch.ops.hgcalml.binned_assign_to_condensates(
        ccoords_s, dist_s, betas_s, mask_s, bins_s, bin_splits, to_filtered, orig_h, row_splits, n_bins, bin_width,
        ccoords_h, dist_h, betas_h, mask_h, row_splits_h, float(beta_threshold), bool(assign_by_max_beta))

    perm = sorting.to(torch.int64)
    assignment = torch.empty_like(assignment_s)
    asso = torch.empty_like(asso_s)
    assignment[perm] = assignment_s
    asso[perm] = asso_s

    alpha_idx = alpha[alpha != -1]
    is_cond = torch.zeros((n,), dtype=torch.bool, device=dev)
    is_cond[alpha_idx.to(torch.int64)] = True
    out = (assignment[:, None], asso, alpha_idx, is_cond[:, None], n_condensates)
    if keep_noise:
        out = merge_noise_as_indiv_cp(*out, row_splits)
    return out
