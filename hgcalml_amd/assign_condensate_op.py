"""`BuildAndAssignCondensatesBinned` — same call signature and return tuple as
modules/assign_condensate_op.py:210-373 of the reference, on torch tensors.
Unlike the reference (whose kernel is CPU only) everything runs on the GPU."""
import math

import torch

from . import globals as gl
from . import ops


def check_condensate_counts(assignment, n_condensates, row_splits):
    """the reference's closing sanity check (modules/assign_condensate_op.py:334-343):
    n_condensates == [0] ++ cumsum(per event: largest shower index + 1). Events without hits
    count as 0 (the reference's reduce_max has no value there). One host synchronisation."""
    a = assignment[:, 0].to(torch.int64)
    rs = row_splits.to(device=a.device, dtype=torch.int64)
    n_events = rs.numel() - 1
    seg = torch.searchsorted(rs[1:].contiguous(), torch.arange(a.numel(), device=a.device), right=True)
    per_event = torch.full((n_events,), -1, dtype=torch.int64, device=a.device).scatter_reduce(
        0, seg, a, reduce="amax", include_self=True) + 1
    expected = torch.cat([torch.zeros(1, dtype=torch.int64, device=a.device), torch.cumsum(per_event, 0)])
    if not torch.equal(expected, n_condensates.to(torch.int64)):
        raise RuntimeError("BuildAndAssignCondensatesBinned: n_condensates %s does not match the assignment (%s)"
                           % (n_condensates.tolist(), expected.tolist()))


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
    n = ccoords.shape[0]
    # the whole chain (shift to the minimum, binning, bin order, high-beta subset, assignment,
    # back to the caller's order) runs inside the library
    n_bins_sc = max(4, min(int(math.ceil(math.pow(n / 5, 1 / 3))), 25))
    assignment, asso, alpha_idx, is_cond, n_condensates = ops.build_and_assign_condensates(
        ccoords, betas, dist, no_condensation_mask, row_splits, beta_threshold, distance_threshold,
        assign_by_max_beta, nbin_dims, n_bins_sc)
    out = (assignment[:, None], asso, alpha_idx, is_cond[:, None], n_condensates)
    if keep_noise:
        out = merge_noise_as_indiv_cp(*out, row_splits)
    if gl.debug_checks:
        check_condensate_counts(out[0], out[4], row_splits)
    return out


# --------------------------------------------------------------------------- ragged index helpers
#
# Pure index arithmetic on the outputs of BuildAndAssignCondensatesBinned
# (modules/assign_condensate_op.py:47-205). The reference returns
# tf.RaggedTensors; here a `Ragged` (flat values + nested row splits) carries the
# same structure. Events without hits are outside what the reference defines
# (its segment reductions return type limits there); they get no showers here.

def _per_event(values, seg, n_events, reduce, empty):
    out = torch.full((n_events,), empty, dtype=values.dtype, device=values.device)
    return out.scatter_reduce(0, seg, values, reduce=reduce, include_self=True)


def calc_ragged_shower_indices(assignment, row_splits, gather_noise=True):
    """Hit indices grouped as [event, shower, hit, 1]
    (modules/assign_condensate_op.py:47-96).

    :param assignment: [nvert, 1], per event consecutive -1 (noise), 0, 1, 2, ...
    :param gather_noise: True: noise is the first shower of every event that has noise;
                         False: noise hits are dropped
    Hits of one shower are listed in ascending index order (the reference's
    tf.argsort leaves that order unspecified).
    """
    from .ragged import Ragged, segment_ids
    dev = assignment.device
    n = assignment.shape[0]
    rs = row_splits.to(device=dev, dtype=torch.int64)
    n_events = rs.numel() - 1
    a = assignment[:, 0].to(torch.int64)
    seg = segment_ids(rs, n)
    back = None
    if gather_noise:
        big = torch.iinfo(torch.int64).max
        a = a - _per_event(a, seg, n_events, "amin", big)[seg]
    else:
        sel = a >= 0
        back = torch.arange(n, device=dev)[sel]
        a, seg = a[sel], seg[sel]
    n_cond = _per_event(a, seg, n_events, "amax", -1) + 1          # showers per event
    n_cond_n = torch.cat([torch.zeros(1, dtype=torch.int64, device=dev), torch.cumsum(n_cond, 0)])
    a_u = a + n_cond_n[seg]
    per_shower = torch.zeros(int(n_cond_n[-1]), dtype=torch.int64, device=dev).scatter_add_(0, a_u, torch.ones_like(a_u))
    order = torch.sort(a_u, stable=True).indices
    if back is not None:
        order = back[order]
    hit_splits = torch.cat([torch.zeros(1, dtype=torch.int64, device=dev), torch.cumsum(per_shower, 0)])
    return Ragged(order.to(torch.int32)[:, None], (n_cond_n, hit_splits))


def calc_ragged_cond_indices(assignment, alpha_idx, n_condensates, row_splits, gather_noise=True, return_reverse=True):
    """Condensation point indices grouped as [event, condensation point, 1]
    (modules/assign_condensate_op.py:99-188); with gather_noise the last noise
    hit of an event leads its list, parallel to calc_ragged_shower_indices.

    return_reverse: also (revidx [nvert, 2] = (event, position in the event's
    list), flat_rev [nvert, 1] = position in the flat list), which gather
    per-condensation-point values back to the hits.
    """
    from .ragged import Ragged, segment_ids
    del n_condensates  # recomputed from the assignment, as the reference does
    dev = assignment.device
    n = assignment.shape[0]
    rs = row_splits.to(device=dev, dtype=torch.int64)
    n_events = rs.numel() - 1
    a = assignment[:, 0].to(torch.int64)
    seg = segment_ids(rs, n)
    zero = torch.zeros(1, dtype=torch.int64, device=dev)

    n_real = _per_event(a, seg, n_events, "amax", -1) + 1           # condensation points per event, without noise
    cond_splits = torch.cat([zero, torch.cumsum(n_real, 0)])
    values = alpha_idx.to(torch.int64)
    if gather_noise:
        idx = torch.arange(n, device=dev)
        last_noise = _per_event(torch.where(a < 0, idx, torch.full_like(idx, -2)), seg, n_events, "amax", -2)
        has_noise = last_noise >= 0
        n_with = n_real + has_noise.to(torch.int64)
        new_splits = torch.cat([zero, torch.cumsum(n_with, 0)])
        merged = torch.empty(int(new_splits[-1]), dtype=torch.int64, device=dev)
        ev_of_alpha = segment_ids(cond_splits, values.numel())
        pos = torch.arange(values.numel(), device=dev) - cond_splits[ev_of_alpha]
        merged[new_splits[ev_of_alpha] + has_noise.to(torch.int64)[ev_of_alpha] + pos] = values
        merged[new_splits[:-1][has_noise]] = last_noise[has_noise]
        values, cond_splits = merged, new_splits
    rc_ass = Ragged(values.to(torch.int32)[:, None], (cond_splits,))
    if not return_reverse:
        return rc_ass
    big = torch.iinfo(torch.int64).max
    shifted = a - _per_event(a, seg, n_events, "amin", big)[seg]
    n_all = _per_event(shifted, seg, n_events, "amax", -1) + 1
    all_splits = torch.cat([zero, torch.cumsum(n_all, 0)])
    revidx = torch.stack([seg, shifted], dim=1).to(torch.int32)
    flat_rev = (shifted + all_splits[seg]).to(torch.int32)[:, None]
    return rc_ass, revidx, flat_rev


def collapse_ragged_noise(ch_input, c_assignement_index):
    """Per event: the noise entries (condensation point assignment < 0) first,
    cut down to their first hit, then the others unchanged
    (modules/assign_condensate_op.py:191-205).

    :param ch_input: Ragged [event, condensation point, hit, ...]
    :param c_assignement_index: Ragged [event, condensation point] (or a flat
           tensor with one entry per condensation point): -1 for noise
    """
    from .ragged import Ragged, segment_ids
    cond_splits, hit_splits = ch_input.nested_row_splits
    flat = c_assignement_index.flat_values if isinstance(c_assignement_index, Ragged) else c_assignement_index
    noise = flat.reshape(flat.shape[0], -1)[:, 0] < 0
    dev = noise.device
    n_conds = noise.numel()
    ev = segment_ids(cond_splits, n_conds)
    n_events = cond_splits.numel() - 1
    # new position of every condensation point: noise ones lead their event, order otherwise kept
    noise_i = noise.to(torch.int64)
    noise_before = torch.cumsum(noise_i, 0) - noise_i
    other_before = torch.cumsum(1 - noise_i, 0) - (1 - noise_i)
    zero = torch.zeros(1, dtype=torch.int64, device=dev)
    ev_noise0 = torch.cat([zero, torch.cumsum(noise_i, 0)])[cond_splits[:-1]]
    ev_other0 = torch.cat([zero, torch.cumsum(1 - noise_i, 0)])[cond_splits[:-1]]
    n_noise_ev = torch.zeros(n_events, dtype=torch.int64, device=dev).scatter_add_(0, ev, noise_i)
    new_pos = torch.where(noise, cond_splits[:-1][ev] + (noise_before - ev_noise0[ev]),
                          cond_splits[:-1][ev] + n_noise_ev[ev] + (other_before - ev_other0[ev]))
    lengths = hit_splits[1:] - hit_splits[:-1]
    new_len_src = torch.where(noise, torch.clamp(lengths, max=1), lengths)
    new_len = torch.empty_like(new_len_src)
    new_len[new_pos] = new_len_src
    src_of_new = torch.empty_like(new_pos)
    src_of_new[new_pos] = torch.arange(n_conds, device=dev)
    new_hit_splits = torch.cat([zero, torch.cumsum(new_len, 0)])
    total = int(new_hit_splits[-1])
    owner = segment_ids(new_hit_splits, total)                      # new condensation point of every kept hit
    within = torch.arange(total, device=dev) - new_hit_splits[owner]
    take = hit_splits[:-1][src_of_new[owner]] + within
    return Ragged(ch_input.flat_values[take], (cond_splits, new_hit_splits))
