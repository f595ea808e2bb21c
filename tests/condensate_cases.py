"""Hand-computed condensate assignments: the expected arrays are literals worked out on
paper from the text of modules/compiled/binned_assign_to_condensates_kernel.cc (pick loop
:187-236, claim rules :86-116) and the wrapper modules/assign_condensate_op.py:252-327.
They pin the oracle (CPU test) and are compared with the GPU result as they stand.

All hits sit on the x axis (y = 0) at multiples of 1/8, so every difference, square and
product below is exact in fp32; groups are 10 apart and cannot see each other. Betas are
distinct, so no tie-break is involved. `beta_threshold` is 0.1; "low" hits have beta 0.05.
"""
import numpy as np

LOW = 0.05


def _case(name, hits, row_splits, by_max_beta, assignment, asso, alpha, ncond):
    x, beta, radius, mask = (np.array(c) for c in zip(*hits))
    cc = np.stack([x, np.zeros_like(x)], axis=1).astype(np.float32)
    return dict(name=name, ccoords=cc, betas=beta.astype(np.float32)[:, None], dist=radius.astype(np.float32)[:, None],
                mask=mask.astype(np.int32)[:, None], row_splits=np.array(row_splits, np.int32), beta_threshold=0.1,
                assign_by_max_beta=by_max_beta, assignment=np.array(assignment, np.int32),
                asso=np.array(asso, np.int32), alpha=np.array(alpha, np.int32), ncond=np.array(ncond, np.int32))


# (x, beta, radius, no_condensation_mask)
_CLAIM_HITS = [
    # group 1: A (r=.5) at 0, B (r=.5) at .875 (|AB| = .875 > .5: both are condensation points)
    (0.0, 0.95, 0.5, 0),     # 0  A1, shower 0
    (0.5, LOW, 0.5, 0),      # 1  d2(A1) = .25 <= .25: claimed, best = .25; d2(B1) = .140625 and
                             #    best * r2 = .25 * .25 = .0625 < .140625: NOT re-assigned although B1 is closer
    (0.875, 0.90, 0.5, 0),   # 2  B1, shower 1
    # group 2: B at .75 from A
    (10.0, 0.85, 0.5, 0),    # 3  A2, shower 2
    (10.5, LOW, 0.5, 0),     # 4  d2(A2) = .25, best = .25; d2(B2) = .0625 and .25 * .25 = .0625 >= .0625: re-assigned
    (10.75, 0.80, 0.5, 0),   # 5  B2, shower 3
    # group 3: B has radius 1, so best * r2 = best: B takes a hit iff it is at least as close as A
    (20.0, 0.75, 0.5, 0),    # 6  A3, shower 4; inside B3's sphere (d2 = .5625) but best = 0: stays its own
    (20.25, LOW, 0.5, 0),    # 7  d2(A3) = .0625; d2(B3) = .25 > .0625: stays with A3
    (20.375, LOW, 0.5, 0),   # 8  d2(A3) = d2(B3) = .140625: equal, the later point (B3) takes it
    (20.5, LOW, 0.5, 0),     # 9  d2(A3) = .25; d2(B3) = .0625: B3
    (20.75, 0.70, 1.0, 0),   # 10 B3, shower 5
    (21.5, LOW, 0.5, 0),     # 11 only in B3's sphere (d2 = .5625 <= 1)
    (22.0, LOW, 0.5, 0),     # 12 d2(B3) = 1.5625 > 1: noise
    # group 4: a high-beta hit that is claimed never becomes a point, also after it changes hands
    (30.0, 0.65, 0.5, 0),    # 13 A4, shower 6
    (30.5, 0.60, 0.5, 0),    # 14 beta above threshold; d2(A4) = .25: claimed; d2(B4) = .0625 = .25 * .25: re-assigned
    (30.75, 0.55, 0.5, 0),   # 15 B4, shower 7 (|A4 B4| = .75 > .5)
]

CASES = [
    _case("min_distance_rule", _CLAIM_HITS, [0, 16], False,
          assignment=[0, 0, 1, 2, 3, 3, 4, 4, 5, 5, 5, 5, -1, 6, 7, 7],
          asso=[0, 0, 2, 3, 5, 5, 6, 6, 10, 10, 10, 10, -1, 13, 15, 15],
          alpha=[0, 2, 3, 5, 6, 10, 13, 15], ncond=[0, 8]),
    # the same hits with assign_by_max_beta: the first point that covers a hit keeps it
    _case("first_coverer_keeps", _CLAIM_HITS, [0, 16], True,
          assignment=[0, 0, 1, 2, 2, 3, 4, 4, 4, 4, 5, 5, -1, 6, 6, 7],
          asso=[0, 0, 2, 3, 3, 5, 6, 6, 6, 6, 10, 10, -1, 13, 13, 15],
          alpha=[0, 2, 3, 5, 6, 10, 13, 15], ncond=[0, 8]),
    # The pick loop tests `no_condensation_mask_h[(row_offset_h + iv_h) > 0]` (:193): entry 0 of the
    # high-beta mask for the very first high-beta hit, entry 1 for every other one. Here entry 1 (hit 1)
    # is set: every scan stops at its first unclaimed hit other than hit 0, so the picks run in position
    # order 1, 2, 3 and hit 0 (beta .5) comes last, although beta order would be 1 (masked), 3, 2, 0.
    _case("mask_entry_1_set", [(0.0, 0.5, 0.5, 0), (10.0, 0.6, 0.5, 1), (20.0, 0.7, 0.5, 0), (30.0, 0.9, 0.5, 0),
                               (30.25, LOW, 0.5, 0),   # in hit 3's sphere
                               (10.0, LOW, 0.5, 0)],   # on top of the masked hit 1, which claims only itself: noise
          [0, 6], True, assignment=[3, 0, 1, 2, 2, -1], asso=[0, 1, 2, 3, 3, -1], alpha=[1, 2, 3, 0], ncond=[0, 4]),
    # entry 2 is set, entries 0 and 1 are not: the early exit never looks at entry 2, so hit 2 is picked
    # by its beta (last) and then claims only itself (radius 0): its neighbour 4 stays noise
    _case("mask_entry_2_set", [(0.0, 0.9, 0.5, 0), (10.0, 0.8, 0.5, 0), (20.0, 0.3, 0.5, 1), (30.0, 0.5, 0.5, 0),
                               (20.25, LOW, 0.5, 0)],
          [0, 5], False, assignment=[0, 1, 3, 2, -1], asso=[0, 1, 2, 3, -1], alpha=[0, 1, 3, 2], ncond=[0, 4]),
    # entry 0 is set (a hit below the beta threshold that the mask puts into the high-beta subset): picked
    # first, claims only itself (hit 1 on top of it stays noise); hit 4 is masked too (entry 3, never seen
    # by the early exit): hit 3 cannot claim it although it is inside its sphere, it is picked last by beta
    _case("mask_entry_0_set", [(0.0, LOW, 0.5, 1), (0.0, LOW, 0.5, 0), (10.0, 0.6, 0.5, 0), (20.0, 0.9, 0.5, 0),
                               (20.25, LOW, 0.5, 1)],
          [0, 5], True, assignment=[0, -1, 2, 1, 3], asso=[0, -1, 2, 3, 4], alpha=[0, 3, 2, 4], ncond=[0, 4]),
    # two events: entry 1 of the WHOLE high-beta mask (hit 1, event 0) also steers event 1, whose entries
    # all have index > 0: its picks run in position order 2, 3, 4 instead of beta order 3, 4, 2
    _case("mask_entry_1_steers_next_event", [(0.0, 0.9, 0.5, 0), (10.0, 0.2, 0.5, 1),
                                             (0.0, 0.5, 0.5, 0), (10.0, 0.9, 0.5, 0), (20.0, 0.7, 0.5, 0)],
          [0, 2, 5], False, assignment=[1, 0, 0, 1, 2], asso=[0, 1, 2, 3, 4], alpha=[1, 0, 2, 3, 4],
          ncond=[0, 2, 5]),
]
