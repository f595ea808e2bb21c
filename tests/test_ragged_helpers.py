"""Post-condensation index helpers (pure index arithmetic, run on the CPU):
brute-force loops over small random assignments and the invariants of the
reference's own test, tests/unit/condensate.py:67-112."""
import numpy as np
import pytest
import torch


def random_assignment(rng, n_events, with_noise, with_empty_event=False):
    """per event: consecutive shower ids 0..S-1, optionally noise (-1); every shower has a hit"""
    a, rs, alpha = [], [0], []
    for e in range(n_events):
        if with_empty_event and e == 1:
            rs.append(rs[-1])
            continue
        n_showers = int(rng.integers(1, 6))
        n_hits = int(rng.integers(n_showers, 40))
        ids = np.concatenate([np.arange(n_showers), rng.integers(0, n_showers, n_hits - n_showers)])
        if with_noise and (e % 2 == 0 or n_events == 1):
            ids = np.concatenate([ids, -np.ones(int(rng.integers(1, 8)), np.int64)])
        ids = rng.permutation(ids)
        base = rs[-1]
        for s in range(n_showers):
            alpha.append(base + int(rng.choice(np.nonzero(ids == s)[0])))
        a.append(ids)
        rs.append(base + len(ids))
    a = np.concatenate(a).astype(np.int32)
    return a, np.array(rs, np.int32), np.array(alpha, np.int32)


@pytest.mark.parametrize("seed", range(6))
@pytest.mark.parametrize("with_noise", [True, False])
def test_ragged_indices_vs_brute_force(seed, with_noise):
    from hgcalml_amd.assign_condensate_op import (calc_ragged_cond_indices, calc_ragged_shower_indices,
                                                  collapse_ragged_noise)
    rng = np.random.default_rng(seed)
    a, rs, alpha = random_assignment(rng, 4, with_noise)
    ta, trs, talpha = torch.from_numpy(a)[:, None], torch.from_numpy(rs), torch.from_numpy(alpha)

    for gather_noise in (True, False):
        got = calc_ragged_shower_indices(ta, trs, gather_noise=gather_noise).to_list()
        want = []
        for e in range(len(rs) - 1):
            ids = a[rs[e]:rs[e + 1]]
            showers = sorted(set(ids.tolist()) - (set() if gather_noise else {-1}))
            want.append([[[int(rs[e] + i)] for i in np.nonzero(ids == s)[0]] for s in showers])
        assert got == want

    rc, rev, flat = calc_ragged_cond_indices(ta, talpha, None, trs)
    want_rc, k = [], 0
    for e in range(len(rs) - 1):
        ids = a[rs[e]:rs[e + 1]]
        row = []
        if (ids < 0).any():
            row.append([int(rs[e] + np.nonzero(ids < 0)[0].max())])   # the last noise hit
        n_sh = ids.max() + 1
        row += [[int(x)] for x in alpha[k:k + n_sh]]
        k += n_sh
        want_rc.append(row)
    assert rc.to_list() == want_rc
    rc_plain = calc_ragged_cond_indices(ta, talpha, None, trs, gather_noise=False, return_reverse=False)
    assert rc_plain.to_list() == [[x for x in row if a[x[0]] >= 0] for row in want_rc]

    # invariants of the reference's test: the condensation point of every shower carries the
    # shower's assignment, and both reverse indices bring it back to every hit
    sh = calc_ragged_shower_indices(ta, trs)
    assert (sh.nested_row_splits[0] == rc.nested_row_splits[0]).all()
    per_hit = sh.gather(ta[:, 0]).to_list()
    per_cond = rc.gather(ta[:, 0]).to_list()
    assert [[min(s) for s in ev] for ev in per_hit] == per_cond
    assert [[max(s) for s in ev] for ev in per_hit] == per_cond
    back = [per_cond[e][p] for e, p in rev.tolist()]
    assert back == a.tolist()
    flat_cond = [x for ev in per_cond for x in ev]
    assert [flat_cond[p] for p in flat[:, 0].tolist()] == a.tolist()

    # noise showers collapse to their first hit and lead the event
    col = collapse_ragged_noise(sh, rc.gather(ta[:, 0])).to_list()
    for ev_col, ev_full, ev_ass in zip(col, sh.to_list(), per_cond):
        want_ev = [s[:1] for s, c in zip(ev_full, ev_ass) if c < 0] + [s for s, c in zip(ev_full, ev_ass) if c >= 0]
        assert ev_col == want_ev


def test_ragged_indices_single_event_and_all_noise():
    from hgcalml_amd.assign_condensate_op import calc_ragged_cond_indices, calc_ragged_shower_indices
    a = torch.tensor([[-1], [-1], [-1]], dtype=torch.int32)
    rs = torch.tensor([0, 3], dtype=torch.int32)
    assert calc_ragged_shower_indices(a, rs).to_list() == [[[[0], [1], [2]]]]
    assert calc_ragged_shower_indices(a, rs, gather_noise=False).to_list() == [[]]
    rc, rev, flat = calc_ragged_cond_indices(a, torch.empty((0,), dtype=torch.int32), None, rs)
    assert rc.to_list() == [[[2]]] and rev.tolist() == [[0, 0]] * 3 and flat[:, 0].tolist() == [0, 0, 0]


@pytest.mark.parametrize("seed", range(6))
def test_merge_noise_as_indiv_cp_vs_per_event_loop(seed):
    """the keep_noise post-pass (modules/assign_condensate_op.py:16-44) of the package, on CPU tensors,
    against the per-event list loop that also pins the oracle: numbering of the noise hits (ascending
    hit index, before the real showers), order of the merged condensation point list, flags, counts"""
    from hgcalml_amd.assign_condensate_op import merge_noise_as_indiv_cp
    from test_oracle_pins import merge_noise_per_event_loop
    rng = np.random.default_rng(100 + seed)
    a, rs, alpha = random_assignment(rng, 5, True)
    if seed == 0:   # one event that is all noise, at the end
        a = np.concatenate([a, -np.ones(4, np.int32)])
        rs = np.concatenate([rs, [rs[-1] + 4]]).astype(np.int32)
    n_events = len(rs) - 1
    per_event = [int(a[rs[e]:rs[e + 1]].max()) + 1 for e in range(n_events)]
    ncond = np.concatenate([[0], np.cumsum(per_event)]).astype(np.int32)
    asso = np.full(len(a), -1, np.int32)
    for e in range(n_events):
        for i in range(rs[e], rs[e + 1]):
            if a[i] >= 0:
                asso[i] = alpha[ncond[e] + a[i]]
    is_cond = np.zeros((len(a), 1), bool)
    is_cond[alpha, 0] = True
    assert any((a[rs[e]:rs[e + 1]] >= 0).all() for e in range(n_events))       # an event without noise
    got = merge_noise_as_indiv_cp(torch.from_numpy(a)[:, None], torch.from_numpy(asso), torch.from_numpy(alpha),
                                  torch.from_numpy(is_cond), torch.from_numpy(ncond), torch.from_numpy(rs))
    want = merge_noise_per_event_loop(a[:, None], asso, alpha, is_cond, ncond, rs)
    assert got[0][:, 0].tolist() == want[0]
    assert got[1].tolist() == want[1]
    assert got[2].tolist() == want[2]
    assert got[3][:, 0].tolist() == want[3]
    assert got[4].tolist() == want[4]
    assert got[0].dtype == torch.int32 and got[3].dtype == torch.bool
