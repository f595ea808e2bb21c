"""Brute-force checkers shared by the oracle pins and the GPU parity tests."""
import numpy as np


def serial_distsq(a, b):
    """((0 + d0^2) + d1^2) + ... in fp32; a [M,C], b [C] or [M,C]"""
    acc = np.zeros(a.shape[0], np.float32)
    for c in range(a.shape[1]):
        d = (a[:, c] - (b[c] if b.ndim == 1 else b[:, c])).astype(np.float32)
        acc = (acc + (d * d).astype(np.float32)).astype(np.float32)
    return acc


def brute_knn_row(coords, lo, hi, i, allowed=None):
    """all other points of the event, ordered by (d^2, index); returns (idx, d^2)"""
    j = np.arange(lo, hi)
    d = serial_distsq(coords[lo:hi], coords[i])
    keep = j != i
    if allowed is not None:
        keep &= allowed[lo:hi]
    j, d = j[keep], d[keep]
    o = np.lexsort((j, d))
    return j[o], d[o]


def check_knn_rows(oracle, idx, dist, coords, row_splits, K, rows, direction=None, tf_compatible=False,
                   radius=None):
    """every listed row: oracle set == brute-force set unless the K-th boundary
    is an exact tie, in which case the row must still be a valid kNN set.
    Returns the number of tie rows."""
    ties = 0
    ev = np.searchsorted(row_splits[1:], rows, side="right")
    allowed = None if direction is None else ~np.isin(direction, (1, 2))
    for i, e in zip(rows, ev):
        lo, hi = row_splits[e], row_splits[e + 1]
        if direction is not None and direction[i] in (0, 2):
            assert idx[i, 0] == i
            assert (idx[i, 1:] == (i if tf_compatible else -1)).all()
            assert (dist[i] == 0).all()
            continue
        bj, bd = brute_knn_row(coords, lo, hi, i, allowed)
        if radius is not None:
            m = bd <= np.float32(np.float32(radius) * np.float32(radius))
            bj, bd = bj[m], bd[m]
        want = min(K - 1, len(bj))
        got_i, got_d = idx[i, 1:], dist[i, 1:]
        valid = got_i >= 0 if not tf_compatible else np.arange(1, K) <= want
        assert idx[i, 0] == i and dist[i, 0] == 0
        assert valid.sum() == want, (i, valid.sum(), want)
        gi, gd = got_i[valid], got_d[valid]
        # padding
        if not tf_compatible:
            assert (got_d[~valid] == 0).all()
        else:
            assert (got_i[~valid] == i).all() and (got_d[~valid] == 0).all()
        # distances bitwise per index, all in the same event, no duplicates
        assert len(set(gi.tolist())) == len(gi)
        assert ((gi >= lo) & (gi < hi)).all()
        ref_d = serial_distsq(coords[gi], coords[i])
        assert (ref_d.view(np.int32) == gd.view(np.int32)).all()
        if want == 0:
            continue
        boundary_tie = want < len(bj) and bd[want - 1] == bd[want]
        if not boundary_tie:
            assert set(gi.tolist()) == set(bj[:want].tolist()), i
        else:
            ties += 1
            dk = bd[want - 1]
            assert (gd <= dk).all()
            assert set(bj[bd < dk].tolist()) <= set(gi.tolist())
    return ties
