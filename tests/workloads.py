"""Seeded synthetic workloads (numpy, host side) shared by the tests and bench.py.

Five configurations of the custom-op hot path:

  cfg1  one event, N=20k, 3-D uniform, K=16, F=32           (plumbing / correctness)
  cfg2  one event, N=150k, 4-D clusters+noise, K=64, F=64   (headline kNN)
  cfg3  16 ragged events, ~1.1M hits, 3-D, K=32, radius 0.1 (ragged + radius + padding)
  cfg4  N=1M banded neighbour table, K=64, F=128            (accumulate fwd+grad)
  cfg5  8 events, 500k hits, 4-D, beta spectrum             (condensate assignment)

Every generator takes a ``scale`` in (0,1] that shrinks the point counts so the
same distributions can be used at sizes a CPU check finishes in seconds.
"""
import numpy as np


def cluster_mixture(rng, n, dims, n_clusters=300, clustered_fraction=0.6, return_truth=False):
    """HGCal-like event: ``n_clusters`` isotropic Gaussian clusters (centres
    uniform in [-1,1]^dims, sigma uniform in [0.02,0.1], sizes log-normal(5,1)
    normalised to ``clustered_fraction`` of the hits) plus uniform noise in
    [-1,1]^dims, shuffled."""
    n_clu = int(round(n * clustered_fraction))
    sizes = rng.lognormal(mean=5.0, sigma=1.0, size=n_clusters)
    sizes = np.floor(sizes / sizes.sum() * n_clu).astype(np.int64)
    sizes[0] += n_clu - sizes.sum()
    centres = rng.uniform(-1.0, 1.0, size=(n_clusters, dims))
    sigmas = rng.uniform(0.02, 0.1, size=n_clusters)
    cid = np.repeat(np.arange(n_clusters), sizes)
    pts = centres[cid] + rng.standard_normal((n_clu, dims)) * sigmas[cid, None]
    noise = rng.uniform(-1.0, 1.0, size=(n - n_clu, dims))
    x = np.concatenate([pts, noise], axis=0).astype(np.float32)
    truth = np.concatenate([cid, np.full(n - n_clu, -1)])
    # distance to the own cluster centre in units of sigma (inf for noise)
    rel = np.full(n, np.inf)
    rel[:n_clu] = np.linalg.norm(pts - centres[cid], axis=1) / sigmas[cid]
    perm = rng.permutation(n)
    if return_truth:
        return x[perm], truth[perm], rel[perm]
    return x[perm]


def cfg1(scale=1.0, seed=1001):
    rng = np.random.default_rng(seed)
    n = max(64, int(20000 * scale))
    return dict(name="cfg1", coords=rng.random((n, 3), dtype=np.float32),
                row_splits=np.array([0, n], np.int32), K=16, n_bins=30, max_radius=None,
                features=rng.standard_normal((n, 32), dtype=np.float32))


def cfg2(scale=1.0, seed=1002):
    rng = np.random.default_rng(seed)
    n = max(256, int(150000 * scale))
    coords = cluster_mixture(rng, n, 4)
    return dict(name="cfg2", coords=coords, row_splits=np.array([0, n], np.int32), K=64, n_bins=30,
                max_radius=None, features=rng.standard_normal((n, 64), dtype=np.float32))


def cfg3(scale=1.0, seed=1003):
    rng = np.random.default_rng(seed)
    sizes = rng.integers(20000, 120001, size=16)
    sizes = np.maximum(40, (sizes * scale).astype(np.int64))
    coords = np.concatenate([cluster_mixture(rng, int(s), 3) for s in sizes], axis=0)
    rs = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)
    K = 32
    # modules/binned_select_knn_op.py:51-63 — from the FIRST event's size
    n_bins = int(min(30, max(5, int(np.float32(sizes[0] / (K / 32)) ** np.float32(1 / 3)))))
    return dict(name="cfg3", coords=coords, row_splits=rs, K=K, n_bins=n_bins, max_radius=0.1)


def cfg4(scale=1.0, seed=1004, window=2000):
    """Random-but-valid banded neighbour table: slot 0 = self, 63 distinct
    others from [i-window, i+window]."""
    rng = np.random.default_rng(seed)
    n = max(2000, int(1000000 * scale))
    K, F = 64, 128
    window = min(window, (n - 1) // 3)
    # distinct non-zero offsets in [-window, window]: sample K-1 of 2*window
    # without replacement per row via random keys (top-k of a random matrix is
    # too big at N=1M, so draw with rejection in blocks)
    idx = np.empty((n, K), np.int32)
    idx[:, 0] = np.arange(n)
    block = 65536
    for s in range(0, n, block):
        e = min(n, s + block)
        m = e - s
        offs = np.empty((m, K - 1), np.int64)
        todo = np.arange(m)
        cand = rng.integers(1, 2 * window + 1, size=(m, K - 1))
        while True:
            srt = np.sort(cand, axis=1)
            dup = (srt[:, 1:] == srt[:, :-1]).any(axis=1)
            good = ~dup
            offs[todo[good]] = cand[good]
            todo = todo[dup]
            if todo.size == 0:
                break
            cand = rng.integers(1, 2 * window + 1, size=(todo.size, K - 1))
        offs = np.where(offs > window, window - offs, offs)  # (window, 2w] -> negative
        nb = np.arange(s, e)[:, None] + offs
        # reflect at the ends so every index stays valid, distinct and != self
        nb = np.where(nb < 0, np.arange(s, e)[:, None] + window - offs, nb)
        nb = np.where(nb >= n, np.arange(s, e)[:, None] - window - offs, nb)
        idx[s:e, 1:] = nb.astype(np.int32)
    distsq = rng.random((n, K), dtype=np.float32) * np.float32(0.5)
    distsq[:, 0] = 0
    return dict(name="cfg4", indices=idx, distsq=distsq, K=K, F=F,
                features=rng.standard_normal((n, F), dtype=np.float32),
                grad_out=rng.standard_normal((n, 2 * F), dtype=np.float32))


def cfg5(scale=1.0, seed=1005, n_events=8, ragged=False):
    """ragged=True: event sizes drawn from U{20k..120k} and rescaled to the same total
    (500,000 * scale for 8 events); otherwise equal events."""
    rng = np.random.default_rng(seed)
    per = max(64, int(62500 * scale))
    sizes = np.full(n_events, per, np.int64)
    if ragged:
        draw = np.random.default_rng(seed + 7).integers(20000, 120001, n_events).astype(np.float64)
        sizes = np.maximum(64, np.floor(draw / draw.sum() * per * n_events)).astype(np.int64)
        sizes[-1] += per * n_events - sizes.sum()
    coords, betas = [], []
    for m in sizes:
        m = int(m)
        x, _, rel = cluster_mixture(rng, m, 4, return_truth=True)
        b = rng.beta(0.5, 2.0, size=m).astype(np.float32)
        core = rel < 1.0  # "core" = within one sigma of the own cluster centre
        b = np.where(core, np.minimum(b + np.float32(0.5), np.float32(0.999)), b).astype(np.float32)
        coords.append(x)
        betas.append(b)
    n = int(sizes.sum())
    return dict(name="cfg5", ccoords=np.concatenate(coords), betas=np.concatenate(betas)[:, None],
                dist=np.full((n, 1), 0.5, np.float32),
                row_splits=np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32),
                beta_threshold=0.1, distance_threshold=1.0)
