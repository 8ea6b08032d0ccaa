"""Shared checks for the parity tests."""
import zlib

import numpy as np


def stable_seed(*parts):
    """A seed that is the same in every process (Python salts str hashes per
    run, so a failing draw seeded by hash() could not be drawn again)."""
    return zlib.crc32(repr(parts).encode())


def to_set(edge_index):
    e = np.asarray(edge_index)
    return set(zip(e[0].tolist(), e[1].tolist()))


def brute_force_knn_f64(x, y, ptr_x, ptr_y, k):
    """Float64 brute force with a stable sort: neighbours by ascending
    distance, ties by ascending row.  Returns (rows [m,k] with -1 padding,
    squared distances [m,k] with inf padding)."""
    x = np.asarray(x, dtype=np.float64)
    y = np.asarray(y, dtype=np.float64)
    if ptr_x is None:
        ptr_x, ptr_y = [0, len(x)], [0, len(y)]
    rows = np.full((len(y), k), -1, dtype=np.int64)
    dist = np.full((len(y), k), np.inf)
    for b in range(len(ptr_x) - 1):
        xs, xe, ys, ye = ptr_x[b], ptr_x[b + 1], ptr_y[b], ptr_y[b + 1]
        if xs == xe or ys == ye:
            continue
        d2 = ((y[ys:ye, None, :] - x[None, xs:xe, :]) ** 2).sum(-1)
        order = np.argsort(d2, axis=1, kind="stable")[:, :k]
        kk = order.shape[1]
        rows[ys:ye, :kk] = order + xs
        dist[ys:ye, :kk] = np.take_along_axis(d2, order, 1)
    return rows, dist


def check_knn_against_exact(edges, x, y, ptr_x, ptr_y, k, rel_tie=1e-6,
                            cosine=False):
    """The tolerance of the parity contract: the returned neighbour set of
    every query equals the exact (float64) one except where distances tie
    within `rel_tie` relative; counts and grouping are exact."""
    x64 = np.asarray(x, dtype=np.float64)
    y64 = np.asarray(y, dtype=np.float64)
    if cosine:
        x64 = x64 / np.linalg.norm(x64, axis=1, keepdims=True)
        y64 = y64 / np.linalg.norm(y64, axis=1, keepdims=True)
    rows, dist = brute_force_knn_f64(x64, y64, ptr_x, ptr_y, k)
    e = np.asarray(edges)
    m = len(y64)
    counts = np.bincount(e[0], minlength=m)
    expect_counts = (rows >= 0).sum(1)
    assert (counts == expect_counts).all(), "per-query neighbour counts differ"
    assert (np.diff(e[0]) >= 0).all(), "edges are not grouped by query"
    starts = np.concatenate([[0], np.cumsum(counts)])
    bad = 0
    for q in range(m):
        got = e[1, starts[q]:starts[q + 1]]
        want = rows[q, :expect_counts[q]]
        if set(got.tolist()) == set(want.tolist()):
            continue
        # every returned neighbour must be within tolerance of the k-th
        # exact distance
        kth = dist[q, expect_counts[q] - 1]
        dg = ((x64[got] - y64[q]) ** 2).sum(-1)
        assert (dg <= kth * (1 + rel_tie) + 1e-30).all(), (
            "query %d returned a neighbour beyond the k-th distance" % q)
        bad += 1
    return bad
