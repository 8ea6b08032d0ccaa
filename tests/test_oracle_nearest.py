"""Pins of the oracle's `nearest` (a literal play-through of the reference's
block of 1,024 threads, csrc/cuda/nearest_cuda.cu:10-66) and of the Python
entry point's host logic.

What pins it: the reference's fixture and error cases
(test/test_nearest.py:11-65), scipy.cluster.vq.vq (the reference's own route
for CPU tensors, torch_cluster/nearest.py:122-124), float64 brute force on
data without ties, numpy float16 arithmetic for the fp16 operation order, and
a closed form of the tie rule written independently of the play-through:
smallest distance, then smallest (row - segment start) % 1024, then smallest
row.
"""
import numpy as np
import pytest
import scipy.cluster.vq
import torch

import pytorch_cluster_amd as pca

X_FIX = [[-1, -1], [-1, +1], [+1, +1], [+1, -1],
         [-2, -2], [-2, +2], [+2, +2], [+2, -2]]
Y_FIX = [[-1, 0], [+1, 0], [-2, 0], [+2, 0]]


def closed_form(dist, starts):
    """dist [n, m_seg] distances of one segment's rows (inf/nan = never
    chosen beyond the limit rule), candidates in row order; returns the
    column the reference's block returns, or -1 when no distance is below
    1e38."""
    n, m = dist.shape
    rel = np.arange(m)
    out = np.full(n, -1, dtype=np.int64)
    for i in range(n):
        ok = dist[i] < 1e38
        if not ok.any():
            continue
        dmin = dist[i][ok].min()
        cand = rel[ok & (dist[i] == dmin)]
        slot = cand % 1024
        best = cand[slot == slot.min()].min()
        out[i] = best
    return out


def expected_rows(x, y, ptr_x, ptr_y, dist_fn):
    out = np.zeros(len(x), dtype=np.int64)
    for b in range(len(ptr_x) - 1):
        xs, xe, ys, ye = ptr_x[b], ptr_x[b + 1], ptr_y[b], ptr_y[b + 1]
        if xs == xe:
            continue
        if ys == ye:
            out[xs:xe] = 0
            continue
        col = closed_form(dist_fn(x[xs:xe], y[ys:ye]), None)
        out[xs:xe] = np.where(col >= 0, col + ys, 0)
    return out


def dist_f32_fma(xq, yc):
    """float32 chain of fused multiply-adds, emulated in float64 (a product
    of two float32 numbers is exact in float64; the sum rounds once more,
    which the test data -- small integers -- never notices)."""
    d = np.zeros((len(xq), len(yc)), dtype=np.float32)
    for c in range(xq.shape[1]):
        diff = (xq[:, None, c] - yc[None, :, c]).astype(np.float32)
        d = (diff.astype(np.float64) ** 2 + d.astype(np.float64)).astype(
            np.float32)
    return d


def dist_f16(xq, yc):
    """c10::Half arithmetic == numpy float16 arithmetic: every operation
    rounds to 16 bits."""
    d = np.zeros((len(xq), len(yc)), dtype=np.float16)
    with np.errstate(over="ignore", invalid="ignore"):
        for c in range(xq.shape[1]):
            diff = xq[:, None, c] - yc[None, :, c]
            d = d + diff * diff
    return d.astype(np.float64)


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.float16])
def test_reference_fixture(oracle, dtype):
    x = np.array(X_FIX, dtype=dtype)
    y = np.array(Y_FIX, dtype=dtype)
    bx = [0, 0, 0, 0, 1, 1, 1, 1]
    by = [0, 0, 1, 1]
    assert oracle.nearest(x, y, bx, by).tolist() == [0, 0, 1, 1, 2, 2, 3, 3]
    assert oracle.nearest(x, y).tolist() == [0, 0, 1, 1, 2, 2, 3, 3]


def _error_cases(fn, x, y):
    # test/test_nearest.py:37-65
    with pytest.raises(ValueError):
        fn(x, y, [0, 0, 0, 0, 1, 1, 1, 1], [0, 0, 0, 0])
    with pytest.raises(ValueError):
        fn(x, y, [0, 0, 0, 0, 1, 1, 1, 1], None)
    with pytest.raises(ValueError):
        fn(x, y, [0, 0, 1, 1, 2, 2, 3, 3], [0, 1, 3, 3])
    with pytest.raises(ValueError):
        fn(x[:7], y, [0, 0, 1, 0, 0, 0, 0], [0, 0, 1, 1])
    with pytest.raises(ValueError):
        fn(x, y, [0, 0, 0, 0, 1, 1, 1, 1], [0, 0, 1, 0])


def test_reference_error_cases(oracle):
    _error_cases(oracle.nearest, np.array(X_FIX, dtype=np.float32),
                 np.array(Y_FIX, dtype=np.float32))


@pytest.mark.parametrize("d", [1, 2, 3, 7, 33])
def test_matches_vq_and_float64_brute_force(oracle, d):
    rng = np.random.default_rng(d)
    x = rng.standard_normal((700, d))
    y = rng.standard_normal((1500, d))  # more than 1,024 candidates
    code, _ = scipy.cluster.vq.vq(x, y)
    got = oracle.nearest(x, y)
    assert (got == code).all()
    d2 = ((x[:, None, :] - y[None, :, :]) ** 2).sum(-1)
    assert (got == d2.argmin(1)).all()
    got32 = oracle.nearest(x.astype(np.float32), y.astype(np.float32))
    # float32 rounding may flip near-ties only
    flipped = got32 != got
    assert flipped.mean() < 0.01
    rows = np.arange(len(x))
    assert np.allclose(d2[rows, got32], d2[rows, got], rtol=1e-5)


def test_segments_and_empty_candidates(oracle):
    rng = np.random.default_rng(5)
    x = rng.standard_normal((50, 3)).astype(np.float32)
    y = rng.standard_normal((40, 3)).astype(np.float32)
    ptr_x = np.array([0, 10, 10, 30, 50])
    ptr_y = np.array([0, 15, 20, 20, 40])  # example 2: rows in x, none in y
    got = oracle.nearest_op(x, y, ptr_x, ptr_y)
    for b in (0, 3):
        xs, xe, ys, ye = ptr_x[b], ptr_x[b + 1], ptr_y[b], ptr_y[b + 1]
        d2 = ((x[xs:xe, None, :].astype(np.float64)
               - y[None, ys:ye, :]) ** 2).sum(-1)
        assert (got[xs:xe] == d2.argmin(1) + ys).all()
    # `best_idx` starts at 0 (csrc/cuda/nearest_cuda.cu:32)
    assert (got[10:30] == 0).all()


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.float16])
def test_tie_rule_is_the_blocks(oracle, dtype):
    """Integer grids: exact ties everywhere, candidate segments longer than
    one pass of the 1,024 threads."""
    rng = np.random.default_rng(11)
    sizes_y = [2500, 0, 1030, 3000]
    sizes_x = [120, 0, 64, 200]
    ptr_y = np.concatenate([[0], np.cumsum(sizes_y)])
    ptr_x = np.concatenate([[0], np.cumsum(sizes_x)])
    y = rng.integers(0, 4, (ptr_y[-1], 3)).astype(dtype)
    x = rng.integers(0, 4, (ptr_x[-1], 3)).astype(dtype)
    got = oracle.nearest_op(x, y, ptr_x, ptr_y)
    fn = dist_f16 if dtype == np.float16 else dist_f32_fma
    want = expected_rows(x, y, ptr_x, ptr_y, fn)
    assert (got == want).all()
    # the rule differs from "lowest row": the test must see that
    lowest = np.zeros(len(x), dtype=np.int64)
    for b in (0, 2, 3):
        xs, xe, ys, ye = ptr_x[b], ptr_x[b + 1], ptr_y[b], ptr_y[b + 1]
        lowest[xs:xe] = fn(x[xs:xe], y[ys:ye]).argmin(1) + ys
    assert (got != lowest).any()


def test_limit_and_nan(oracle):
    # float32: distances of 1e38 and more, inf and NaN are never taken
    y = np.array([[3e19, 0, 0], [np.inf, 0, 0], [np.nan, 0, 0], [9e18, 0, 0]],
                 dtype=np.float32)
    x = np.array([[-3e19, 0, 0], [0, 0, 0]], dtype=np.float32)
    got = oracle.nearest_op(x, np.concatenate([np.ones((2, 3), np.float32), y]),
                            [0, 2], [0, 6])
    # row 0: candidates 0, 1 at ~9e38 (inf in float32? no: 9e38 overflows)
    assert got.tolist()[1] == 0  # (1,1,1) is nearest to the origin
    far = oracle.nearest_op(x[:1], y[:3], [0, 1], [0, 3])
    assert far.tolist() == [0]  # nothing below 1e38: index 0
    ok = oracle.nearest_op(x[1:], y, [0, 1], [0, 4])
    assert ok.tolist() == [3]  # 8.1e37 < 1e38 <= 9e38
    # fp16: the limit is +inf, overflowing distances are not taken
    y16 = np.array([[60000.0], [300.0]], dtype=np.float16)
    x16 = np.array([[-60000.0], [100.0]], dtype=np.float16)
    assert oracle.nearest_op(x16, y16, [0, 2], [0, 2]).tolist() == [0, 1]
    assert oracle.nearest_op(x16[:1], y16[:1], [0, 1], [0, 1]).tolist() == [0]


def test_fp16_operation_order(oracle):
    rng = np.random.default_rng(2)
    x = (rng.standard_normal((300, 5)) * 3).astype(np.float16)
    y = (rng.standard_normal((1200, 5)) * 3).astype(np.float16)
    ptr = np.array([0, 300]), np.array([0, 1200])
    got = oracle.nearest_op(x, y, *ptr)
    want = expected_rows(x, y, ptr[0], ptr[1], dist_f16)
    assert (got == want).all()


# ---- host logic of the Python entry point, operator replaced by the oracle --

@pytest.fixture
def oracle_nearest_op(monkeypatch, oracle):
    def fake(x, y, ptr_x, ptr_y):
        return torch.from_numpy(oracle.nearest_op(
            x.numpy(), y.numpy(), ptr_x.numpy(), ptr_y.numpy()))
    monkeypatch.setattr(torch.ops.torch_cluster, "nearest", fake)


def test_wrapper_fixture_and_errors(oracle_nearest_op):
    x = torch.tensor(X_FIX, dtype=torch.float)
    y = torch.tensor(Y_FIX, dtype=torch.float)
    bx = torch.tensor([0, 0, 0, 0, 1, 1, 1, 1])
    by = torch.tensor([0, 0, 1, 1])
    assert pca.nearest(x, y, bx, by).tolist() == [0, 0, 1, 1, 2, 2, 3, 3]
    assert pca.nearest(x, y).tolist() == [0, 0, 1, 1, 2, 2, 3, 3]

    def fn(x, y, bx, by):
        t = lambda b: None if b is None else torch.tensor(b)
        return pca.nearest(x, y, t(bx), t(by))
    _error_cases(fn, x, y)


def test_wrapper_matches_oracle_entry_point(oracle_nearest_op, oracle):
    rng = np.random.default_rng(9)
    x = rng.standard_normal((200, 3)).astype(np.float32)
    y = rng.standard_normal((90, 3)).astype(np.float32)
    bx = np.sort(rng.integers(0, 4, 200))
    by = np.sort(np.concatenate([np.arange(4), rng.integers(0, 4, 86)]))
    got = pca.nearest(torch.from_numpy(x), torch.from_numpy(y),
                      torch.from_numpy(bx), torch.from_numpy(by))
    assert (got.numpy() == oracle.nearest(x, y, bx, by)).all()
    # one-dimensional inputs are columns
    g1 = pca.nearest(torch.from_numpy(x[:, 0].copy()),
                     torch.from_numpy(y[:, 0].copy()))
    assert (g1.numpy() == oracle.nearest(x[:, 0], y[:, 0])).all()


def test_cpu_tensors_are_searched_on_the_host():
    x = torch.rand(8, 3)
    assert pca.nearest(x, x).tolist() == list(range(8))
    schema = str(torch.ops.torch_cluster.nearest.default._schema)
    assert "Tensor ptr_x, Tensor ptr_y" in schema
