"""GPU parity of `nearest` (pca_nearest through the C ABI, the TorchScript
operator and the Python entry point) against the oracle's play-through of the
reference kernel (csrc/cuda/nearest_cuda.cu:10-66).  Row numbers must be
identical, ties and corner rules included."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

import pytorch_cluster_amd as pca  # noqa: E402
from pytorch_cluster_amd import capi  # noqa: E402
from gpu_common import DEV, dev, ragged_ptrs  # noqa: E402

TORCH_DTYPE = {np.float32: torch.float32, np.float64: torch.float64,
               np.float16: torch.float16}


def gpu_nearest(x, y, ptr_x, ptr_y):
    out = capi.nearest_rows(dev(x), dev(y), dev(ptr_x, torch.long),
                            dev(ptr_y, torch.long))
    torch.cuda.synchronize()
    return out.cpu().numpy()


def matched_ptrs(rng, n, m, segments):
    """Segments of x and y; one segment empty on both sides."""
    if segments == 1:
        return None, None
    ptr_x = ragged_ptrs(rng, n, segments)
    ptr_y = ragged_ptrs(rng, m, segments)
    return ptr_x, ptr_y


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.float16])
@pytest.mark.parametrize("d", [1, 2, 3, 4, 5, 8, 9, 16, 33, 64, 128, 130])
@pytest.mark.parametrize("segments", [1, 5])
def test_random_points(oracle, dtype, d, segments):
    rng = np.random.default_rng(1000 * d + segments)
    n, m = 3000, 2600
    x = rng.standard_normal((n, d)).astype(dtype)
    y = rng.standard_normal((m, d)).astype(dtype)
    ptr_x, ptr_y = matched_ptrs(rng, n, m, segments)
    got = gpu_nearest(x, y, ptr_x, ptr_y)
    px = ptr_x if ptr_x is not None else [0, n]
    py = ptr_y if ptr_y is not None else [0, m]
    want = oracle.nearest_op(x, y, px, py)
    assert (got == want).all()


@pytest.mark.parametrize("dtype,d", [(np.float32, 3), (np.float32, 2),
                                     (np.float32, 8), (np.float32, 12),
                                     (np.float32, 40), (np.float32, 128),
                                     (np.float32, 200),
                                     (np.float64, 3), (np.float16, 3)])
def test_ties_follow_the_reference_block(oracle, dtype, d):
    """Integer grids: exact ties everywhere; candidate segments longer than
    1,024 rows, so the winner is often not the lowest row."""
    rng = np.random.default_rng(7 + d)
    sizes_y = [2500, 0, 1030, 5000]
    sizes_x = [700, 0, 64, 900]
    ptr_y = np.concatenate([[0], np.cumsum(sizes_y)]).astype(np.int64)
    ptr_x = np.concatenate([[0], np.cumsum(sizes_x)]).astype(np.int64)
    if d <= 3:
        y = rng.integers(0, 4, (ptr_y[-1], d)).astype(dtype)
        x = rng.integers(0, 4, (ptr_x[-1], d)).astype(dtype)
    else:  # rows drawn from a small pool: duplicates in any dimension
        pool = rng.integers(0, 3, (48, d)).astype(dtype)
        y = pool[rng.integers(0, 48, ptr_y[-1])]
        x = pool[rng.integers(0, 48, ptr_x[-1])]
    got = gpu_nearest(x, y, ptr_x, ptr_y)
    want = oracle.nearest_op(x, y, ptr_x, ptr_y)
    assert (got == want).all()
    # duplicates of the winner exist at lower rows for many of them
    first = np.array([np.flatnonzero((y == y[w]).all(1))[0] for w in want])
    assert (first != want).any()


@pytest.mark.parametrize("slices", [1, 3])
def test_sliced_candidates(oracle, monkeypatch, slices):
    """Several slices of a segment's candidates and the merge of their
    results (the slice count is read from the environment at every call)."""
    monkeypatch.setenv("PCA_KNN_SLICES", str(slices))
    rng = np.random.default_rng(21)
    n, m = 1500, 9000
    x = rng.integers(0, 12, (n, 3)).astype(np.float32)
    y = rng.integers(0, 12, (m, 3)).astype(np.float32)
    ptr_x = np.array([0, 600, 600, 1500], dtype=np.int64)
    ptr_y = np.array([0, 5000, 5000, 9000], dtype=np.int64)
    got = gpu_nearest(x, y, ptr_x, ptr_y)
    assert (got == oracle.nearest_op(x, y, ptr_x, ptr_y)).all()


def test_limit_nan_and_empty_candidates(oracle):
    # float32, matrix-core kernel (d = 3) and any-dimension kernel (d = 9)
    for d in (3, 9):
        y = np.zeros((6, d), dtype=np.float32)
        y[0, 0], y[1, 0], y[2, 0], y[3, 0] = 3e19, np.inf, np.nan, 9e18
        y[4, 0], y[5, 0] = -2.5e19, 1e30
        x = np.zeros((4, d), dtype=np.float32)
        x[0, 0], x[2, 0], x[3, 0] = -3e19, np.nan, 2e19
        ptr_x = np.array([0, 4, 4], dtype=np.int64)
        ptr_y = np.array([0, 6, 6], dtype=np.int64)
        got = gpu_nearest(x, y, ptr_x, ptr_y)
        want = oracle.nearest_op(x, y, ptr_x, ptr_y)
        assert (got == want).all(), (d, got, want)
        assert got[2] == 0  # a NaN row finds nothing: index 0
    # rows whose segment of y is empty get 0; so does everything when y is
    x = np.random.default_rng(0).standard_normal((300, 3)).astype(np.float32)
    y = x[:40].copy()
    ptr_x = np.array([0, 100, 300], dtype=np.int64)
    ptr_y = np.array([0, 40, 40], dtype=np.int64)
    got = gpu_nearest(x, y, ptr_x, ptr_y)
    assert (got == oracle.nearest_op(x, y, ptr_x, ptr_y)).all()
    assert (got[100:] == 0).all()
    none = capi.nearest_rows(dev(x), torch.empty(0, 3, device=DEV))
    assert (none.cpu().numpy() == 0).all()
    assert capi.nearest_rows(torch.empty(0, 3, device=DEV), dev(y)).numel() == 0
    # fp16: the limit is +inf
    y16 = np.array([[60000.0], [300.0]], dtype=np.float16)
    x16 = np.array([[-60000.0], [100.0]], dtype=np.float16)
    assert gpu_nearest(x16, y16, None, None).tolist() == [0, 1]
    assert gpu_nearest(x16[:1], y16[:1], None, None).tolist() == [0]


@pytest.mark.parametrize("d", [3, 32])
def test_far_apart_clusters(oracle, d):
    """Squared distances beyond 1e10 (the kNN limit) are ordinary here."""
    rng = np.random.default_rng(3)
    y = (rng.standard_normal((4000, d)) * 10 + 5e6).astype(np.float32)
    x = (rng.standard_normal((2500, d)) * 10).astype(np.float32)
    got = gpu_nearest(x, y, None, None)
    assert (got == oracle.nearest_op(x, y, [0, 2500], [0, 4000])).all()


def test_codebook_assignment_in_feature_space(oracle):
    """20,000 feature rows of 64 components to the nearest of 4,096 code
    vectors, several slices of the code book (matrix-core kernel, merge)."""
    rng = np.random.default_rng(12)
    y = rng.standard_normal((4096 * 5, 64)).astype(np.float32)
    x = (y[rng.integers(0, len(y), 20000)]
         + 0.3 * rng.standard_normal((20000, 64))).astype(np.float32)
    got = gpu_nearest(x, y, None, None)
    assert (got == oracle.nearest_op(x, y, [0, len(x)], [0, len(y)])).all()


def _filter_cases():
    """Inputs for the feature-space search: random rows, exact ties beyond
    1,024 candidates, the limits, far-apart clusters, a code book with exact
    duplicates, segments without rows on either side."""
    for d in (9, 16, 33, 64, 128):
        for segments in (1, 5):
            rng = np.random.default_rng(1000 * d + segments)
            n, m = 3000, 2600
            x = rng.standard_normal((n, d)).astype(np.float32)
            y = rng.standard_normal((m, d)).astype(np.float32)
            ptr_x, ptr_y = matched_ptrs(rng, n, m, segments)
            yield "random d=%d segments=%d" % (d, segments), x, y, ptr_x, ptr_y
    for d in (12, 40, 128):
        rng = np.random.default_rng(7 + d)
        ptr_y = np.array([0, 2500, 2500, 3530, 8530], dtype=np.int64)
        ptr_x = np.array([0, 700, 700, 764, 1664], dtype=np.int64)
        pool = rng.integers(0, 3, (48, d)).astype(np.float32)
        y = pool[rng.integers(0, 48, ptr_y[-1])]
        x = pool[rng.integers(0, 48, ptr_x[-1])]
        yield "ties d=%d" % d, x, y, ptr_x, ptr_y
    y = np.zeros((6, 9), dtype=np.float32)
    y[0, 0], y[1, 0], y[2, 0], y[3, 0] = 3e19, np.inf, np.nan, 9e18
    y[4, 0], y[5, 0] = -2.5e19, 1e30
    x = np.zeros((4, 9), dtype=np.float32)
    x[0, 0], x[2, 0], x[3, 0] = -3e19, np.nan, 2e19
    yield ("limits", x, y, np.array([0, 4, 4], dtype=np.int64),
           np.array([0, 6, 6], dtype=np.int64))
    rng = np.random.default_rng(3)
    y = (rng.standard_normal((4000, 32)) * 10 + 5e6).astype(np.float32)
    x = (rng.standard_normal((2500, 32)) * 10).astype(np.float32)
    yield "far apart", x, y, None, None
    # one far cluster among near ones: distances on both sides of 1e10
    y = np.concatenate([y[:100], (rng.standard_normal((300, 32))).astype(
        np.float32)])
    x = np.concatenate([x[:200], (rng.standard_normal((200, 32)) * 10
                                  + 5e6).astype(np.float32)])
    yield "near and far", x, y, None, None
    rng = np.random.default_rng(12)
    y = rng.standard_normal((4096 * 5, 64)).astype(np.float32)
    y[1::7] = y[0::7][:len(y[1::7])]  # exact duplicates in the code book
    x = (y[rng.integers(0, len(y), 20000)]
         + 0.3 * rng.standard_normal((20000, 64))).astype(np.float32)
    x[::3] = y[rng.integers(0, len(y), len(x[::3]))]  # rows that ARE codes
    yield "code book", x, y, None, None
    # a query segment without candidates, and the other way round
    rng = np.random.default_rng(5)
    x = rng.standard_normal((700, 24)).astype(np.float32)
    y = rng.standard_normal((900, 24)).astype(np.float32)
    yield ("empty segments", x, y, np.array([0, 300, 300, 700], dtype=np.int64),
           np.array([0, 0, 500, 900], dtype=np.int64))


def test_feature_space_cases_agree_with_the_oracle(oracle):
    """The matrix-core search of fp32 rows, 8 < d <= 128, on inputs that
    stress its first bound (taken from one row per lane of the first step),
    its filter near ties and the limits."""
    for name, x, y, ptr_x, ptr_y in _filter_cases():
        got = gpu_nearest(x, y, ptr_x, ptr_y)
        px = ptr_x if ptr_x is not None else [0, len(x)]
        py = ptr_y if ptr_y is not None else [0, len(y)]
        want = oracle.nearest_op(x, y, px, py)
        bad = np.flatnonzero(got != want)
        assert bad.size == 0, (name, bad[:5], got[bad[:5]], want[bad[:5]])


def test_first_step_shorter_than_a_tile(oracle):
    """Fewer candidates than the 32 rows of a step, down to one: the first
    bound only looks at rows that exist."""
    rng = np.random.default_rng(77)
    for m in (1, 2, 5, 31, 33):
        y = rng.integers(0, 3, (m, 20)).astype(np.float32)
        x = rng.integers(0, 3, (500, 20)).astype(np.float32)
        got = gpu_nearest(x, y, None, None)
        assert (got == oracle.nearest_op(x, y, [0, 500], [0, m])).all(), m


def test_unsupported_and_invalid():
    x = torch.rand(8, 3, device=DEV).to(torch.bfloat16)
    with pytest.raises(capi.PcaError):
        capi.nearest_rows(x, x)
    with pytest.raises(RuntimeError, match="BFloat16"):
        pca.nearest(x, x)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.float16])
def test_entry_point_fixture(dtype):
    # test/test_nearest.py:11-65 of the reference
    x = torch.tensor([[-1, -1], [-1, +1], [+1, +1], [+1, -1],
                      [-2, -2], [-2, +2], [+2, +2], [+2, -2]],
                     dtype=dtype, device=DEV)
    y = torch.tensor([[-1, 0], [+1, 0], [-2, 0], [+2, 0]], dtype=dtype,
                     device=DEV)
    t = lambda v: torch.tensor(v, device=DEV)
    bx, by = t([0, 0, 0, 0, 1, 1, 1, 1]), t([0, 0, 1, 1])
    out = pca.nearest(x, y, bx, by)
    assert out.dtype == torch.long and out.device == x.device
    assert out.tolist() == [0, 0, 1, 1, 2, 2, 3, 3]
    assert pca.nearest(x, y).tolist() == [0, 0, 1, 1, 2, 2, 3, 3]
    with pytest.raises(ValueError):
        pca.nearest(x, y, bx, t([0, 0, 0, 0]))
    with pytest.raises(ValueError):
        pca.nearest(x, y, bx, batch_y=None)
    with pytest.raises(ValueError):
        pca.nearest(x, y, t([0, 0, 1, 1, 2, 2, 3, 3]), t([0, 1, 3, 3]))
    with pytest.raises(ValueError):
        pca.nearest(x[:7], y, t([0, 0, 1, 0, 0, 0, 0]), by)
    with pytest.raises(ValueError):
        pca.nearest(x, y, bx, t([0, 0, 1, 0]))


def test_operator_flattens_trailing_dimensions(oracle):
    rng = np.random.default_rng(4)
    x = rng.standard_normal((500, 2, 2)).astype(np.float32)
    y = rng.standard_normal((300, 2, 2)).astype(np.float32)
    ptr_x = torch.tensor([0, 500], device=DEV)
    ptr_y = torch.tensor([0, 300], device=DEV)
    got = torch.ops.torch_cluster.nearest(dev(x), dev(y), ptr_x, ptr_y)
    want = oracle.nearest_op(x, y, [0, 500], [0, 300])
    assert (got.cpu().numpy() == want).all()


def test_lidar_scale_assignment(oracle):
    """About a million rows assigned to 130 thousand candidates in 8 ragged
    clouds: a sample of rows against the oracle, every row against the
    properties that do not depend on the size (right segment; no candidate
    of a sampled row is nearer)."""
    g = torch.Generator().manual_seed(0)
    sizes = torch.randint(60000, 200001, (8,), generator=g)
    xs, ys = [], []
    for nb in sizes.tolist():
        pts = torch.randn(nb, 3, generator=g) * torch.tensor([30.0, 30.0, 2.0])
        xs.append(pts)
        ys.append(pts[::8] + 0.01 * torch.randn((nb + 7) // 8, 3, generator=g))
    x, y = torch.cat(xs), torch.cat(ys)
    ptr_x = torch.tensor([0] + [len(a) for a in xs]).cumsum(0)
    ptr_y = torch.tensor([0] + [len(a) for a in ys]).cumsum(0)
    out = capi.nearest_rows(x.to(DEV), y.to(DEV), ptr_x.to(DEV),
                            ptr_y.to(DEV)).cpu()
    seg = torch.bucketize(torch.arange(len(x)), ptr_x[1:], right=True)
    assert ((out >= ptr_y[seg]) & (out < ptr_y[seg + 1])).all()
    rng = np.random.default_rng(0)
    pick = np.sort(rng.choice(len(x), 3000, replace=False))
    # the oracle on the sampled rows: same segments, only those rows of x
    xn, yn = x.numpy(), y.numpy()
    counts = np.bincount(seg.numpy()[pick], minlength=8)
    sub_ptr = np.concatenate([[0], np.cumsum(counts)])
    want = oracle.nearest_op(xn[pick], yn, sub_ptr, ptr_y.numpy())
    assert (out.numpy()[pick] == want).all()
