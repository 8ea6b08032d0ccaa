"""Pins the CPU oracle (oracle/) before anything is checked against it.

Every check here is independent of the oracle's own formulas: the reference's
inline fixtures and README outputs, the reference's compiled CPU operators
(oracle/_ref), scipy's KD-tree as the reference's own large tests use it, and
float64 brute force with a stable argsort.
"""
import numpy as np
import pytest
import scipy.spatial

from helpers import brute_force_knn_f64, to_set

SQUARE2 = np.array([[-1, -1], [-1, +1], [+1, +1], [+1, -1],
                    [-1, -1], [-1, +1], [+1, +1], [+1, -1]], dtype=np.float32)
CORNERS = np.array([[-1, -1], [-1, +1], [+1, +1], [+1, -1]], dtype=np.float32)


# ---- reference fixtures: test/test_knn.py:16-52 ---------------------------

@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_knn_fixture_sets(oracle, dtype):
    x = SQUARE2.astype(dtype)
    y = np.array([[1, 0], [-1, 0]], dtype=dtype)
    bx = np.array([0, 0, 0, 0, 1, 1, 1, 1])
    by = np.array([0, 1])
    assert to_set(oracle.knn(x, y, 2)) == {(0, 2), (0, 3), (1, 0), (1, 1)}
    assert to_set(oracle.knn(x, y, 2, bx, by)) == \
        {(0, 2), (0, 3), (1, 4), (1, 5)}
    assert to_set(oracle.knn(x, y, 2, bx, by, cosine=True)) == \
        {(0, 2), (0, 3), (1, 4), (1, 5)}
    # skipping a batch id (test/test_knn.py:48-52)
    bx = np.array([0, 0, 0, 0, 2, 2, 2, 2])
    by = np.array([0, 2])
    assert to_set(oracle.knn(x, y, 2, bx, by)) == \
        {(0, 2), (0, 3), (1, 4), (1, 5)}


# ---- test/test_knn.py:57-75 -----------------------------------------------

def test_knn_graph_fixture_sets(oracle):
    e = oracle.knn_graph(CORNERS, 2, flow="target_to_source")
    assert to_set(e) == {(0, 1), (0, 3), (1, 0), (1, 2), (2, 1), (2, 3),
                         (3, 0), (3, 2)}
    e = oracle.knn_graph(CORNERS, 2, flow="source_to_target")
    assert to_set(e) == {(1, 0), (3, 0), (0, 1), (2, 1), (1, 2), (3, 2),
                         (0, 3), (2, 3)}


# ---- README.md:178-191, 207-220: ordered outputs ---------------------------

def test_readme_ordered_outputs(oracle):
    x = np.array([[-1., -1.], [-1., 1.], [1., -1.], [1., 1.]],
                 dtype=np.float32)
    batch = np.zeros(4, dtype=np.int64)
    want = [[1, 2, 0, 3, 0, 3, 1, 2], [0, 0, 1, 1, 2, 2, 3, 3]]
    assert oracle.knn_graph(x, 2, batch, loop=False).tolist() == want
    assert oracle.radius_graph(x, 2.5, batch, loop=False).tolist() == want


# ---- test/test_radius.py:25-61 ----------------------------------------------

@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_radius_fixture_sets(oracle, dtype):
    x = SQUARE2.astype(dtype)
    y = np.array([[0, 0], [0, 1]], dtype=dtype)
    bx = np.array([0, 0, 0, 0, 1, 1, 1, 1])
    by = np.array([0, 1])
    assert to_set(oracle.radius(x, y, 2, max_num_neighbors=4)) == \
        {(0, 0), (0, 1), (0, 2), (0, 3), (1, 1), (1, 2), (1, 5), (1, 6)}
    assert to_set(oracle.radius(x, y, 2, bx, by, max_num_neighbors=4)) == \
        {(0, 0), (0, 1), (0, 2), (0, 3), (1, 5), (1, 6)}
    bx = np.array([0, 0, 0, 0, 2, 2, 2, 2])
    by = np.array([0, 2])
    assert to_set(oracle.radius(x, y, 2, bx, by, max_num_neighbors=4)) == \
        {(0, 0), (0, 1), (0, 2), (0, 3), (1, 5), (1, 6)}


# ---- test/test_radius.py:66-116 ---------------------------------------------

def test_radius_graph_fixtures(oracle):
    e = oracle.radius_graph(CORNERS, 2.5, flow="target_to_source")
    assert to_set(e) == {(0, 1), (0, 3), (1, 0), (1, 2), (2, 1), (2, 3),
                         (3, 0), (3, 2)}
    e = oracle.radius_graph(CORNERS, 2.5, flow="source_to_target")
    assert to_set(e) == {(1, 0), (3, 0), (0, 1), (2, 1), (1, 2), (3, 2),
                         (0, 3), (2, 3)}

    def degrees(e):
        return set(np.unique(e[1], return_counts=True)[1].tolist())

    e = oracle.radius_graph(CORNERS, 100, max_num_neighbors=1)
    assert degrees(e) == {1}
    same = np.full((4, 2), -1, dtype=np.float32)
    e = oracle.radius_graph(same, 100, max_num_neighbors=1)
    assert degrees(e) == {1}
    batch = np.array([0, 0, 0, 0, 1, 1, 1, 1])
    e = oracle.radius_graph(SQUARE2, 100, batch, max_num_neighbors=1)
    assert degrees(e) == {1}
    assert [i // 4 for i in e[0].tolist()] == batch.tolist()


# ---- scipy cross-checks: test/test_knn.py:78-88, test/test_radius.py:119-133

def test_knn_graph_large_vs_ckdtree(oracle):
    rng = np.random.default_rng(12345)
    x = rng.standard_normal((1000, 3)).astype(np.float32)
    e = oracle.knn_graph(x, 5, flow="target_to_source", loop=True)
    _, col = scipy.spatial.cKDTree(x).query(x, k=5)
    truth = {(i, j) for i, ns in enumerate(col) for j in ns}
    assert to_set(e) == truth


def test_radius_graph_large_vs_ckdtree(oracle):
    rng = np.random.default_rng(54321)
    x = rng.standard_normal((1000, 3)).astype(np.float32)
    e = oracle.radius_graph(x, 0.5, flow="target_to_source", loop=True,
                            max_num_neighbors=2000)
    col = scipy.spatial.cKDTree(x).query_ball_point(x, r=0.5)
    truth = {(i, j) for i, ns in enumerate(col) for j in ns}
    assert to_set(e) == truth


# ---- float64 brute force: order, ties, k > segment size --------------------

@pytest.mark.parametrize("fma_mode", [0, 1])
@pytest.mark.parametrize("d", [1, 2, 3, 5, 16])
def test_knn_matches_stable_brute_force(oracle, fma_mode, d):
    rng = np.random.default_rng(d)
    # coordinates on a coarse grid: many exact distance ties, all sums exact
    # in float32, so the float32 oracle must equal float64 brute force exactly
    # (including the ascending-row tie order)
    x = rng.integers(0, 6, (300, d)).astype(np.float32)
    y = rng.integers(0, 6, (70, d)).astype(np.float32)
    ptr_x = np.array([0, 100, 100, 103, 300])
    ptr_y = np.array([0, 20, 35, 50, 70])
    k = 7
    _, col, dist = oracle.knn_dense(x, y, ptr_x, ptr_y, k, fma_mode=fma_mode)
    rows, d2 = brute_force_knn_f64(x, y, ptr_x, ptr_y, k)
    assert (col == rows).all()
    valid = rows >= 0
    assert (dist[valid] == d2[valid]).all()
    # segment 1 has no x rows, segment 2 has 3 < k
    assert (col[20:35] == -1).all()
    assert ((col[35:50] >= 0).sum(1) == 3).all()


def test_knn_sentinel_drops_far_candidates(oracle):
    # squared distance >= 1e10 is never returned (csrc/cuda/knn_cuda.cu:48,68)
    x = np.array([[0.0], [1.0], [2e5]], dtype=np.float32)
    y = np.array([[0.0]], dtype=np.float32)
    e = oracle.knn_op(x, y, None, None, 3)
    assert e.tolist() == [[0, 0], [0, 1]]


def test_knn_k_limit(oracle):
    x = np.zeros((4, 2), dtype=np.float32)
    with pytest.raises(RuntimeError, match="smaller than or equal to 100"):
        oracle.knn_op(x, x, None, None, 101)


def test_cosine_equals_euclidean_on_normalised_rows(oracle):
    # closed form: for unit vectors |a-b|^2 = 2 (1 - a.b), so the cosine
    # ranking of raw rows is the Euclidean ranking of the normalised rows
    rng = np.random.default_rng(7)
    x = rng.standard_normal((400, 6))
    y = rng.standard_normal((50, 6))
    xn = x / np.linalg.norm(x, axis=1, keepdims=True)
    yn = y / np.linalg.norm(y, axis=1, keepdims=True)
    got = oracle.knn_op(x, y, None, None, 9, cosine=True)
    rows, _ = brute_force_knn_f64(xn, yn, None, None, 9)
    assert (got[1].reshape(50, 9) == rows).all()


@pytest.mark.parametrize("ignore_same", [False, True])
def test_radius_first_m_in_row_order(oracle, ignore_same):
    # CUDA rule (csrc/cuda/radius_cuda.cu:26-41): the first max_num_neighbors
    # hits in ascending x row order, self excluded before counting
    rng = np.random.default_rng(3)
    x = rng.random((500, 3)).astype(np.float32)
    ptr = np.array([0, 200, 200, 500])
    r, cap = 0.3, 5
    e = oracle.radius_op(x, x, ptr, ptr, r, cap,
                         ignore_same_index=ignore_same)
    r2 = np.float32(float(r) * float(r))
    want = []
    for b in range(3):
        for q in range(ptr[b], ptr[b + 1]):
            hits = 0
            for j in range(ptr[b], ptr[b + 1]):
                d = np.float32(0)
                for c in range(3):
                    t = np.float32(x[j, c] - x[q, c])
                    d = np.float32(np.float64(t) * np.float64(t)
                                   + np.float64(d))  # one rounding = fma
                if d < r2 and not (ignore_same and j == q):
                    want.append((q, j))
                    hits += 1
                    if hits >= cap:
                        break
    assert list(zip(e[0].tolist(), e[1].tolist())) == want


# ---- the reference's own CPU operators (oracle/_ref) -----------------------

def test_ref_knn_identical_on_uniform_clouds(ref):
    rng = np.random.default_rng(0)
    x = rng.random((4 * 2048, 3), dtype=np.float32)
    ptr = np.arange(5) * 2048
    ours = ref.knn_op(x, x, ptr, ptr, 17, fma_mode=0)
    theirs = ref.ref_knn(x, x, ptr, ptr, 17)
    # no exact ties in continuous data: same edges in the same order
    assert (ours == theirs).all()
    # fused arithmetic may only reorder neighbours that tie within rounding
    fused = ref.knn_op(x, x, ptr, ptr, 17, fma_mode=1)
    assert fused.shape == theirs.shape
    diff = (fused != theirs).any(0)
    assert diff.mean() < 1e-3


def test_ref_knn_small_segments_and_empty(ref):
    rng = np.random.default_rng(1)
    x = rng.random((40, 2), dtype=np.float32)
    y = rng.random((9, 2), dtype=np.float32)
    ptr_x = np.array([0, 3, 3, 40])
    ptr_y = np.array([0, 4, 6, 9])
    ours = ref.knn_op(x, y, ptr_x, ptr_y, 5, fma_mode=0)
    theirs = ref.ref_knn(x, y, ptr_x, ptr_y, 5)
    assert (ours == theirs).all()
    assert np.bincount(ours[0], minlength=9).tolist() == \
        [3, 3, 3, 3, 0, 0, 5, 5, 5]


def test_ref_radius_untruncated_sets_equal(ref):
    rng = np.random.default_rng(2)
    x = rng.random((3000, 3), dtype=np.float32)
    y = rng.random((700, 3), dtype=np.float32)
    ptr_x = np.array([0, 1000, 3000])
    ptr_y = np.array([0, 300, 700])
    ours = ref.radius_op(x, y, ptr_x, ptr_y, 0.1, 3000, fma_mode=0)
    theirs = ref.ref_radius(x, y, ptr_x, ptr_y, 0.1, 3000)
    assert to_set(ours) == to_set(theirs)


def test_ref_radius_truncated_counts_and_subset(ref):
    # the CPU reference keeps a different subset when it truncates (KD-tree
    # visiting order); counts per query agree and both are subsets of the
    # untruncated result
    rng = np.random.default_rng(4)
    x = rng.random((2000, 3), dtype=np.float32)
    ours = ref.radius_op(x, x, None, None, 0.2, 8, ignore_same_index=True,
                         fma_mode=0)
    theirs = ref.ref_radius(x, x, None, None, 0.2, 8, ignore_same_index=True)
    full = to_set(ref.radius_op(x, x, None, None, 0.2, 2000,
                                ignore_same_index=True, fma_mode=0))
    assert (np.bincount(ours[0], minlength=2000) ==
            np.bincount(theirs[0], minlength=2000)).all()
    assert to_set(ours) <= full and to_set(theirs) <= full


# ---- 16-bit element types ---------------------------------------------------

def _bits(t):
    import torch
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


@pytest.mark.parametrize("kind", [0, 1])
def test_16bit_rounding_matches_torch(oracle, kind):
    import torch
    dt = torch.float16 if kind == 0 else torch.bfloat16
    rng = np.random.default_rng(kind)
    vals = np.concatenate(
        [rng.standard_normal(3000).astype(np.float32) * s
         for s in (1e-8, 1e-5, 1e-3, 1, 100, 6e4, 1e5)] +
        [np.array([0, -0.0, np.inf, -np.inf, 65504, 65519.99, 65520, 6.1e-5,
                   5.96e-8, 2.98e-8, 2.9802325e-8, 8.9e-8], dtype=np.float32)])
    want = torch.from_numpy(vals).to(dt).to(torch.float32).numpy()
    got = np.array([oracle.round16(v, kind) for v in vals], dtype=np.float32)
    assert (got.view(np.uint32) == want.view(np.uint32)).all()


@pytest.mark.parametrize("kind", [0, 1])
def test_16bit_knn_matches_torch_scalar_semantics(oracle, kind):
    # independent restatement with torch CPU tensors of the 16-bit type: every
    # elementwise operator rounds once, like c10::Half / c10::BFloat16
    import torch
    dt = torch.float16 if kind == 0 else torch.bfloat16
    g = torch.Generator().manual_seed(kind)
    x = torch.randn(60, 3, generator=g).to(dt)
    y = torch.randn(9, 3, generator=g).to(dt)
    k = 5
    got, dist = oracle.knn_op16(_bits(x), _bits(y), None, None, k, False, kind)
    acc = torch.zeros(9, 60, dtype=dt)
    for c in range(3):
        diff = y[:, None, c] - x[None, :, c]
        acc = acc + diff * diff
    d = acc.to(torch.float32).numpy()
    order = np.argsort(d, axis=1, kind="stable")[:, :k]
    assert (got[1].reshape(9, k) == order).all()
    assert (dist.reshape(9, k) == np.take_along_axis(d, order, 1)).all()
