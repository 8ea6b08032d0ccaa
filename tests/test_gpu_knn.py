"""GPU parity of the kNN path against the CPU oracle, through the C ABI and
through the registered operator / Python entry points.

Bar: integer outputs (edge indices, counts, order) bit-exact against the
oracle evaluated with fused multiply-adds (the arithmetic the kernels use);
distances bit-exact as well.  Against float64 brute force the neighbour sets
may differ only where distances tie within 1e-6 relative.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

import pytorch_cluster_amd as pca  # noqa: E402
from pytorch_cluster_amd import capi, testing  # noqa: E402
from gpu_common import (use_strategy, DEV, dev, gpu_knn, oracle_knn_edges,  # noqa: E402
                        ragged_ptrs)
from helpers import (brute_force_knn_f64, check_knn_against_exact,  # noqa
                     stable_seed, to_set)


def tensor(v, dtype=torch.float32):
    return torch.tensor(v, dtype=dtype, device=DEV)


# ---- the reference's fixtures (test/test_knn.py:16-75, README.md:188-191) --

def test_reference_fixtures():
    x = tensor([[-1, -1], [-1, +1], [+1, +1], [+1, -1],
                [-1, -1], [-1, +1], [+1, +1], [+1, -1]])
    y = tensor([[1, 0], [-1, 0]])
    batch_x = tensor([0, 0, 0, 0, 1, 1, 1, 1], torch.long)
    batch_y = tensor([0, 1], torch.long)

    e = pca.knn(x, y, 2)
    assert to_set(e.cpu()) == {(0, 2), (0, 3), (1, 0), (1, 1)}
    jit = torch.jit.script(pca.knn)
    assert to_set(jit(x, y, 2).cpu()) == {(0, 2), (0, 3), (1, 0), (1, 1)}
    e = pca.knn(x, y, 2, batch_x, batch_y)
    assert to_set(e.cpu()) == {(0, 2), (0, 3), (1, 4), (1, 5)}
    e = pca.knn(x, y, 2, batch_x, batch_y, cosine=True)
    assert to_set(e.cpu()) == {(0, 2), (0, 3), (1, 4), (1, 5)}
    batch_x = tensor([0, 0, 0, 0, 2, 2, 2, 2], torch.long)
    batch_y = tensor([0, 2], torch.long)
    e = pca.knn(x, y, 2, batch_x, batch_y)
    assert to_set(e.cpu()) == {(0, 2), (0, 3), (1, 4), (1, 5)}
    assert e.dtype == torch.long and e.is_cuda and e.is_contiguous()


def test_reference_knn_graph_fixtures():
    x = tensor([[-1, -1], [-1, +1], [+1, +1], [+1, -1]])
    e = pca.knn_graph(x, k=2, flow='target_to_source')
    assert to_set(e.cpu()) == {(0, 1), (0, 3), (1, 0), (1, 2), (2, 1), (2, 3),
                               (3, 0), (3, 2)}
    e = pca.knn_graph(x, k=2, flow='source_to_target')
    assert to_set(e.cpu()) == {(1, 0), (3, 0), (0, 1), (2, 1), (1, 2), (3, 2),
                               (0, 3), (2, 3)}
    jit = torch.jit.script(pca.knn_graph)
    e = jit(x, k=2, flow='source_to_target')
    assert to_set(e.cpu()) == {(1, 0), (3, 0), (0, 1), (2, 1), (1, 2), (3, 2),
                               (0, 3), (2, 3)}
    x = tensor([[-1., -1.], [-1., 1.], [1., -1.], [1., 1.]])
    batch = tensor([0, 0, 0, 0], torch.long)
    e = pca.knn_graph(x, k=2, batch=batch, loop=False)
    assert e.tolist() == [[1, 2, 0, 3, 0, 3, 1, 2], [0, 0, 1, 1, 2, 2, 3, 3]]


def test_knn_graph_large_vs_ckdtree():
    # test/test_knn.py:78-88
    import scipy.spatial
    g = torch.Generator().manual_seed(3)
    x = torch.randn(1000, 3, generator=g)
    e = pca.knn_graph(x.to(DEV), k=5, flow='target_to_source', loop=True)
    _, col = scipy.spatial.cKDTree(x.numpy()).query(x.numpy(), k=5)
    truth = {(i, j) for i, ns in enumerate(col) for j in ns}
    assert to_set(e.cpu()) == truth


# ---- bit-exact parity against the oracle -----------------------------------

@pytest.fixture(params=["1", "0"], ids=["matrix_cores", "vector_alu"])
def lowd_path(request, monkeypatch):
    # both low-dimensional Euclidean kernels (lists of more than 32 entries
    # and the cosine distance always run on the vector-ALU kernel)
    monkeypatch.setenv("PCA_KNN_LOWD_MATRIX_CORES", request.param)
    return request.param


@pytest.mark.parametrize("d", [1, 2, 3, 4, 5, 8])
@pytest.mark.parametrize("k", [1, 7, 16, 17, 32, 33, 64, 100])
def test_parity_single_segment(oracle, lowd_path, d, k):
    rng = np.random.default_rng(100 * d + k)
    n = int(rng.choice([1023, 1024, 1025, 2500]))
    m = int(rng.choice([255, 256, 257, 700]))
    x = rng.random((n, d), dtype=np.float32)
    y = rng.random((m, d), dtype=np.float32)
    got, gd = gpu_knn(x, y, None, None, k)
    want, wd = oracle_knn_edges(oracle, x, y, None, None, k)
    assert got.shape == want.shape
    assert (got == want).all()
    assert (gd == wd).all()


@pytest.mark.parametrize("d,k,segments", [(3, 5, 2), (3, 21, 16), (2, 16, 7),
                                          (4, 9, 33), (8, 24, 5), (3, 48, 3)])
def test_parity_ragged_segments(oracle, lowd_path, d, k, segments):
    rng = np.random.default_rng(d * 1000 + k * 10 + segments)
    n, m = 6000, 1900
    x = rng.standard_normal((n, d)).astype(np.float32)
    y = rng.standard_normal((m, d)).astype(np.float32)
    ptr_x = ragged_ptrs(rng, n, segments)
    ptr_y = ragged_ptrs(rng, m, segments)
    got, gd = gpu_knn(x, y, ptr_x, ptr_y, k)
    want, wd = oracle_knn_edges(oracle, x, y, ptr_x, ptr_y, k)
    assert got.shape == want.shape
    assert (got == want).all()
    assert (gd == wd).all()


def test_k_larger_than_segment_and_empty_segments(oracle, lowd_path):
    rng = np.random.default_rng(5)
    x = rng.random((40, 3), dtype=np.float32)
    y = rng.random((600, 3), dtype=np.float32)
    ptr_x = np.array([0, 3, 3, 40, 40])
    ptr_y = np.array([0, 300, 310, 599, 600])
    got, _ = gpu_knn(x, y, ptr_x, ptr_y, 5)
    want, _ = oracle_knn_edges(oracle, x, y, ptr_x, ptr_y, 5)
    assert (got == want).all()
    counts = np.bincount(got[0], minlength=600)
    assert (counts[:300] == 3).all() and (counts[300:310] == 0).all()
    assert (counts[310:599] == 5).all() and counts[599] == 0


def test_exact_ties_keep_lowest_rows(oracle, lowd_path):
    # integer grid: many exactly equal distances; order must be by
    # (distance, row) -- float64 stable brute force is the independent check
    rng = np.random.default_rng(11)
    x = rng.integers(0, 5, (3000, 3)).astype(np.float32)
    y = rng.integers(0, 5, (500, 3)).astype(np.float32)
    ptr_x = np.array([0, 1000, 3000])
    ptr_y = np.array([0, 200, 500])
    for k in (6, 30):
        got, gd = gpu_knn(x, y, ptr_x, ptr_y, k)
        rows, d2 = brute_force_knn_f64(x, y, ptr_x, ptr_y, k)
        assert (got[1].reshape(500, k) == rows).all()
        assert (gd.reshape(500, k) == d2).all()


@pytest.mark.parametrize("d", [2, 3, 4])
@pytest.mark.parametrize("k", [4, 7, 8, 15, 16, 21, 24, 31, 32])
@pytest.mark.parametrize("case", ["uniform", "grid_ties", "duplicates",
                                  "bad_rows"])
def test_scans_that_start_from_sampled_rows(oracle, d, k, case):
    # unsliced scans over 1-8 LDS tiles of 1,024 rows take their first bound
    # from one exactly evaluated row per 16 (the row the matrix cores rate
    # nearest): whatever the sample, the edges are the checker's
    rng = np.random.default_rng(stable_seed("seeded", d, k, case))
    sizes = [1024, 1500, 4096, 333, 2049]  # (333: too short to sample)
    ptr_x = np.concatenate([[0], np.cumsum(sizes)])
    n = int(ptr_x[-1])
    if case == "uniform":
        x = rng.random((n, d), dtype=np.float32)
    elif case == "grid_ties":
        x = rng.integers(0, 6, (n, d)).astype(np.float32)
    elif case == "duplicates":
        x = rng.random((n, d), dtype=np.float32)
        x[::3] = x[1::3][:len(x[::3])]
        x[ptr_x[2]:ptr_x[2] + 2000] = 0.25
    else:
        x = rng.standard_normal((n, d)).astype(np.float32)
        bad = rng.choice(n, 400, replace=False)
        x[bad[:100], 0] = np.nan
        x[bad[100:200], d - 1] = np.inf
        x[bad[200:300]] = 3e5          # squared distance beyond the limit
        x[bad[300:]] *= 1e19           # norm that is not moderate
    m_sizes = [200, 130, 257, 40, 128]
    ptr_y = np.concatenate([[0], np.cumsum(m_sizes)])
    y = np.concatenate([x[ptr_x[b]:ptr_x[b + 1]][rng.choice(sizes[b], ms)]
                        for b, ms in enumerate(m_sizes)])
    if case == "uniform":
        y = y + rng.random(y.shape, dtype=np.float32) * 0.01
    got, gd = gpu_knn(x, y, ptr_x, ptr_y, k)
    want, wd = oracle_knn_edges(oracle, x, y, ptr_x, ptr_y, k)
    assert got.shape == want.shape
    assert (got == want).all()
    assert (gd == wd).all()


def test_duplicate_points(oracle):
    x = np.zeros((700, 3), dtype=np.float32)
    got, gd = gpu_knn(x, x[:300], None, None, 9)
    assert (got[1].reshape(300, 9) == np.arange(9)).all()
    assert (gd == 0).all()


def test_sentinel_and_nan_candidates(oracle, lowd_path):
    # distance >= 1e10 or NaN is never returned
    # (csrc/cuda/knn_cuda.cu:48,68 in the reference)
    x = np.array([[0.0, 0.0], [1.0, 0.0], [2e5, 0.0], [np.nan, 0.0],
                  [3.0, 0.0], [np.inf, 0.0]], dtype=np.float32)
    y = np.array([[0.0, 0.0], [np.nan, 1.0]], dtype=np.float32)
    got, gd = gpu_knn(x, y, None, None, 5)
    want, wd = oracle_knn_edges(oracle, x, y, None, None, 5)
    assert got.tolist() == want.tolist() == [[0, 0, 0], [0, 1, 4]]
    assert gd.tolist() == [0.0, 1.0, 9.0]


@pytest.mark.parametrize("d,k", [(2, 4), (3, 16), (3, 40), (6, 10)])
def test_cosine_parity(oracle, d, k):
    rng = np.random.default_rng(d + k)
    x = rng.standard_normal((2100, d)).astype(np.float32)
    y = rng.standard_normal((333, d)).astype(np.float32)
    ptr_x = np.array([0, 900, 2100])
    ptr_y = np.array([0, 100, 333])
    got, gd = gpu_knn(x, y, ptr_x, ptr_y, k, cosine=True)
    want, wd = oracle_knn_edges(oracle, x, y, ptr_x, ptr_y, k, cosine=True)
    assert got.shape == want.shape
    assert (got == want).all()
    assert (gd == wd).all()
    # slightly negative cosine distances (x == y up to scale) stay ordered
    got, gd = gpu_knn(x, 3.0 * x[:64], None, None, 3, cosine=True)
    want, wd = oracle_knn_edges(oracle, x, 3.0 * x[:64], None, None, 3,
                                cosine=True)
    assert (got == want).all() and (gd == wd).all()


@pytest.mark.parametrize("d,k,cosine", [(9, 5, False), (16, 16, False),
                                        (17, 33, True), (33, 8, False),
                                        (128, 32, False), (128, 32, True),
                                        (40, 33, False), (128, 48, True),
                                        (100, 50, False), (64, 64, True),
                                        (128, 64, False), (128, 65, False),
                                        (300, 7, False), (515, 3, True)])
@pytest.mark.parametrize("path", ["default", "exact_mfma", "any_dimension",
                                  "any_dimension_sliced"])
def test_parity_high_dimension(oracle, monkeypatch, d, k, cosine, path):
    # default: the fp16 matrix-core filter (up to 512 components); the other
    # kernels of these shapes -- the exact split-bf16 kernel (d <= 128,
    # k <= 64) and the any-dimension kernel, in one slice and in several --
    # serve as its last resort and beyond 512 components
    if path == "exact_mfma":
        monkeypatch.setenv("PCA_KNN_FEAT", "0")
    elif path != "default":
        monkeypatch.setenv("PCA_KNN_NO_MFMA", "1")
        monkeypatch.setenv("PCA_KNN_SLICES",
                           "1" if path == "any_dimension" else "5")
    rng = np.random.default_rng(d * 7 + k)
    n, m = 1500, 300
    x = rng.standard_normal((n, d)).astype(np.float32)
    y = rng.standard_normal((m, d)).astype(np.float32)
    ptr_x = np.array([0, 40, 40, 1500])
    ptr_y = np.array([0, 100, 130, 300])
    got, gd = gpu_knn(x, y, ptr_x, ptr_y, k, cosine=cosine)
    want, wd = oracle_knn_edges(oracle, x, y, ptr_x, ptr_y, k, cosine=cosine)
    assert got.shape == want.shape
    assert (got == want).all()
    assert (gd == wd).all()


@pytest.mark.parametrize("d,k", [(3, 16), (2, 8), (8, 24), (24, 16),
                                 (128, 32)])
@pytest.mark.parametrize("case", ["offset", "huge", "tiny", "mixed_scale",
                                  "clustered"])
def test_prefilter_never_drops_a_neighbour(oracle, lowd_path, d, k, case):
    # the expanded-form pre-filter must stay conservative where it is least
    # accurate: tight clusters far from the origin, coordinates near the
    # overflow / underflow ends of fp32, wildly mixed scales
    rng = np.random.default_rng(stable_seed((d, k, case)))
    n, m = 5000, 600
    if case == "offset":
        x = 1000.0 + 1e-2 * rng.standard_normal((n, d))
        y = 1000.0 + 1e-2 * rng.standard_normal((m, d))
    elif case == "huge":
        x = 1e17 * rng.standard_normal((n, d))
        y = 1e17 * rng.standard_normal((m, d))
        y[:50] = x[:50]  # exact duplicates at distance 0
    elif case == "tiny":
        x = 1e-21 * rng.standard_normal((n, d))
        y = 1e-21 * rng.standard_normal((m, d))
    elif case == "mixed_scale":
        scale = 10.0 ** rng.integers(-6, 7, (n, 1))
        x = scale * rng.standard_normal((n, d))
        y = (10.0 ** rng.integers(-6, 7, (m, 1))) * rng.standard_normal((m, d))
    else:
        centres = 50.0 * rng.standard_normal((20, d))
        x = centres[rng.integers(0, 20, n)] + 1e-3 * rng.standard_normal((n, d))
        y = centres[rng.integers(0, 20, m)] + 1e-3 * rng.standard_normal((m, d))
    x = x.astype(np.float32)
    y = y.astype(np.float32)
    ptr_x = np.array([0, 2000, 5000])
    ptr_y = np.array([0, 250, 600])
    got, gd = gpu_knn(x, y, ptr_x, ptr_y, k)
    want, wd = oracle_knn_edges(oracle, x, y, ptr_x, ptr_y, k)
    assert got.shape == want.shape
    assert (got == want).all()
    assert (gd == wd).all()


@pytest.mark.parametrize("d,k", [(2, 8), (3, 16), (4, 24), (7, 32), (12, 8),
                                 (16, 24), (40, 16), (128, 32)])
@pytest.mark.parametrize("case", ["full_mantissa", "binade_edges",
                                  "norm_limit", "non_finite", "tiny_segments"])
def test_split_bf16_filter_edge_cases(oracle, d, k, case):
    # the matrix-core pre-filters (low-dimensional and feature-space kernels)
    # work on bf16 hi/lo splits of the operands:
    # values that round up across a power of two, rows around the norm above
    # which the filter is switched off, non-finite rows and queries mixed in,
    # and segments much shorter than a 32-row step
    rng = np.random.default_rng(stable_seed((d, k, case, "bf16")))
    n, m = 6000, 700
    ptr_x = np.array([0, 2500, 6000])
    ptr_y = np.array([0, 300, 700])
    if case == "full_mantissa":
        # every mantissa bit set, random exponents: the worst case of the
        # split's rounding
        bits = (rng.integers(100, 140, (n + m, d)).astype(np.uint32) << 23) \
            | 0x7fffff | (rng.integers(0, 2, (n + m, d)).astype(np.uint32) << 31)
        v = bits.view(np.float32)
        x, y = v[:n], v[n:]
    elif case == "binade_edges":
        base = 2.0 ** rng.integers(-3, 8, (n + m, d))
        v = base * (1.0 - rng.integers(0, 4, (n + m, d)) * 2.0 ** -24)
        v = v * rng.choice([-1.0, 1.0], (n + m, d))
        x, y = v[:n], v[n:]
    elif case == "norm_limit":
        # squared norms on both sides of 1e30
        scale = 10.0 ** rng.uniform(14.5, 15.5, (n + m, 1))
        v = scale * rng.standard_normal((n + m, d))
        x, y = v[:n], v[n:]
        y[:40] = x[:40]
    elif case == "non_finite":
        x = rng.standard_normal((n, d))
        y = rng.standard_normal((m, d))
        for arr, cnt in ((x, 300), (y, 40)):
            idx = rng.integers(0, arr.shape[0], cnt)
            arr[idx, rng.integers(0, d, cnt)] = rng.choice(
                [np.inf, -np.inf, np.nan, 3e38, -3e38], cnt)
    else:
        x = 10.0 * rng.standard_normal((n, d))
        y = 10.0 * rng.standard_normal((m, d))
        cuts = np.sort(rng.choice(np.arange(1, n), 199, replace=False))
        ptr_x = np.concatenate([[0], cuts, [n]])
        cuts = np.sort(rng.choice(np.arange(1, m), 199, replace=False))
        ptr_y = np.concatenate([[0], cuts, [m]])
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.ascontiguousarray(y, dtype=np.float32)
    with np.errstate(all="ignore"):
        got, gd = gpu_knn(x, y, ptr_x, ptr_y, k)
        want, wd = oracle_knn_edges(oracle, x, y, ptr_x, ptr_y, k)
    assert got.shape == want.shape
    assert (got == want).all()
    assert (gd == wd).all()


@pytest.mark.parametrize("d,k", [(3, 16), (24, 16), (128, 32), (100, 7)])
@pytest.mark.parametrize("case", ["parallel", "random", "scaled_copies",
                                  "zero_rows"])
def test_cosine_prefilter_never_drops_a_neighbour(oracle, d, k, case):
    rng = np.random.default_rng(stable_seed((d, k, case, "cos")))
    n, m = 4000, 500
    if case == "parallel":
        # all rows within a narrow cone: cosine distances ~1e-6, many
        # near-ties and slightly negative values
        axis = rng.standard_normal((1, d))
        x = axis * rng.uniform(0.5, 2.0, (n, 1)) + 1e-3 * rng.standard_normal((n, d))
        y = axis * rng.uniform(0.5, 2.0, (m, 1)) + 1e-3 * rng.standard_normal((m, d))
    elif case == "random":
        x = rng.standard_normal((n, d))
        y = rng.standard_normal((m, d))
    elif case == "scaled_copies":
        x = rng.standard_normal((n, d))
        y = x[rng.integers(0, n, m)] * rng.uniform(1e-3, 1e3, (m, 1))
    else:
        x = rng.standard_normal((n, d))
        y = rng.standard_normal((m, d))
        x[::97] = 0.0
        y[::31] = 0.0
    x = x.astype(np.float32)
    y = y.astype(np.float32)
    ptr_x = np.array([0, 1500, 4000])
    ptr_y = np.array([0, 200, 500])
    got, gd = gpu_knn(x, y, ptr_x, ptr_y, k, cosine=True)
    want, wd = oracle_knn_edges(oracle, x, y, ptr_x, ptr_y, k, cosine=True)
    assert got.shape == want.shape
    assert (got == want).all()
    assert (gd == wd).all()


def test_two_queries_per_lane_path(oracle, monkeypatch):
    monkeypatch.setenv("PCA_KNN_LOWD_MATRIX_CORES", "0")
    rng = np.random.default_rng(77)
    x = rng.random((5000, 3), dtype=np.float32)
    y = rng.random((1500, 3), dtype=np.float32)
    ptr_x = np.array([0, 2000, 5000])
    ptr_y = np.array([0, 515, 1500])
    want, wd = oracle_knn_edges(oracle, x, y, ptr_x, ptr_y, 16)
    for qpt in ("1", "2"):
        monkeypatch.setenv("PCA_KNN_QUERIES_PER_LANE", qpt)
        got, gd = gpu_knn(x, y, ptr_x, ptr_y, 16)
        assert (got == want).all() and (gd == wd).all()


@pytest.mark.parametrize("slices", [1, 2, 3, 5, 8, 16])
@pytest.mark.parametrize("qpt", ["1", "2", "matrix_cores"])
def test_sliced_segments_merge_exactly(oracle, monkeypatch, slices, qpt):
    # every segment's x rows cut into `slices` parts that share pruning
    # bounds and are merged by key: same bits as the unsliced scan, including
    # exact distance ties across slices (integer grid) and slices shorter
    # than k
    monkeypatch.setenv("PCA_KNN_SLICES", str(slices))
    if qpt == "matrix_cores":
        monkeypatch.setenv("PCA_KNN_LOWD_MATRIX_CORES", "1")
    else:
        monkeypatch.setenv("PCA_KNN_LOWD_MATRIX_CORES", "0")
        monkeypatch.setenv("PCA_KNN_QUERIES_PER_LANE", qpt)
    rng = np.random.default_rng(slices)
    x = rng.integers(0, 7, (9000, 3)).astype(np.float32)
    y = rng.integers(0, 7, (1100, 3)).astype(np.float32)
    ptr_x = np.array([0, 5000, 5000, 5013, 9000])
    ptr_y = np.array([0, 600, 650, 900, 1100])
    for k in (16, 21):
        got, gd = gpu_knn(x, y, ptr_x, ptr_y, k)
        want, wd = oracle_knn_edges(oracle, x, y, ptr_x, ptr_y, k)
        assert got.shape == want.shape
        assert (got == want).all()
        assert (gd == wd).all()
    xr = rng.standard_normal((30000, 3)).astype(np.float32)
    got, gd = gpu_knn(xr, xr[:700], None, None, 10)
    want, wd = oracle_knn_edges(oracle, xr, xr[:700], None, None, 10)
    assert (got == want).all() and (gd == wd).all()
    got, gd = gpu_knn(xr[:6000], xr[:300], None, None, 5, cosine=True)
    want, wd = oracle_knn_edges(oracle, xr[:6000], xr[:300], None, None, 5,
                                cosine=True)
    assert (got == want).all() and (gd == wd).all()


def test_against_float64_within_tie_tolerance():
    rng = np.random.default_rng(9)
    x = rng.random((4000, 3), dtype=np.float32)
    ptr = np.array([0, 1500, 4000])
    got, _ = gpu_knn(x, x, ptr, ptr, 12, want_dist=False)
    bad = check_knn_against_exact(got, x, x, ptr, ptr, 12)
    assert bad <= 2  # queries whose k-th and (k+1)-th distances tie in fp32


def test_operator_errors():
    x = torch.rand(10, 3, device=DEV)
    op = torch.ops.torch_cluster.knn
    with pytest.raises(RuntimeError, match="smaller than or equal to 100"):
        op(x, x, None, None, 101, False, 1)
    with pytest.raises(RuntimeError, match="must be contiguous"):
        op(torch.rand(3, 10, device=DEV).t(), x, None, None, 2, False, 1)
    with pytest.raises(RuntimeError, match="Input mismatch"):
        op(x, torch.rand(10, 2, device=DEV), None, None, 2, False, 1)
    with pytest.raises(RuntimeError, match="Input mismatch"):
        op(x, x, torch.tensor([0, 10], device=DEV),
           torch.tensor([0, 5, 10], device=DEV), 2, False, 1)
    # x decides the branch (csrc/knn.cpp:26); the other tensors must follow it
    with pytest.raises(RuntimeError, match="y must be CPU tensor"):
        op(x.cpu(), x, None, None, 2, False, 1)
    with pytest.raises(RuntimeError, match="y must be CUDA tensor"):
        op(x, x.cpu(), None, None, 2, False, 1)


def test_runs_on_the_current_stream(oracle):
    rng = np.random.default_rng(21)
    x = rng.random((3000, 3), dtype=np.float32)
    want, _ = oracle_knn_edges(oracle, x, x, None, None, 8)
    xs = dev(x)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        e = pca.knn(xs, xs, 8)
    side.synchronize()
    assert (e.cpu().numpy() == want).all()


# ---- the benchmark configurations -----------------------------------------------

# (every configuration under "scan" and under "auto", the library's default,
# which bins the large ones)
STRATEGIES = ["scan", "auto"]


@pytest.mark.parametrize("strategy", STRATEGIES)
def test_config1_knn_graph_1024(oracle, strategy):
    data = testing.uniform_cloud(0)
    x = data["x"]
    with use_strategy(strategy):
        e = pca.knn_graph(x.to(DEV), k=16, loop=False,
                          flow='source_to_target')
    want = oracle.knn_graph(x.numpy(), 16, loop=False,
                            flow='source_to_target')
    assert e.shape == (2, 16384)
    assert (e.cpu().numpy() == want).all()


@pytest.mark.parametrize("strategy", STRATEGIES)
@pytest.mark.parametrize("batch_size", [None, 16])
def test_config2_batched_knn_graph(oracle, strategy, batch_size):
    data = testing.uniform_batched(0)
    x, batch = data["x"], data["batch"]
    with use_strategy(strategy):
        e = pca.knn_graph(x.to(DEV), k=20, batch=batch.to(DEV), loop=False,
                          batch_size=batch_size)
    want = oracle.knn_graph(x.numpy(), 20, batch.numpy(), loop=False)
    assert e.shape == (2, 16 * 4096 * 20)
    assert (e.cpu().numpy() == want).all()


def test_config4_feature_space_reduced(oracle):
    # the 200,000 x 128 / 50,000 x 128 workload at 1/25 of the rows, Euclidean
    # and cosine, bit-exact against the oracle
    data = testing.feature_space(0, n=8000, m=2000, d=128)
    x, y = data["x"], data["y"]
    for cosine in (False, True):
        e = pca.knn(x.to(DEV), y.to(DEV), 32, cosine=cosine).cpu().numpy()
        want = oracle.knn(x.numpy(), y.numpy(), 32, cosine=cosine)
        assert (e == want).all()


@pytest.mark.parametrize("cosine", [False, True])
def test_config4_feature_space_full_size(oracle, cosine):
    # 200,000 x 128 against 50,000 queries, k = 32: size-independent
    # properties at full size, exact parity on a strided sample of the queries
    data = testing.feature_space(0)
    x, y = data["x"], data["y"]
    e = pca.knn(x.to(DEV), y.to(DEV), 32, cosine=cosine).cpu().numpy()
    m, n = y.shape[0], x.shape[0]
    assert e.shape == (2, 32 * m)
    assert (e[0] == np.repeat(np.arange(m), 32)).all()
    cols = e[1].reshape(m, 32)
    assert cols.min() >= 0 and cols.max() < n
    # 32 different rows per query
    assert (np.diff(np.sort(cols, axis=1), axis=1) > 0).all()
    sample = np.arange(0, m, 250)
    xs, ys = x.numpy().astype(np.float64), y.numpy()[sample].astype(np.float64)
    if cosine:
        xs = xs / np.linalg.norm(xs, axis=1, keepdims=True)
        ys = ys / np.linalg.norm(ys, axis=1, keepdims=True)
        dist = 1.0 - ys @ xs.T
    else:
        dist = ((ys ** 2).sum(1)[:, None] + (xs ** 2).sum(1)[None, :]
                - 2.0 * ys @ xs.T)
    got = np.take_along_axis(dist, cols[sample], 1)
    # ascending, and nothing left out is closer than the k-th returned
    assert (np.diff(got, axis=1) >= -1e-5).all()
    kth = np.partition(dist, 31, axis=1)[:, 31]
    assert (got[:, -1] <= kth + 1e-5).all()
    want, _ = oracle_knn_edges(oracle, x.numpy(), y.numpy()[sample], None,
                               None, 32, cosine)
    assert (cols[sample] == want[1].reshape(len(sample), 32)).all()


@pytest.mark.parametrize("strategy", STRATEGIES)
def test_config5_ragged_lidar_full_size(oracle, strategy):
    data = testing.lidar_scans(0)
    x, y = data["x"], data["y"]
    bx, by, B = data["batch_x"], data["batch_y"], data["batch_size"]
    with use_strategy(strategy):
        if strategy == "auto":
            assert torch.ops.pytorch_cluster_amd.strategy_for(
                "knn", x.shape[0], y.shape[0], B) == "binned"
        e = pca.knn(x.to(DEV), y.to(DEV), 16, bx.to(DEV), by.to(DEV),
                    batch_size=B).cpu().numpy()
    m = y.shape[0]
    # size-independent properties at full size
    assert e.shape == (2, 16 * m)
    assert (e[0] == np.repeat(np.arange(m), 16)).all()
    assert (bx.numpy()[e[1]] == by.numpy()[e[0]]).all()
    d2 = ((x.numpy()[e[1]].astype(np.float64)
           - y.numpy()[e[0]].astype(np.float64)) ** 2).sum(1).reshape(m, 16)
    assert (np.diff(d2, axis=1) >= -1e-6 * d2[:, 1:] - 1e-12).all()
    # every query is its own nearest neighbour candidate (y is a subset of x)
    assert (d2[:, 0] == 0).all()
    # exact parity on a strided sample of the queries
    ptr_x = testing.pointers(bx, B).numpy()
    sample = np.arange(0, m, 101)
    ys = y.numpy()[sample]
    ptr_ys = np.searchsorted(sample, testing.pointers(by, B).numpy())
    want, _ = oracle_knn_edges(oracle, x.numpy(), ys, ptr_x, ptr_ys, 16)
    got = e[1].reshape(m, 16)[sample]
    assert (got == want[1].reshape(len(sample), 16)).all()


@pytest.mark.parametrize("flow", ["source_to_target", "target_to_source"])
@pytest.mark.parametrize("loop", [False, True])
def test_graph_epilogue_in_the_output_pass(oracle, flow, loop):
    """knn_graph drops self-pairs and orients the edges while they are
    written (edge flags of pca_knn); order and content are those of the
    reference's mask + stack (torch_cluster/knn.py:135-144), including the
    rows that keep k + 1 edges because duplicates precede them."""
    rng = np.random.default_rng(5)
    x = rng.integers(0, 6, (3000, 3)).astype(np.float32)  # many duplicates
    batch = np.sort(rng.integers(0, 5, 3000))
    batch[batch == 2] = 3  # an example without rows
    for k in (1, 7, 20):
        want = oracle.knn_graph(x, k, batch, loop=loop, flow=flow)
        got = pca.knn_graph(dev(x), k, dev(batch), loop=loop, flow=flow)
        assert got.cpu().numpy().tolist() == want.tolist()
    # the C entry point with distances: they follow the kept edges
    ptr = np.searchsorted(batch, np.arange(6)).astype(np.int64)
    e, d = capi.knn_edges(dev(x), dev(x), dev(ptr), dev(ptr), 8,
                          want_dist=True, drop_self=True, x_first=True)
    e, d = e.cpu().numpy(), d.cpu().numpy()
    full, dfull = gpu_knn(x, x, ptr, ptr, 8)
    keep = full[0] != full[1]
    assert e.tolist() == full[::-1][:, keep].tolist()
    assert (d == dfull[keep]).all()


def test_operators_refuse_graph_capture():
    # the size of an edge list depends on the data: knn / radius read it from
    # the device before they return, which a capturing stream cannot do --
    # they say so instead of breaking the capture halfway
    x = torch.rand(500, 3, device=DEV)
    pca.knn(x, x, 3)  # (everything lazy is done before the capture)
    for call in (lambda: pca.knn(x, x, 3),
                 lambda: pca.radius(x, x, 0.1)):
        graph = torch.cuda.CUDAGraph()
        with pytest.raises(RuntimeError, match="cannot be captured"):
            with torch.cuda.graph(graph):
                call()
        torch.cuda.synchronize()
    # and work as before afterwards
    assert pca.knn(x, x, 3).shape == (2, 1500)
