"""GPU parity of the radius path against the CPU oracle (bit-exact: edge
sets, order and counts), through the C ABI and the Python entry points."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

import pytorch_cluster_amd as pca  # noqa: E402
from pytorch_cluster_amd import testing  # noqa: E402
from gpu_common import DEV, dev, gpu_radius, ragged_ptrs, use_strategy  # noqa: E402
from helpers import stable_seed, to_set  # noqa: E402


def tensor(v, dtype=torch.float32):
    return torch.tensor(v, dtype=dtype, device=DEV)


def to_degree(e):
    _, counts = torch.unique(e[1], return_counts=True)
    return counts.tolist()


# ---- the reference's fixtures (test/test_radius.py:25-116) -----------------

def test_reference_fixtures():
    x = tensor([[-1, -1], [-1, +1], [+1, +1], [+1, -1],
                [-1, -1], [-1, +1], [+1, +1], [+1, -1]])
    y = tensor([[0, 0], [0, 1]])
    batch_x = tensor([0, 0, 0, 0, 1, 1, 1, 1], torch.long)
    batch_y = tensor([0, 1], torch.long)
    full = {(0, 0), (0, 1), (0, 2), (0, 3), (1, 1), (1, 2), (1, 5), (1, 6)}
    assert to_set(pca.radius(x, y, 2, max_num_neighbors=4).cpu()) == full
    jit = torch.jit.script(pca.radius)
    assert to_set(jit(x, y, 2, max_num_neighbors=4).cpu()) == full
    part = {(0, 0), (0, 1), (0, 2), (0, 3), (1, 5), (1, 6)}
    e = pca.radius(x, y, 2, batch_x, batch_y, max_num_neighbors=4)
    assert to_set(e.cpu()) == part
    batch_x = tensor([0, 0, 0, 0, 2, 2, 2, 2], torch.long)
    batch_y = tensor([0, 2], torch.long)
    e = pca.radius(x, y, 2, batch_x, batch_y, max_num_neighbors=4)
    assert to_set(e.cpu()) == part


def test_reference_radius_graph_fixtures():
    x = tensor([[-1, -1], [-1, +1], [+1, +1], [+1, -1]])
    e = pca.radius_graph(x, r=2.5, flow='target_to_source')
    assert to_set(e.cpu()) == {(0, 1), (0, 3), (1, 0), (1, 2), (2, 1), (2, 3),
                               (3, 0), (3, 2)}
    e = pca.radius_graph(x, r=2.5, flow='source_to_target')
    assert to_set(e.cpu()) == {(1, 0), (3, 0), (0, 1), (2, 1), (1, 2), (3, 2),
                               (0, 3), (2, 3)}
    jit = torch.jit.script(pca.radius_graph)
    e = jit(x, r=2.5, flow='source_to_target')
    assert to_set(e.cpu()) == {(1, 0), (3, 0), (0, 1), (2, 1), (1, 2), (3, 2),
                               (0, 3), (2, 3)}
    e = pca.radius_graph(x, r=100, flow='source_to_target',
                         max_num_neighbors=1)
    assert set(to_degree(e)) == {1}
    same = tensor([[-1, -1]] * 4)
    e = pca.radius_graph(same, r=100, flow='source_to_target',
                         max_num_neighbors=1)
    assert set(to_degree(e)) == {1}
    x8 = tensor([[-1, -1], [-1, +1], [+1, +1], [+1, -1],
                 [-1, -1], [-1, +1], [+1, +1], [+1, -1]])
    batch = tensor([0, 0, 0, 0, 1, 1, 1, 1], torch.long)
    e = pca.radius_graph(x8, r=100, batch=batch, flow='source_to_target',
                         max_num_neighbors=1)
    assert set(to_degree(e)) == {1}
    assert [int(i / 4) for i in e[0].tolist()] == batch.tolist()
    # README.md:217-220, ordered
    x = tensor([[-1., -1.], [-1., 1.], [1., -1.], [1., 1.]])
    e = pca.radius_graph(x, r=2.5, batch=tensor([0] * 4, torch.long))
    assert e.tolist() == [[1, 2, 0, 3, 0, 3, 1, 2], [0, 0, 1, 1, 2, 2, 3, 3]]


def test_radius_graph_large_vs_ckdtree():
    # test/test_radius.py:119-133
    import scipy.spatial
    g = torch.Generator().manual_seed(4)
    x = torch.randn(1000, 3, generator=g)
    e = pca.radius_graph(x.to(DEV), r=0.5, flow='target_to_source', loop=True,
                         max_num_neighbors=2000)
    col = scipy.spatial.cKDTree(x.numpy()).query_ball_point(x.numpy(), r=0.5)
    truth = {(i, j) for i, ns in enumerate(col) for j in ns}
    assert to_set(e.cpu()) == truth


# ---- bit-exact parity against the oracle -----------------------------------

@pytest.fixture(params=["0", "1"], ids=["wave_per_query", "matrix_cores"])
def radius_path(request, monkeypatch):
    # both fp32 kernels, whatever the problem size would select
    monkeypatch.setenv("PCA_RADIUS_MATRIX_CORES", request.param)
    return request.param


@pytest.mark.parametrize("d", [1, 2, 3, 4, 7, 16])
@pytest.mark.parametrize("cap,ignore", [(1, False), (5, True), (32, False),
                                        (64, True), (5000, False)])
def test_parity_ragged(oracle, radius_path, d, cap, ignore):
    rng = np.random.default_rng(31 * d + cap)
    n = 3000
    x = rng.random((n, d), dtype=np.float32)
    segments = int(rng.choice([1, 2, 9]))
    ptr = ragged_ptrs(rng, n, segments)
    # radius chosen so the mean degree is a few dozen in any dimension
    r = 0.5 * (40.0 / n) ** (1.0 / d)
    got = gpu_radius(x, x, ptr, ptr, r, cap, ignore)
    want = oracle.radius_op(x, x, ptr, ptr, r, cap, 1, ignore)
    assert got.shape == want.shape
    assert (got == want).all()


def test_parity_bipartite_with_empty_segments(oracle, radius_path):
    rng = np.random.default_rng(8)
    x = rng.random((5000, 3), dtype=np.float32)
    y = rng.random((777, 3), dtype=np.float32)
    ptr_x = np.array([0, 0, 2000, 2000, 5000])
    ptr_y = np.array([0, 100, 400, 401, 777])
    for cap in (3, 32):
        got = gpu_radius(x, y, ptr_x, ptr_y, 0.11, cap)
        want = oracle.radius_op(x, y, ptr_x, ptr_y, 0.11, cap)
        assert (got == want).all()


def test_strict_inequality_at_the_radius(oracle, radius_path):
    # points exactly at distance r are excluded (dist < r*r, strict)
    x = np.array([[0, 0], [3, 4], [5, 0], [0, 4.9999995]], dtype=np.float32)
    y = np.array([[0, 0]], dtype=np.float32)
    got = gpu_radius(x, y, None, None, 5.0, 8)
    want = oracle.radius_op(x, y, None, None, 5.0, 8)
    assert got.tolist() == want.tolist() == [[0, 0], [0, 3]]


@pytest.mark.parametrize("d", [2, 3, 5])
@pytest.mark.parametrize("case", ["offset", "clusters", "non_finite",
                                  "huge", "dense_early_exit"])
def test_filter_never_drops_a_neighbour(oracle, radius_path, d, case):
    # where the split-bf16 pre-filter is least accurate or switched off, and
    # where queries fill up early and whole waves leave the scan
    rng = np.random.default_rng(stable_seed((d, case, "radius")))
    n, m, cap, r = 7000, 900, 16, 0.05
    ptr_x = np.array([0, 3000, 7000])
    ptr_y = np.array([0, 500, 900])
    if case == "offset":
        x = 300.0 + 0.2 * rng.random((n, d))
        y = 300.0 + 0.2 * rng.random((m, d))
    elif case == "clusters":
        centres = 40.0 * rng.standard_normal((30, d))
        x = centres[rng.integers(0, 30, n)] + 0.03 * rng.standard_normal((n, d))
        y = centres[rng.integers(0, 30, m)] + 0.03 * rng.standard_normal((m, d))
    elif case == "non_finite":
        x = 0.3 * rng.random((n, d))
        y = 0.3 * rng.random((m, d))
        for arr, cnt in ((x, 400), (y, 50)):
            idx = rng.integers(0, arr.shape[0], cnt)
            arr[idx, rng.integers(0, d, cnt)] = rng.choice(
                [np.inf, -np.inf, np.nan, 3e38], cnt)
    elif case == "huge":
        x = 1e16 * rng.standard_normal((n, d))
        y = 1e16 * rng.standard_normal((m, d))
        y[:60] = x[:60]
        r = 1e15
    else:
        x = 0.1 * rng.random((n, d))
        y = 0.1 * rng.random((m, d))
        cap, r = 4, 0.08
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.ascontiguousarray(y, dtype=np.float32)
    with np.errstate(all="ignore"):
        got = gpu_radius(x, y, ptr_x, ptr_y, r, cap)
        want = oracle.radius_op(x, y, ptr_x, ptr_y, r, cap)
    assert got.shape == want.shape
    assert (got == want).all()


def test_operator_errors():
    x = torch.rand(10, 3, device=DEV)
    op = torch.ops.torch_cluster.radius
    with pytest.raises(RuntimeError, match="must be contiguous"):
        op(torch.rand(3, 10, device=DEV).t(), x, None, None, 1.0, 4, 1, False)
    with pytest.raises(RuntimeError, match="Input mismatch"):
        op(x, torch.rand(10, 2, device=DEV), None, None, 1.0, 4, 1, False)
    with pytest.raises(RuntimeError, match="must be CUDA tensor"):
        op(x, x.cpu(), None, None, 1.0, 4, 1, False)


# ---- benchmark configuration 3 -------------------------------------------------

@pytest.mark.parametrize("strategy", ["scan", "auto", "binned"])
def test_config3_gaussian_mixture_radius_graph(oracle, strategy):
    data = testing.gaussian_mixture_batched(0)
    x, batch = data["x"], data["batch"]
    with use_strategy(strategy):
        e = pca.radius_graph(x.to(DEV), r=0.05, batch=batch.to(DEV),
                             max_num_neighbors=32, loop=False,
                             batch_size=data["batch_size"])
    want = oracle.radius_graph(x.numpy(), 0.05, batch.numpy(), loop=False,
                               max_num_neighbors=32)
    assert e.shape == want.shape
    assert (e.cpu().numpy() == want).all()
    assert (batch.numpy()[want[0]] == batch.numpy()[want[1]]).all()


@pytest.mark.parametrize("flow", ["source_to_target", "target_to_source"])
@pytest.mark.parametrize("loop", [False, True])
def test_graph_orientation_in_the_output_pass(oracle, radius_path, flow, loop):
    """radius_graph's flow flip (torch_cluster/radius.py:143-148) is applied
    while the edges are written (edge flags of pca_radius)."""
    rng = np.random.default_rng(8)
    x = rng.random((2500, 3)).astype(np.float32)
    batch = np.sort(rng.integers(0, 4, 2500))
    want = oracle.radius_graph(x, 0.12, batch, loop=loop, flow=flow,
                               max_num_neighbors=9)
    got = pca.radius_graph(dev(x), 0.12, dev(batch), loop=loop, flow=flow,
                           max_num_neighbors=9)
    assert got.cpu().numpy().tolist() == want.tolist()


# ---- feature space: the matrix-core filter in front of the exact distances
# (knn_feat_small_impl.hpp, RADIUS) against the plain scan and the checker

def _feature_case(rng, kind, n, m, d):
    x = rng.standard_normal((n, d)).astype(np.float32)
    y = rng.standard_normal((m, d)).astype(np.float32)
    if kind == "rows_as_queries":
        y[: m // 2] = x[rng.integers(0, n, m // 2)]
    elif kind == "clusters":
        c = rng.standard_normal((30, d)).astype(np.float32)
        x = (c[rng.integers(0, 30, n)] +
             0.3 * rng.standard_normal((n, d))).astype(np.float32)
        y = (c[rng.integers(0, 30, m)] +
             0.3 * rng.standard_normal((m, d))).astype(np.float32)
    elif kind == "duplicates":
        x = x[rng.integers(0, 50, n)]
        y = x[rng.integers(0, n, m)].copy()
    elif kind == "large_rows":
        x[rng.integers(0, n, 4)] *= 1e4
        y[[1, m - 1]] *= 1e5
    elif kind == "not_finite":
        x[7, 2] = np.nan
        x[n // 3] = np.inf
        y[3, 0] = np.nan
    return x, y


@pytest.mark.parametrize("kind", ["plain", "rows_as_queries", "clusters",
                                  "duplicates", "large_rows", "not_finite"])
@pytest.mark.parametrize("d", [9, 24, 64, 100, 128])
def test_feature_space_parity(oracle, monkeypatch, kind, d):
    monkeypatch.setenv("PCA_RADIUS_FEAT", "1")
    rng = np.random.default_rng(d * 13 + len(kind))
    n, m = 2600, 420
    x, y = _feature_case(rng, kind, n, m, d)
    ptr_x = np.array([0, 40, 40, 1500, n])
    ptr_y = np.array([0, 30, 50, 300, m])
    # radii from "a handful of neighbours" to "more than the limit"
    base = float(np.sqrt(2.0 * d)) if kind not in ("clusters", "duplicates") \
        else 0.45 * float(np.sqrt(d))
    for r, cap, ignore in ((0.8 * base, 32, False), (0.9 * base, 5, False),
                           (1.1 * base, 32, False), (0.7 * base, 17, True),
                           (1e-3, 8, False)):
        got = gpu_radius(x, y, ptr_x, ptr_y, r, cap, ignore)
        want = oracle.radius_op(x, y, ptr_x, ptr_y, r, cap, 1, ignore)
        assert got.shape == want.shape, (r, cap)
        assert (got == want).all(), (r, cap)


def test_feature_space_graph_is_the_plain_scan_s(monkeypatch):
    # 20 clouds of 900 points with 64 features, as a graph layer asks for
    # them: the default path against the plain scan of the library
    g = torch.Generator().manual_seed(11)
    x = torch.randn(20 * 900, 64, generator=g).to(DEV)
    batch = torch.arange(20, device=DEV).repeat_interleave(900)
    a = pca.radius_graph(x, 9.2, batch, max_num_neighbors=32, batch_size=20)
    monkeypatch.setenv("PCA_RADIUS_FEAT", "0")
    b = pca.radius_graph(x, 9.2, batch, max_num_neighbors=32, batch_size=20)
    assert a.shape == b.shape and a.shape[1] > 20 * 900
    assert bool((a == b).all())
