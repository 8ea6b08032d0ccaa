"""GPU parity of the binned radius search (pca_radius_binned through the C
ABI): the same edges in the same order as pca_radius, i.e. as the reference
kernel (csrc/cuda/radius_cuda.cu:9-42) - per query the first
max_num_neighbors rows, by ascending row number, with a squared distance
strictly below r * r.  Checked against the CPU oracle, and against the
scanning kernels at full size.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from pytorch_cluster_amd import capi, testing  # noqa: E402
from gpu_common import DEV, dev, ragged_ptrs  # noqa: E402


@pytest.fixture(autouse=True, params=["1", "0"],
                ids=["matrix_cores", "vector_alu"])
def scan_kind(request, monkeypatch):
    # both scans of a tile, whichever is the default
    monkeypatch.setenv("PCA_RADIUS_BINNED_MATRIX_CORES", request.param)
    return request.param


def gpu_radius_binned(x, y, ptr_x, ptr_y, r, max_nn, ignore_same=False):
    e = capi.radius_edges(dev(x), dev(y), dev(ptr_x, torch.long),
                          dev(ptr_y, torch.long), r, max_nn, ignore_same,
                          binned=True)
    torch.cuda.synchronize()
    return e.cpu().numpy()


@pytest.mark.parametrize("d", [1, 2, 3])
@pytest.mark.parametrize("cap,ignore", [(1, False), (5, True), (32, False),
                                        (17, True)])
def test_parity_ragged(oracle, d, cap, ignore):
    rng = np.random.default_rng(31 * d + cap)
    n = 4000
    x = rng.random((n, d), dtype=np.float32)
    segments = int(rng.choice([1, 2, 9]))
    ptr = ragged_ptrs(rng, n, segments)
    # mean degree of a few dozen: the cap cuts most lists
    r = 0.5 * (40.0 / n) ** (1.0 / d)
    got = gpu_radius_binned(x, x, ptr, ptr, r, cap, ignore)
    want = oracle.radius_op(x, x, ptr, ptr, r, cap, 1, ignore)
    assert got.shape == want.shape
    assert (got == want).all()


def test_bipartite_with_empty_segments(oracle):
    rng = np.random.default_rng(8)
    x = rng.random((5000, 3), dtype=np.float32)
    y = rng.random((777, 3), dtype=np.float32)
    ptr_x = np.array([0, 0, 2000, 2000, 5000])
    ptr_y = np.array([0, 100, 400, 401, 777])
    for cap in (3, 32):
        got = gpu_radius_binned(x, y, ptr_x, ptr_y, 0.11, cap)
        want = oracle.radius_op(x, y, ptr_x, ptr_y, 0.11, cap)
        assert (got == want).all()


def test_strict_inequality_at_the_radius(oracle):
    x = np.array([[0, 0], [3, 4], [5, 0], [0, 4.9999995]], dtype=np.float32)
    y = np.array([[0, 0]], dtype=np.float32)
    got = gpu_radius_binned(x, y, None, None, 5.0, 8)
    assert got.tolist() == [[0, 0], [0, 3]]
    # a grid: many rows at exactly the radius
    g = np.stack(np.meshgrid(np.arange(30), np.arange(30)), -1)
    x = g.reshape(-1, 2).astype(np.float32)
    got = gpu_radius_binned(x, x, None, None, 5.0, 32)
    want = oracle.radius_op(x, x, None, None, 5.0, 32)
    assert (got == want).all()


def test_fewer_rows_than_slots_and_nothing_in_range(oracle):
    rng = np.random.default_rng(3)
    x = rng.random((20, 3), dtype=np.float32)
    y = rng.random((50, 3), dtype=np.float32)
    for r in (10.0, 1e-4):
        got = gpu_radius_binned(x, y, None, None, r, 32)
        want = oracle.radius_op(x, y, None, None, r, 32)
        assert got.shape == want.shape and (got == want).all()


def test_rows_and_queries_that_are_not_finite(oracle):
    rng = np.random.default_rng(5)
    x = rng.standard_normal((3000, 3)).astype(np.float32)
    y = rng.standard_normal((300, 3)).astype(np.float32)
    x[7, 0] = np.nan
    x[100:140] = np.nan
    x[900, 1] = np.inf
    y[2, 2] = np.nan
    y[3, 0] = -np.inf
    got = gpu_radius_binned(x, y, None, None, 0.4, 16)
    want = oracle.radius_op(x, y, None, None, 0.4, 16)
    assert got.shape == want.shape and (got == want).all()


def test_clustered_clouds_against_the_scanning_kernels():
    """8 x 16,384 points in 32 clusters each, mean degree in the hundreds:
    the lists are full long before the last row in range is seen."""
    c = testing.gaussian_mixture_batched(0)
    x = c["x"].to(DEV)
    ptr = (torch.arange(9) * 16384).to(DEV)
    for ignore in (False, True):
        a = capi.radius_edges(x, x, ptr, ptr, 0.05, 32, ignore)
        b = capi.radius_edges(x, x, ptr, ptr, 0.05, 32, ignore, binned=True)
        assert torch.equal(a, b)
    a = capi.radius_edges(x, x, ptr, ptr, 0.05, 32, True, x_first=True)
    b = capi.radius_edges(x, x, ptr, ptr, 0.05, 32, True, x_first=True,
                          binned=True)
    assert torch.equal(a, b)


def test_lidar_like_scans_against_the_scanning_kernels():
    c = testing.lidar_scans(0, scans=3, min_points=60000, max_points=90000)
    x, y = c["x"].to(DEV), c["y"].to(DEV)
    px = testing.pointers(c["batch_x"], 3).to(DEV)
    py = testing.pointers(c["batch_y"], 3).to(DEV)
    a = capi.radius_edges(x, y, px, py, 0.3, 24)
    b = capi.radius_edges(x, y, px, py, 0.3, 24, binned=True)
    assert torch.equal(a, b)


def test_strategy_switch_of_the_entry_points():
    import pytorch_cluster_amd as pca
    g = torch.Generator().manual_seed(6)
    x = torch.rand(6000, 3, generator=g).to(DEV)
    y = torch.rand(900, 3, generator=g).to(DEV)
    bx = torch.arange(3).repeat_interleave(2000).to(DEV)
    by = torch.arange(3).repeat_interleave(300).to(DEV)

    def run():
        return (pca.radius(x, y, 0.1, bx, by, max_num_neighbors=20),
                pca.radius_graph(x, 0.08, bx, loop=False),
                pca.radius_graph(x, 0.08, bx, loop=True,
                                 flow="target_to_source"),
                pca.radius(x, y, 0.1, bx, by, max_num_neighbors=40))
    want = run()
    try:
        pca.set_search_strategy("binned")
        got = run()
    finally:
        pca.set_search_strategy("scan")
    for a, b in zip(want, got):
        assert torch.equal(a, b)


@pytest.mark.parametrize("cap", [33, 40, 41, 50, 57, 64])
def test_more_than_32_neighbours(oracle, cap, scan_kind):
    """Lists of 40 to 64 entries (matrix-core scan only): dense
    neighbourhoods, so that the cap cuts most lists, and some below it."""
    if scan_kind == "0":
        pytest.skip("wide lists exist for the matrix-core scan only")
    rng = np.random.default_rng(cap)
    x = rng.random((6000, 3)).astype(np.float32)
    x[:800] = np.round(x[:800] * 8) / 8       # exact ties and duplicates
    y = rng.random((500, 3)).astype(np.float32)
    ptr_x = np.array([0, 2500, 6000], dtype=np.int64)
    ptr_y = np.array([0, 200, 500], dtype=np.int64)
    for r in (0.12, 0.3):
        got = gpu_radius_binned(x, y, ptr_x, ptr_y, r, cap)
        want = oracle.radius_op(x, y, ptr_x, ptr_y, r, cap)
        assert np.array_equal(got, want)
    a = capi.radius_edges(dev(x), dev(x), None, None, 0.2, cap, True)
    b = capi.radius_edges(dev(x), dev(x), None, None, 0.2, cap, True,
                          binned=True)
    assert torch.equal(a, b)


def test_unsupported_shapes_are_refused():
    x = torch.rand(100, 4, device=DEV)
    with pytest.raises(RuntimeError, match="binned search"):
        capi.radius_edges(x, x, None, None, 0.1, 8, binned=True)
    x = torch.rand(100, 3, device=DEV)
    with pytest.raises(RuntimeError, match="binned search"):
        capi.radius_edges(x, x, None, None, 0.1, 65, binned=True)
