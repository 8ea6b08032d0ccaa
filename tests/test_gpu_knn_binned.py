"""GPU parity of the binned kNN search (pca_knn_binned through the C ABI).

It stands under the same operator as pca_knn and must return the same edges
and distances, bit for bit and in the same order: checked against the CPU
oracle (the reference kernel's scan, csrc/cuda/knn_cuda.cu:30-84, evaluated
with fused multiply-adds) at sizes the oracle finishes in seconds, and against
the scanning kernels of pca_knn at full size.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from pytorch_cluster_amd import capi, testing  # noqa: E402
from gpu_common import DEV, dev, gpu_knn, oracle_knn_edges, ragged_ptrs  # noqa


@pytest.fixture(autouse=True, params=["1", "0"],
                ids=["matrix_cores", "vector_alu"])
def scan_kind(request, monkeypatch):
    # both scans of a tile, whichever is the default
    monkeypatch.setenv("PCA_KNN_BINNED_MATRIX_CORES", request.param)
    return request.param


def gpu_knn_binned(x, y, ptr_x, ptr_y, k, want_dist=True, **kw):
    e, d = capi.knn_edges(dev(x), dev(y), dev(ptr_x, torch.long),
                          dev(ptr_y, torch.long), k, False, want_dist,
                          binned=True, **kw)
    torch.cuda.synchronize()
    return e.cpu().numpy(), (None if d is None else d.cpu().numpy())


def check(oracle, x, y, ptr_x, ptr_y, k):
    want_e, want_d = oracle_knn_edges(oracle, x, y, ptr_x, ptr_y, k)
    got_e, got_d = gpu_knn_binned(x, y, ptr_x, ptr_y, k)
    assert got_e.shape == want_e.shape
    assert (got_e == want_e).all()
    assert (got_d.view(np.uint32) == want_d.view(np.uint32)).all()


@pytest.mark.parametrize("d", [1, 2, 3])
@pytest.mark.parametrize("k", [1, 5, 8, 16, 17, 32])
def test_random_clouds(oracle, d, k):
    rng = np.random.default_rng(10 * d + k)
    x = rng.standard_normal((5000, d)).astype(np.float32)
    y = rng.standard_normal((700, d)).astype(np.float32)
    check(oracle, x, y, None, None, k)


@pytest.mark.parametrize("segments", [2, 5, 40])
@pytest.mark.parametrize("k", [3, 16, 24])
def test_ragged_segments(oracle, segments, k):
    """Segments of uneven size, one of them empty, some shorter than k."""
    rng = np.random.default_rng(segments + k)
    n, m = 6000, 1500
    ptr_x = ragged_ptrs(rng, n, segments)
    ptr_y = ragged_ptrs(rng, m, segments)
    x = rng.random((n, 3)).astype(np.float32)
    y = rng.random((m, 3)).astype(np.float32)
    check(oracle, x, y, ptr_x, ptr_y, k)


@pytest.mark.parametrize("d", [2, 3])
@pytest.mark.parametrize("k", [4, 16, 32])
def test_ties_go_to_the_lower_row(oracle, d, k):
    """Points on a coarse integer grid: most k-th distances are shared by
    several rows, which the binned search meets out of row order."""
    rng = np.random.default_rng(d * 100 + k)
    x = rng.integers(0, 6, (4000, d)).astype(np.float32)
    y = rng.integers(0, 6, (500, d)).astype(np.float32)
    ptr_x = np.array([0, 2500, 4000], dtype=np.int64)
    ptr_y = np.array([0, 200, 500], dtype=np.int64)
    check(oracle, x, y, ptr_x, ptr_y, k)


def test_all_rows_equal(oracle):
    x = np.ones((3000, 3), dtype=np.float32)
    y = np.ones((130, 3), dtype=np.float32)
    check(oracle, x, y, None, None, 16)


def test_self_search_lidar_like(oracle):
    """Queries that are rows of x (every 4th), strongly varying density."""
    c = testing.lidar_scans(0, scans=2, min_points=4000, max_points=6000)
    x, y = c["x"].numpy(), c["y"].numpy()
    ptr_x = testing.pointers(c["batch_x"], 2).numpy()
    ptr_y = testing.pointers(c["batch_y"], 2).numpy()
    check(oracle, x, y, ptr_x, ptr_y, 16)


def test_queries_far_from_the_rows(oracle):
    rng = np.random.default_rng(7)
    x = rng.random((3000, 3)).astype(np.float32)
    y = (rng.random((300, 3)) * 50 - 25).astype(np.float32)
    check(oracle, x, y, None, None, 10)


def test_rows_and_queries_that_are_not_finite(oracle):
    """NaN and infinite coordinates never make a neighbour (their distances
    are not below 1e10); neither do rows farther than 1e5 away."""
    rng = np.random.default_rng(8)
    x = rng.standard_normal((2000, 3)).astype(np.float32)
    y = rng.standard_normal((200, 3)).astype(np.float32)
    x[5, 1] = np.nan
    x[64:96] = np.nan          # a whole tile's worth, wherever they land
    x[700, 0] = np.inf
    x[701, 2] = -np.inf
    x[900] = 3e5               # squared distance 2.7e11 >= 1e10
    y[3, 0] = np.nan
    y[4, 2] = np.inf
    y[5] = 3e5                 # finds only x[900]
    check(oracle, x, y, None, None, 8)


def test_fewer_rows_than_k_and_single_rows(oracle):
    rng = np.random.default_rng(9)
    ptr_x = np.array([0, 1, 4, 4, 40, 300], dtype=np.int64)
    ptr_y = np.array([0, 3, 5, 9, 9, 100], dtype=np.int64)
    x = rng.random((300, 2)).astype(np.float32)
    y = rng.random((100, 2)).astype(np.float32)
    check(oracle, x, y, ptr_x, ptr_y, 12)


def test_edge_options_match_the_scanning_search():
    g = torch.Generator().manual_seed(4)
    x = torch.rand(5000, 3, generator=g).to(DEV)
    ptr = torch.tensor([0, 1000, 5000], device=DEV)
    for drop_self, x_first in ((True, False), (False, True), (True, True)):
        a, _ = capi.knn_edges(x, x, ptr, ptr, 9, drop_self=drop_self,
                              x_first=x_first)
        b, _ = capi.knn_edges(x, x, ptr, ptr, 9, drop_self=drop_self,
                              x_first=x_first, binned=True)
        assert torch.equal(a, b)


def test_full_size_against_the_scanning_kernels():
    """The ragged LiDAR-like workload at full size (1M points, 258k queries):
    identical edges and distances from both searches."""
    c = testing.lidar_scans(0)
    x, y = c["x"].to(DEV), c["y"].to(DEV)
    px = testing.pointers(c["batch_x"], c["batch_size"]).to(DEV)
    py = testing.pointers(c["batch_y"], c["batch_size"]).to(DEV)
    a, da = capi.knn_edges(x, y, px, py, 16, want_dist=True)
    b, db = capi.knn_edges(x, y, px, py, 16, want_dist=True, binned=True)
    assert torch.equal(a, b)
    assert torch.equal(da.view(torch.int32), db.view(torch.int32))


def test_queries_ordered_beside_the_rows(monkeypatch):
    """From 131,072 queries on, the queries are ordered on a second stream
    while the rows are ordered on the caller's: same edges with and without
    it, call after call, on the default stream and on another one."""
    c = testing.lidar_scans(0)
    x, y = c["x"].to(DEV), c["y"].to(DEV)
    px = testing.pointers(c["batch_x"], c["batch_size"]).to(DEV)
    py = testing.pointers(c["batch_y"], c["batch_size"]).to(DEV)
    monkeypatch.setenv("PCA_BINNED_SIDE_STREAM", "0")
    want, want_dist = capi.knn_edges(x, y, px, py, 16, want_dist=True,
                                     binned=True)
    monkeypatch.delenv("PCA_BINNED_SIDE_STREAM")
    other = torch.cuda.Stream()
    for stream in (torch.cuda.current_stream(), other, other):
        stream.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(stream):
            # (other work of the caller's stream right before and after)
            noise = torch.rand(1 << 20, device=DEV).sort().values
            got, got_dist = capi.knn_edges(x, y, px, py, 16, want_dist=True,
                                           binned=True)
            total = got.sum() + noise.numel()
        torch.cuda.current_stream().wait_stream(stream)
        torch.cuda.synchronize()
        assert torch.equal(got, want)
        assert torch.equal(got_dist.view(torch.int32),
                           want_dist.view(torch.int32))
        assert int(total) == int(want.sum()) + (1 << 20)
    # the nearest search: 1M searching rows
    monkeypatch.setenv("PCA_BINNED_SIDE_STREAM", "0")
    want = capi.nearest_rows(x, y, px, py, binned=True)
    monkeypatch.delenv("PCA_BINNED_SIDE_STREAM")
    for _ in range(2):
        assert torch.equal(capi.nearest_rows(x, y, px, py, binned=True), want)


def test_crowded_cells_and_many_segments():
    """What the ordering of the rows has to cope with: most rows in a handful of
    cells (duplicates, a dense clump beside a sparse cloud), more segments
    than rows per segment, a single row."""
    rng = np.random.default_rng(21)
    clump = np.repeat(rng.random((5, 3)), 3000, axis=0)
    clump += 1e-6 * rng.standard_normal(clump.shape)
    x = np.concatenate([clump, rng.random((5000, 3)) * 50.0,
                        np.repeat(rng.random((1, 3)), 4000, axis=0)])
    x = x[rng.permutation(len(x))].astype(np.float32)
    y = x[::3].copy()
    a, da = capi.knn_edges(dev(x), dev(y), None, None, 9, want_dist=True)
    b, db = capi.knn_edges(dev(x), dev(y), None, None, 9, want_dist=True,
                           binned=True)
    assert torch.equal(a, b) and torch.equal(da.view(torch.int32),
                                             db.view(torch.int32))
    # 700 segments of ~30 rows, some empty
    n = 21000
    x = rng.random((n, 3)).astype(np.float32)
    ptr = ragged_ptrs(rng, n, 700)
    a, _ = capi.knn_edges(dev(x), dev(x), dev(ptr), dev(ptr), 4)
    b, _ = capi.knn_edges(dev(x), dev(x), dev(ptr), dev(ptr), 4, binned=True)
    assert torch.equal(a, b)
    one = dev(x[:1])
    b, _ = capi.knn_edges(one, one, None, None, 3, binned=True)
    assert b.cpu().tolist() == [[0], [0]]


@pytest.mark.parametrize("m", [1, 32, 33, 8192, 8224, 131071, 131072,
                               196608, 196640])
def test_task_counts_at_the_edges(m):
    """Blocks of 32 queries: one, one and a bit, a whole workgroup of the
    ordering kernels (256 blocks) and one more, the first size ordered on a
    second stream (131,072 queries), the last size whose long blocks are
    split (6,144 blocks) and the first that is not.  Clustered queries (long
    and short spans) in two segments, against the scanning kernels."""
    g = torch.Generator().manual_seed(m)
    x = torch.rand(40000, 3, generator=g)
    y = torch.cat([torch.rand(m - m // 2, 3, generator=g) ** 3,
                   torch.rand(m // 2, 3, generator=g)])
    ptr_x = torch.tensor([0, 15000, 40000])
    ptr_y = torch.tensor([0, m - m // 2, m])
    x, y, ptr_x, ptr_y = (t.to(DEV) for t in (x, y, ptr_x, ptr_y))
    a, da = capi.knn_edges(x, y, ptr_x, ptr_y, 7, want_dist=True)
    b, db = capi.knn_edges(x, y, ptr_x, ptr_y, 7, want_dist=True, binned=True)
    assert torch.equal(a, b)
    assert torch.equal(da.view(torch.int32), db.view(torch.int32))
    assert torch.equal(capi.nearest_rows(y, x, ptr_y, ptr_x),
                       capi.nearest_rows(y, x, ptr_y, ptr_x, binned=True))


def test_uniform_clouds_against_the_scanning_kernels():
    c = testing.uniform_batched(0)
    x = c["x"].to(DEV)
    ptr = (torch.arange(17) * 4096).to(DEV)
    a, da = capi.knn_edges(x, x, ptr, ptr, 21, want_dist=True)
    b, db = capi.knn_edges(x, x, ptr, ptr, 21, want_dist=True, binned=True)
    assert torch.equal(a, b)
    assert torch.equal(da.view(torch.int32), db.view(torch.int32))


def test_unsupported_shapes_are_refused():
    x = torch.rand(100, 4, device=DEV)
    with pytest.raises(RuntimeError, match="binned search"):
        capi.knn_edges(x, x, None, None, 4, binned=True)
    x = torch.rand(100, 3, device=DEV)
    with pytest.raises(RuntimeError, match="binned search"):
        capi.knn_edges(x, x, None, None, 65, binned=True)


@pytest.mark.parametrize("k", [33, 40, 41, 50, 57, 64])
def test_more_than_32_neighbours(oracle, k, scan_kind):
    """Lists of 40 to 64 entries (matrix-core scan only)."""
    if scan_kind == "0":
        pytest.skip("wide lists exist for the matrix-core scan only")
    rng = np.random.default_rng(k)
    x = rng.random((4000, 3)).astype(np.float32)
    x[:500] = np.round(x[:500] * 4) / 4      # some exact ties
    y = rng.random((300, 3)).astype(np.float32)
    ptr_x = np.array([0, 45, 2000, 4000], dtype=np.int64)   # 45 rows < k
    ptr_y = np.array([0, 20, 150, 300], dtype=np.int64)
    check(oracle, x, y, ptr_x, ptr_y, k)


def test_strategy_switch_of_the_entry_points():
    """`set_search_strategy("binned")` sends knn / knn_graph of low-dimensional
    fp32 points through the binned search (same edges), leaves everything
    else on the scanning kernels, and can be switched back."""
    import pytorch_cluster_amd as pca
    g = torch.Generator().manual_seed(5)
    x = torch.rand(6000, 3, generator=g).to(DEV)
    y = torch.rand(900, 3, generator=g).to(DEV)
    bx = torch.arange(3).repeat_interleave(2000).to(DEV)
    by = torch.arange(3).repeat_interleave(300).to(DEV)
    hi = torch.rand(500, 16, generator=g).to(DEV)
    assert pca.get_search_strategy() == "scan"
    want = (pca.knn(x, y, 7, bx, by), pca.knn_graph(x, 6, bx, loop=False),
            pca.knn_graph(x, 6, bx, loop=True, flow="target_to_source"),
            pca.knn(hi, hi, 4), pca.knn(x, y, 5, bx, by, cosine=True))
    try:
        pca.set_search_strategy("binned")
        assert pca.get_search_strategy() == "binned"
        got = (pca.knn(x, y, 7, bx, by), pca.knn_graph(x, 6, bx, loop=False),
               pca.knn_graph(x, 6, bx, loop=True, flow="target_to_source"),
               pca.knn(hi, hi, 4), pca.knn(x, y, 5, bx, by, cosine=True))
        jit = torch.jit.script(pca.knn)
        assert torch.equal(jit(x, y, 7, bx, by), want[0])
    finally:
        pca.set_search_strategy("scan")
    for a, b in zip(want, got):
        assert torch.equal(a, b)
    with pytest.raises(RuntimeError, match="scan.*binned"):
        pca.set_search_strategy("tree")
    assert pca.get_search_strategy() == "scan"


def test_auto_strategy_bins_large_examples_only(monkeypatch):
    """"auto" picks per call; whatever it picks, the edges are the same."""
    import pytorch_cluster_amd as pca
    g = torch.Generator().manual_seed(9)
    small = torch.rand(20000, 3, generator=g).to(DEV)
    large = torch.rand(140000, 3, generator=g).to(DEV)
    y = large[::2].contiguous()
    want_small = pca.knn(small, small[::10].contiguous(), 8)
    want_large = pca.knn(large, y, 8)
    try:
        pca.set_search_strategy("auto")
        assert pca.get_search_strategy() == "auto"
        assert torch.equal(pca.knn(small, small[::10].contiguous(), 8),
                           want_small)
        assert torch.equal(pca.knn(large, y, 8), want_large)
        assert torch.equal(pca.radius(large, y, 0.02, max_num_neighbors=8),
                           _scan_radius(pca, large, y))
    finally:
        pca.set_search_strategy("scan")


def _scan_radius(pca, x, y):
    before = pca.get_search_strategy()
    pca.set_search_strategy("scan")
    try:
        return pca.radius(x, y, 0.02, max_num_neighbors=8)
    finally:
        pca.set_search_strategy(before)


def test_many_small_segments(oracle):
    rng = np.random.default_rng(11)
    sizes_x = rng.integers(0, 70, 300)
    sizes_y = rng.integers(0, 20, 300)
    ptr_x = np.concatenate([[0], np.cumsum(sizes_x)]).astype(np.int64)
    ptr_y = np.concatenate([[0], np.cumsum(sizes_y)]).astype(np.int64)
    x = rng.random((ptr_x[-1], 3)).astype(np.float32)
    y = rng.random((ptr_y[-1], 3)).astype(np.float32)
    check(oracle, x, y, ptr_x, ptr_y, 6)


def test_three_million_rows_against_the_scanning_kernels(scan_kind):
    """One large segment (positions and tile numbers far beyond 16 bits) and
    coordinates with a large common offset."""
    if scan_kind == "0":
        pytest.skip("one scan kind is enough at this size")
    g = torch.Generator().manual_seed(12)
    x = (torch.rand(3000000, 3, generator=g) * 100.0 + 5000.0).to(DEV)
    y = x[::37].contiguous()
    a, da = capi.knn_edges(x, y, None, None, 8, want_dist=True)
    b, db = capi.knn_edges(x, y, None, None, 8, want_dist=True, binned=True)
    assert torch.equal(a, b)
    assert torch.equal(da.view(torch.int32), db.view(torch.int32))


def test_rows_searching_for_themselves_share_one_order(oracle):
    """x and y the same buffer (the graph entry points): the order along the
    curve is computed once and serves both sides."""
    rng = np.random.default_rng(21)
    x = rng.integers(0, 7, (5000, 3)).astype(np.float32)   # ties everywhere
    ptr = np.array([0, 1200, 1200, 5000], dtype=np.int64)
    xt, pt = dev(x), dev(ptr, torch.long)
    e, d = capi.knn_edges(xt, xt, pt, pt, 9, want_dist=True, binned=True)
    want_e, want_d = oracle_knn_edges(oracle, x, x, ptr, ptr, 9)
    assert (e.cpu().numpy() == want_e).all()
    assert (d.cpu().numpy().view(np.uint32) == want_d.view(np.uint32)).all()
    r = capi.radius_edges(xt, xt, pt, pt, 1.5, 12, True, binned=True)
    want_r = oracle.radius_op(x, x, ptr, ptr, 1.5, 12, 1, True)
    assert (r.cpu().numpy() == want_r).all()


def test_auto_strategy_crossover():
    """Where "auto" changes its mind: the decisions at the benchmark sizes,
    that more rows per example never turn a binned search back into a scan,
    and -- at sizes on both sides of every switch -- the same edges from
    either strategy."""
    import pytorch_cluster_amd as pca
    pick = torch.ops.pytorch_cluster_amd.strategy_for
    before = pca.get_search_strategy()
    pca.set_search_strategy("auto")
    try:
        # small clouds are scanned, large ones binned
        assert pick("knn", 1024, 1024, 1) == "scan"
        assert pick("knn", 16 * 4096, 16 * 4096, 16) == "scan"
        assert pick("radius", 8 * 16384, 8 * 16384, 8) == "scan"
        assert pick("knn", 1033867, 258468, 8) == "binned"
        assert pick("knn", 1000000, 1000000, 1) == "binned"
        assert pick("radius", 1000000, 1000000, 1) == "binned"
        assert pick("nearest", 129236, 1033867, 8) == "binned"
        # a handful of queries against many rows: binning the rows costs more
        # than looking at them
        assert pick("knn", 1000000, 50, 1) == "scan"
        for op in ("knn", "radius", "nearest"):
            for segments in (1, 8):
                sizes = [2 ** e for e in range(8, 24)]
                picks = [pick(op, n * segments, n * segments, segments)
                         for n in sizes]
                first = picks.index("binned")
                assert all(p == "binned" for p in picks[first:]), (op, picks)
                assert 2 ** 12 <= sizes[first] <= 2 ** 17, (op, sizes[first])
                # same edges just below and just above the switch
                g = torch.Generator().manual_seed(first)
                for n in (sizes[first - 1], sizes[first]):
                    x = torch.rand(n * segments, 3, generator=g).to(DEV)
                    b = (torch.arange(n * segments) // n).to(DEV)
                    results = []
                    for strategy in ("scan", "binned", "auto"):
                        pca.set_search_strategy(strategy)
                        if op == "knn":
                            results.append(pca.knn(x, x, 5, b, b,
                                                   batch_size=segments))
                        elif op == "radius":
                            results.append(pca.radius(
                                x, x, 0.6 * n ** (-1 / 3), b, b,
                                max_num_neighbors=10, batch_size=segments))
                        else:
                            results.append(pca.nearest(x, x[::3].contiguous(),
                                                       b, b[::3].contiguous()))
                    pca.set_search_strategy("auto")
                    assert torch.equal(results[0], results[1])
                    assert torch.equal(results[0], results[2])
        # the forced strategies answer for themselves
        pca.set_search_strategy("scan")
        assert pick("knn", 10 ** 7, 10 ** 7, 1) == "scan"
        pca.set_search_strategy("binned")
        assert pick("knn", 10, 10, 1) == "binned"
    finally:
        pca.set_search_strategy(before)
