"""The operators on CPU tensors: the package's own host searches
(pytorch_cluster_amd/csrc/cpu_search.cpp, k-d trees / tiled scans on host
threads), where the reference runs knn_cpu / radius_cpu
(csrc/cpu/knn_cpu.cpp:7-105, csrc/cpu/radius_cpu.cpp:7-117).  They keep the
result contract of the GPU kernels, so the CPU checker's edges are expected bit
for bit, in order -- including BASELINE configs[0], `knn_graph` of 1,024 points
on the CPU.
"""
import numpy as np
import pytest
import torch

import pytorch_cluster_amd as pca
from pytorch_cluster_amd import testing


def bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def test_config1_knn_graph_on_the_cpu(oracle):
    x = testing.uniform_cloud(0)["x"]
    for flow in ("source_to_target", "target_to_source"):
        for loop in (False, True):
            got = pca.knn_graph(x, 16, loop=loop, flow=flow)
            want = oracle.knn_graph(x.numpy(), 16, loop=loop, flow=flow)
            assert got.dtype == torch.long and got.device.type == "cpu"
            assert (got.numpy() == want).all()
    scripted = torch.jit.script(pca.knn_graph)
    assert torch.equal(scripted(x, 16), pca.knn_graph(x, 16))


def test_reference_fixtures_on_the_cpu():
    # the reference's own fixtures (test/test_knn.py:16-75,
    # test/test_radius.py:25-116, README.md:178-220; committed as
    # tests/golden/reference_fixtures.json) and the vectors of its compiled CPU
    # operators, through the operators on CPU tensors
    from test_golden import arr, check_edges, fixtures, ref_vectors

    def t(v, dtype=torch.float32):
        return None if v is None else torch.tensor(v, dtype=dtype)

    fx = fixtures()
    for c in fx["knn"]:
        if c["cosine"]:
            continue  # (GPU only, as in the reference)
        check_edges(c, pca.knn(t(c["x"]), t(c["y"]), c["k"],
                               t(c["batch_x"], torch.long),
                               t(c["batch_y"], torch.long)).numpy())
    for c in fx["knn_graph"]:
        check_edges(c, pca.knn_graph(t(c["x"]), c["k"],
                                     t(c["batch"], torch.long),
                                     loop=c["loop"], flow=c["flow"]).numpy())
    for c in fx["radius"]:
        check_edges(c, pca.radius(t(c["x"]), t(c["y"]), c["r"],
                                  t(c["batch_x"], torch.long),
                                  t(c["batch_y"], torch.long),
                                  max_num_neighbors=c["max_num_neighbors"])
                    .numpy())
    for c in fx["radius_graph"]:
        check_edges(c, pca.radius_graph(t(c["x"]), c["r"],
                                        t(c["batch"], torch.long),
                                        loop=c["loop"],
                                        flow=c["flow"]).numpy())
    v = ref_vectors()
    f = torch.from_numpy
    e = torch.ops.torch_cluster.knn(f(v["knn3_x"]), f(v["knn3_y"]),
                                    f(v["knn3_ptr_x"]), f(v["knn3_ptr_y"]),
                                    int(v["knn3_k"]), False, 1)
    assert (e.numpy() == v["knn3_edges"]).all()
    e = torch.ops.torch_cluster.knn(f(v["knn16_x"]), f(v["knn16_y"]), None,
                                    None, int(v["knn16_k"]), False, 1)
    assert (e.numpy() == v["knn16_edges"]).all()
    e = torch.ops.torch_cluster.radius(f(v["rad_x"]), f(v["rad_y"]),
                                       f(v["rad_ptr_x"]), f(v["rad_ptr_y"]),
                                       float(v["rad_r"]), int(v["rad_max"]),
                                       1, False)
    assert (e.numpy() == v["rad_edges"]).all()
    x = torch.rand(10, 3)
    with pytest.raises(RuntimeError,
                       match="`cosine` argument not supported on CPU"):
        pca.knn(x, x, 2, cosine=True)
    with pytest.raises(RuntimeError,
                       match="`cosine` argument not supported on CPU"):
        torch.ops.torch_cluster.knn(x, x, None, None, 2, True, 1)


@pytest.mark.parametrize("d,k", [(1, 3), (2, 16), (3, 17), (5, 8), (8, 32),
                                 (9, 5), (40, 12), (130, 100)])
def test_knn_matches_the_checker(oracle, d, k):
    rng = np.random.default_rng(d * 13 + k)
    x = rng.standard_normal((3000, d)).astype(np.float32)
    y = rng.standard_normal((400, d)).astype(np.float32)
    ptr_x = np.array([0, 60, 60, 1400, 3000])
    ptr_y = np.array([0, 100, 130, 131, 400])
    want = oracle.knn_op(x, y, ptr_x, ptr_y, k, False, fma_mode=1)
    got = torch.ops.torch_cluster.knn(
        torch.from_numpy(x), torch.from_numpy(y), torch.from_numpy(ptr_x),
        torch.from_numpy(ptr_y), k, False, 3)
    assert got.shape == want.shape and (got.numpy() == want).all()


def test_knn_ties_nan_and_sentinel(oracle):
    # integer grid: exact ties, settled by row number
    rng = np.random.default_rng(5)
    x = rng.integers(0, 4, (2000, 3)).astype(np.float32)
    y = rng.integers(0, 4, (150, 3)).astype(np.float32)
    want = oracle.knn_op(x, y, None, None, 40, False, fma_mode=1)
    got = pca.knn(torch.from_numpy(x), torch.from_numpy(y), 40)
    assert (got.numpy() == want).all()
    # rows with NaN / infinite coordinates and rows beyond the 1e10 limit are
    # never returned; a NaN query has no neighbours
    x = rng.standard_normal((300, 3)).astype(np.float32)
    x[3, 1] = np.nan
    x[10] = np.inf
    x[20] = 2e5      # squared distance 1.2e11
    y = x[:50].copy()
    y[7] = np.nan
    want = oracle.knn_op(x, y, None, None, 100, False, fma_mode=1)
    got = pca.knn(torch.from_numpy(x), torch.from_numpy(y), 100)
    assert got.shape == want.shape and (got.numpy() == want).all()


@pytest.mark.parametrize("d", [1, 3, 8, 20])
@pytest.mark.parametrize("cap,ignore", [(4, False), (32, True), (1000, True)])
def test_radius_matches_the_checker(oracle, d, cap, ignore):
    rng = np.random.default_rng(d + cap)
    x = rng.random((2500, d)).astype(np.float32)
    ptr = np.array([0, 900, 900, 2500])
    r = 0.25 * d ** 0.5
    want = oracle.radius_op(x, x, ptr, ptr, r, cap, 1, ignore)
    got = torch.ops.torch_cluster.radius(
        torch.from_numpy(x), torch.from_numpy(x), torch.from_numpy(ptr),
        torch.from_numpy(ptr), r, cap, 2, ignore)
    assert got.shape == want.shape and (got.numpy() == want).all()
    # a sparse result has storage of its own
    assert got.untyped_storage().nbytes() <= max(16 * got.shape[1] * 2, 64)


@pytest.mark.parametrize("dtype,kind", [(torch.float16, 0),
                                        (torch.bfloat16, 1)])
def test_16bit_points(oracle, dtype, kind):
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(600, 4, generator=g) * 2).to(dtype)
    y = (torch.randn(70, 4, generator=g) * 2).to(dtype)
    ptr_x = np.array([0, 250, 600])
    ptr_y = np.array([0, 30, 70])
    want, _ = oracle.knn_op16(bits(x), bits(y), ptr_x, ptr_y, 9, False, kind)
    got = torch.ops.torch_cluster.knn(x, y, torch.from_numpy(ptr_x),
                                      torch.from_numpy(ptr_y), 9, False, 1)
    assert (got.numpy() == want).all()
    want = oracle.radius_op16(bits(x), bits(x), ptr_x, ptr_x, 1.5, 6, True,
                              kind)
    got = torch.ops.torch_cluster.radius(x, x, torch.from_numpy(ptr_x),
                                         torch.from_numpy(ptr_x), 1.5, 6, 1,
                                         True)
    assert got.shape == want.shape and (got.numpy() == want).all()


def test_fp64_and_integer_points(oracle):
    rng = np.random.default_rng(8)
    x = rng.standard_normal((800, 3))
    want = oracle.knn_op(x, x[:90], None, None, 6, False, fma_mode=1)
    got = pca.knn(torch.from_numpy(x), torch.from_numpy(x[:90]), 6)
    assert (got.numpy() == want).all()
    xi = rng.integers(-50, 50, (500, 3))
    want = oracle.knn_op(xi.astype(np.float64), xi[:40].astype(np.float64),
                         None, None, 5, False, fma_mode=1)
    got = pca.knn(torch.from_numpy(xi), torch.from_numpy(xi[:40]), 5)
    assert (got.numpy() == want).all()


def test_radius_graph_and_threads(oracle):
    c3 = testing.gaussian_mixture_batched(0, clouds=3, points=3000)
    before = torch.get_num_threads()
    try:
        for threads in (1, 4):
            torch.set_num_threads(threads)
            got = pca.radius_graph(c3["x"], 0.05, c3["batch"],
                                   max_num_neighbors=32)
            want = oracle.radius_graph(c3["x"].numpy(), 0.05,
                                       c3["batch"].numpy(),
                                       max_num_neighbors=32)
            assert got.shape == want.shape and (got.numpy() == want).all()
    finally:
        torch.set_num_threads(before)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("d", [1, 3, 7, 40])
def test_fps_on_the_cpu_matches_the_checker(oracle, dtype, d):
    rng = np.random.default_rng(d)
    x = rng.standard_normal((3000, d)).astype(dtype)
    ptr = np.array([0, 700, 700, 1001, 3000])
    for ratio in (0.25, [0.5, 1.0, 0.01, 0.1]):
        # the CPU operator sizes the samples in float, whatever the points'
        # type (csrc/cpu/fps_cpu.cpp:25-27)
        out_ptr = oracle.fps_out_ptr(ptr, ratio, np.float32)
        share = torch.tensor(ratio, dtype=torch.float32)
        got = torch.ops.torch_cluster.fps(torch.from_numpy(x),
                                          torch.from_numpy(ptr), share, False)
        want = oracle.fps_op(x, ptr, ratio)
        if dtype == np.float32:
            assert (got.numpy() == want).all()
        else:
            # (the checker sizes in the points' type: compare per example)
            mine = oracle.fps_out_ptr(ptr, ratio, np.float64)
            for b in range(4):
                n = min(out_ptr[b + 1] - out_ptr[b], mine[b + 1] - mine[b])
                assert (got.numpy()[out_ptr[b]:out_ptr[b] + n]
                        == want[mine[b]:mine[b] + n]).all()
        assert got.numel() == out_ptr[-1]


def test_fps_entry_point_on_the_cpu(oracle, ref):
    # the reference's fixture (test/test_fps.py:16-65) on CPU tensors
    x = torch.tensor([[-1.0, -1.0], [-1.0, 1.0], [1.0, 1.0], [1.0, -1.0],
                      [-2.0, -2.0], [-2.0, 2.0], [2.0, 2.0], [2.0, -2.0]])
    batch = torch.tensor([0, 0, 0, 0, 1, 1, 1, 1])
    assert pca.fps(x, batch, random_start=False).tolist() == [0, 2, 4, 6]
    assert pca.fps(x, batch, ratio=0.5,
                   random_start=False).tolist() == [0, 2, 4, 6]
    assert pca.fps(x, batch, ratio=torch.tensor([0.5, 0.5]),
                   random_start=False).tolist() == [0, 2, 4, 6]
    assert pca.fps(x, ptr=[0, 4, 8], ratio=0.5,
                   random_start=False).tolist() == [0, 2, 4, 6]
    assert pca.fps(x, random_start=False).sort()[0].tolist() == [0, 5, 6, 7]

    @torch.jit.script
    def fps2(x: torch.Tensor, ratio: torch.Tensor) -> torch.Tensor:
        return pca.fps(x, None, ratio, False)
    assert fps2(x, torch.tensor([0.5])).sort()[0].tolist() == [0, 5, 6, 7]
    # integer grid: exact ties, by the kernels' rule (slot of 256, then row)
    rng = np.random.default_rng(11)
    g = rng.integers(0, 5, (1500, 3)).astype(np.float32)
    ptr = np.array([0, 600, 1500])
    got = pca.fps(torch.from_numpy(g), ptr=torch.from_numpy(ptr), ratio=0.05,
                  random_start=False)
    assert (got.numpy() == oracle.fps_op(g, ptr, 0.05)).all()
    # a random start is a row of the example, and the rest follows from it
    torch.manual_seed(4)
    pts = rng.standard_normal((900, 3)).astype(np.float32)
    ptr = np.array([0, 300, 900])
    got = pca.fps(torch.from_numpy(pts), ptr=torch.from_numpy(ptr),
                  ratio=0.1).numpy()
    assert 0 <= got[0] < 300 and 300 <= got[30] < 900
    want = oracle.fps_op(pts, ptr, 0.1, start=[got[0], got[30] - 300])
    assert (got == want).all()
    # and the reference's compiled CPU operator, where no near-tie decides
    # (it sums the squares in another order)
    big = rng.standard_normal((4000, 3)).astype(np.float32)
    ptr = np.array([0, 1500, 4000])
    got = pca.fps(torch.from_numpy(big), ptr=torch.from_numpy(ptr),
                  ratio=0.05, random_start=False).numpy()
    want = ref.ref_fps(big, ptr, 0.05)
    assert got.shape == want.shape
    first_diff = np.flatnonzero(got != want)
    assert first_diff.size == 0 or first_diff[0] > 50


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("d", [1, 2, 3, 16, 100])
def test_nearest_on_the_cpu_matches_the_checker(oracle, dtype, d):
    rng = np.random.default_rng(d + 100)
    x = rng.standard_normal((5000, d)).astype(dtype)
    y = rng.standard_normal((1300, d)).astype(dtype)
    ptr_x = np.array([0, 1200, 1200, 5000])
    ptr_y = np.array([0, 300, 300, 1300])
    got = torch.ops.torch_cluster.nearest(
        torch.from_numpy(x), torch.from_numpy(y), torch.from_numpy(ptr_x),
        torch.from_numpy(ptr_y))
    assert (got.numpy() == oracle.nearest_op(x, y, ptr_x, ptr_y)).all()
    # brute force in float64 where no near-tie decides
    if dtype == np.float64:
        for b in (0, 2):
            xs = x[ptr_x[b]:ptr_x[b + 1]][:200]
            ys = y[ptr_y[b]:ptr_y[b + 1]]
            dd = ((xs[:, None, :] - ys[None, :, :]) ** 2).sum(-1)
            assert (got.numpy()[ptr_x[b]:ptr_x[b] + 200]
                    == dd.argmin(1) + ptr_y[b]).all()


def test_nearest_entry_point_on_the_cpu(oracle):
    # the reference's fixture (test/test_nearest.py:11-64) on CPU tensors
    x = torch.tensor([[-1.0, -1.0], [-1.0, 1.0], [1.0, 1.0], [1.0, -1.0],
                      [-2.0, -2.0], [-2.0, 2.0], [2.0, 2.0], [2.0, -2.0]])
    y = torch.tensor([[-1.0, 0.0], [1.0, 0.0], [-2.0, 0.0], [2.0, 0.0]])
    batch_x = torch.tensor([0, 0, 0, 0, 1, 1, 1, 1])
    batch_y = torch.tensor([0, 0, 1, 1])
    assert pca.nearest(x, y, batch_x, batch_y).tolist() \
        == [0, 0, 1, 1, 2, 2, 3, 3]
    assert pca.nearest(x, y).tolist() == [0, 0, 1, 1, 2, 2, 3, 3]
    with pytest.raises(ValueError, match="'batch_x' is not sorted"):
        pca.nearest(x, y, torch.tensor([0, 0, 1, 0, 1, 1, 1, 1]), batch_y)
    with pytest.raises(ValueError, match="do not occur in 'batch_y'"):
        pca.nearest(x, y, batch_x, torch.tensor([0, 0, 0, 0]))
    # ties (integer grid), NaN rows and rows beyond the 1e38 limit
    rng = np.random.default_rng(2)
    gx = rng.integers(0, 4, (3000, 2)).astype(np.float32)
    gy = rng.integers(0, 4, (2500, 2)).astype(np.float32)
    gy[5] = np.nan
    gy[9] = 3e19
    gx[17] = np.nan
    got = pca.nearest(torch.from_numpy(gx), torch.from_numpy(gy))
    assert (got.numpy() == oracle.nearest_op(gx, gy, [0, 3000],
                                             [0, 2500])).all()
    assert got[17] == 0  # nothing qualifies for a NaN row
