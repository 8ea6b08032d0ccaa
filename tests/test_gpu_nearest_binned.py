"""GPU parity of the binned `nearest` search (pca_nearest_binned through the
C ABI): the same rows as pca_nearest, i.e. as the reference kernel
(csrc/cuda/nearest_cuda.cu:10-66), its order among equal distances included.
Checked against the oracle, and against the scanning kernels at full size."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

import pytorch_cluster_amd as pca  # noqa: E402
from pytorch_cluster_amd import capi, testing  # noqa: E402
from gpu_common import DEV, dev, ragged_ptrs  # noqa: E402


def gpu_nearest_binned(x, y, ptr_x, ptr_y):
    out = capi.nearest_rows(dev(x), dev(y), dev(ptr_x, torch.long),
                            dev(ptr_y, torch.long), binned=True)
    torch.cuda.synchronize()
    return out.cpu().numpy()


@pytest.mark.parametrize("d", [1, 2, 3])
@pytest.mark.parametrize("segments", [1, 5])
def test_random_points(oracle, d, segments):
    rng = np.random.default_rng(1000 * d + segments)
    n, m = 3000, 2600
    x = rng.standard_normal((n, d)).astype(np.float32)
    y = rng.standard_normal((m, d)).astype(np.float32)
    ptr_x = ragged_ptrs(rng, n, segments)
    ptr_y = ragged_ptrs(rng, m, segments)
    got = gpu_nearest_binned(x, y, ptr_x if segments > 1 else None,
                             ptr_y if segments > 1 else None)
    want = oracle.nearest_op(x, y, ptr_x, ptr_y)
    assert (got == want).all()


@pytest.mark.parametrize("d", [2, 3])
def test_ties_follow_the_reference_block(oracle, d):
    """Integer grids: exact ties everywhere; candidate segments longer than
    1,024 rows, so the winner is often not the lowest row."""
    rng = np.random.default_rng(7 + d)
    sizes_y = [2500, 0, 1030, 5000]
    sizes_x = [700, 0, 64, 900]
    ptr_y = np.concatenate([[0], np.cumsum(sizes_y)]).astype(np.int64)
    ptr_x = np.concatenate([[0], np.cumsum(sizes_x)]).astype(np.int64)
    y = rng.integers(0, 4, (ptr_y[-1], d)).astype(np.float32)
    x = rng.integers(0, 4, (ptr_x[-1], d)).astype(np.float32)
    got = gpu_nearest_binned(x, y, ptr_x, ptr_y)
    want = oracle.nearest_op(x, y, ptr_x, ptr_y)
    assert (got == want).all()
    lowest = np.array([ptr_y[s] + np.argmin(((y[ptr_y[s]:ptr_y[s + 1]]
                                              - x[i]) ** 2).sum(1))
                       if ptr_y[s + 1] > ptr_y[s] else 0
                       for s in range(4) for i in range(ptr_x[s], ptr_x[s + 1])])
    assert (want != lowest).any()  # the rule is not "lowest row"


def test_nothing_found_and_rows_that_are_not_finite(oracle):
    rng = np.random.default_rng(3)
    x = rng.standard_normal((500, 3)).astype(np.float32)
    y = rng.standard_normal((800, 3)).astype(np.float32)
    x[3, 0] = np.nan
    x[4, 1] = np.inf
    x[5] = 1e20          # squared distances overflow the limit of 1e38
    y[10, 2] = np.nan
    y[11] = np.inf
    ptr_x = np.array([0, 200, 200, 500], dtype=np.int64)
    ptr_y = np.array([0, 300, 800, 800], dtype=np.int64)   # last one: no rows
    got = gpu_nearest_binned(x, y, ptr_x, ptr_y)
    want = oracle.nearest_op(x, y, ptr_x, ptr_y)
    assert (got == want).all()


def test_lidar_like_scans_against_the_scanning_kernel():
    c = testing.lidar_scans(0, query_stride=8)
    x, y = c["x"].to(DEV), c["y"].to(DEV)
    px = testing.pointers(c["batch_x"], 8).to(DEV)
    py = testing.pointers(c["batch_y"], 8).to(DEV)
    a = capi.nearest_rows(x, y, px, py)
    b = capi.nearest_rows(x, y, px, py, binned=True)
    assert torch.equal(a, b)


def test_strategy_switch_of_the_entry_point():
    g = torch.Generator().manual_seed(2)
    x = torch.rand(5000, 3, generator=g).to(DEV)
    y = torch.rand(1200, 3, generator=g).to(DEV)
    bx = torch.arange(2).repeat_interleave(2500).to(DEV)
    by = torch.arange(2).repeat_interleave(600).to(DEV)
    want = pca.nearest(x, y, bx, by)
    try:
        pca.set_search_strategy("binned")
        got = pca.nearest(x, y, bx, by)
        got16 = pca.nearest(x.half(), y.half(), bx, by)   # not binned: fp16
    finally:
        pca.set_search_strategy("scan")
    assert torch.equal(want, got)
    assert torch.equal(got16, pca.nearest(x.half(), y.half(), bx, by))


def test_more_than_three_dimensions_are_refused():
    x = torch.rand(100, 4, device=DEV)
    with pytest.raises(RuntimeError, match="binned search"):
        capi.nearest_rows(x, x, None, None, binned=True)


def test_graph_capture_takes_the_scanning_kernel():
    """A stream that is being captured never gets the binned search (its
    sorts would record memset nodes): the operator scans instead, the C entry
    point says so.  Replays give the eager result every time."""
    import pytorch_cluster_amd as pca
    from pytorch_cluster_amd import capi
    from pytorch_cluster_amd._native import capi as lib
    g = torch.Generator().manual_seed(3)
    n, m = 150000, 90000
    x = torch.rand(n, 3, generator=g).to(DEV)
    y = torch.rand(m, 3, generator=g).to(DEV)
    ptr_x = torch.tensor([0, 70000, n], device=DEV)
    ptr_y = torch.tensor([0, 40000, m], device=DEV)
    before = pca.get_search_strategy()
    pca.set_search_strategy("binned")
    try:
        op = torch.ops.torch_cluster.nearest
        want = op(x, y, ptr_x, ptr_y)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out = op(x, y, ptr_x, ptr_y)
            # the C entry point on the capturing stream: refused, nothing
            # recorded
            edges, num_edges, _d, _ws = None, None, None, None
            ws = torch.empty(lib.pca_nearest_binned_workspace_bytes(n, m, 3, 2),
                             dtype=torch.uint8, device=DEV)
            res = torch.empty(n, dtype=torch.long, device=DEV)
            rc = lib.pca_nearest_binned(
                capi._dev_ptr(x), capi._dev_ptr(y), capi._dev_ptr(ptr_x),
                capi._dev_ptr(ptr_y), n, m, 3, 2, capi._dev_ptr(res),
                capi._dev_ptr(ws), ws.numel(),
                capi._stream_handle(None, x.device))
            assert rc == -5 and b"captured" in lib.pca_last_error()
        for _ in range(3):
            out.zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, want)
            # (eager work between the replays)
            assert torch.equal(op(x, y, ptr_x, ptr_y), want)
    finally:
        pca.set_search_strategy(before)
