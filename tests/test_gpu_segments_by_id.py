"""Segments given as the rows' sorted example ids (PCA_SEGMENTS_BY_ID): the
pointers are derived on the device, inside the launch that prepares a search.
Parity with the same search given the pointers -- and through that with the
CPU checker -- on every kernel family that plans its work differently, with
examples that have no rows at all on one or both sides.
"""
import numpy as np
import pytest
import torch

import pytorch_cluster_amd as pca
from pytorch_cluster_amd import capi
from gpu_common import (DEV, dev, gpu_knn, gpu_radius, oracle_knn_edges,
                        ragged_ptrs)

pytestmark = pytest.mark.gpu


def _ids(ptr):
    return np.repeat(np.arange(len(ptr) - 1), np.diff(ptr)).astype(np.int64)


def test_segment_pointers_entry_point():
    rng = np.random.default_rng(0)
    for segments, n, m in ((1, 10, 7), (5, 1000, 40), (70, 5000, 9000),
                           (3000, 20000, 500)):
        ptr_x = ragged_ptrs(rng, n, segments)
        ptr_y = ragged_ptrs(rng, m, segments)
        gx, gy = capi.segment_pointers(dev(_ids(ptr_x)), dev(_ids(ptr_y)),
                                       segments)
        torch.cuda.synchronize()
        assert gx.cpu().numpy().tolist() == ptr_x.tolist()
        assert gy.cpu().numpy().tolist() == ptr_y.tolist()


@pytest.mark.parametrize("d,k,cosine,dtype", [
    (3, 16, False, np.float32),     # matrix-core scan, plan inside its set-up
    (3, 40, False, np.float32),     # vector-ALU scan
    (2, 8, True, np.float32),       # cosine scan
    (40, 12, False, np.float32),    # fp16 filter on the matrix cores
    (700, 5, False, np.float32),    # any-dimension kernel
    (3, 9, False, np.float64),      # any-type kernel
])
def test_knn_by_id_matches_pointers(oracle, d, k, cosine, dtype):
    rng = np.random.default_rng(d * 3 + k)
    n, m, segments = 6000, 1500, 6
    x = rng.standard_normal((n, d)).astype(dtype)
    y = rng.standard_normal((m, d)).astype(dtype)
    ptr_x = ragged_ptrs(rng, n, segments)
    ptr_y = ragged_ptrs(rng, m, segments)
    want, _ = capi.knn_edges(dev(x), dev(y), dev(ptr_x), dev(ptr_y), k, cosine)
    got, _ = capi.knn_edges(dev(x), dev(y), dev(_ids(ptr_x)), dev(_ids(ptr_y)),
                            k, cosine, ids_examples=segments)
    torch.cuda.synchronize()
    assert got.shape == want.shape and (got == want).all()
    if dtype == np.float32:
        ref, _ = oracle_knn_edges(oracle, x, y, ptr_x, ptr_y, k, cosine)
        assert (got.cpu().numpy() == ref).all()
    # the graph options ride along
    want, _ = capi.knn_edges(dev(x), dev(x), dev(ptr_x), dev(ptr_x), k, cosine,
                             drop_self=True, x_first=True)
    got, _ = capi.knn_edges(dev(x), dev(x), dev(_ids(ptr_x)), dev(_ids(ptr_x)),
                            k, cosine, drop_self=True, x_first=True,
                            ids_examples=segments)
    torch.cuda.synchronize()
    assert got.shape == want.shape and (got == want).all()


@pytest.mark.parametrize("mc", ["0", "1"])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_radius_by_id_matches_pointers(oracle, monkeypatch, mc, dtype):
    monkeypatch.setenv("PCA_RADIUS_MATRIX_CORES", mc)
    rng = np.random.default_rng(5)
    n, m, segments = 5000, 2000, 5
    x = rng.random((n, 3)).astype(dtype)
    y = rng.random((m, 3)).astype(dtype)
    ptr_x = ragged_ptrs(rng, n, segments)
    ptr_y = ragged_ptrs(rng, m, segments)
    want = capi.radius_edges(dev(x), dev(y), dev(ptr_x), dev(ptr_y), 0.12, 20)
    got = capi.radius_edges(dev(x), dev(y), dev(_ids(ptr_x)), dev(_ids(ptr_y)),
                            0.12, 20, ids_examples=segments)
    torch.cuda.synchronize()
    assert got.shape == want.shape and (got == want).all()
    if dtype == np.float32:
        ref = oracle.radius_op(x, y, ptr_x, ptr_y, 0.12, 20, 1, False)
        assert (got.cpu().numpy() == ref).all()


def test_fixed_scratch_entry_point_takes_ids(oracle):
    rng = np.random.default_rng(8)
    x = rng.random((3000, 3)).astype(np.float32)
    ptr = ragged_ptrs(rng, 3000, 4)
    want, _ = capi.knn_edges(dev(x), dev(x), dev(ptr), dev(ptr), 10)
    got, _ = capi.knn_edges(dev(x), dev(x), dev(_ids(ptr)), dev(_ids(ptr)), 10,
                            fixed_scratch=True, ids_examples=4)
    torch.cuda.synchronize()
    assert (got == want).all()


@pytest.mark.parametrize("strategy", ["scan", "binned", "auto"])
def test_wrappers_with_batch_size_take_the_id_path(oracle, strategy):
    # with batch_size the Python entry points hand the example ids over as
    # they are; without it they go through pointers: same edges
    rng = np.random.default_rng(11)
    n = 40000
    x = torch.from_numpy(rng.random((n, 3)).astype(np.float32)).to(DEV)
    ptr = ragged_ptrs(rng, n, 5)
    batch = torch.from_numpy(_ids(ptr)).to(DEV)
    y = x[::7].contiguous()
    by = batch[::7].contiguous()
    before = pca.get_search_strategy()
    pca.set_search_strategy(strategy)
    try:
        for loop in (False, True):
            for flow in ("source_to_target", "target_to_source"):
                a = pca.knn_graph(x, 6, batch, loop=loop, flow=flow,
                                  batch_size=5)
                b = pca.knn_graph(x, 6, batch, loop=loop, flow=flow)
                assert a.shape == b.shape and (a == b).all()
                a = pca.radius_graph(x, 0.02, batch, loop=loop, flow=flow,
                                     batch_size=5, max_num_neighbors=12)
                b = pca.radius_graph(x, 0.02, batch, loop=loop, flow=flow,
                                     max_num_neighbors=12)
                assert a.shape == b.shape and (a == b).all()
        a = pca.knn(x, y, 9, batch, by, batch_size=5)
        b = pca.knn(x, y, 9, batch, by)
        assert (a == b).all()
        want = oracle.knn(x.cpu().numpy(), y.cpu().numpy(), 9,
                          batch.cpu().numpy(), by.cpu().numpy())
        assert (a.cpu().numpy() == want).all()
        a = pca.radius(x, y, 0.03, batch, by, max_num_neighbors=15,
                       batch_size=5)
        b = pca.radius(x, y, 0.03, batch, by, max_num_neighbors=15)
        assert (a == b).all()
        # a batch_size beyond the ids in use: trailing examples without rows
        a = pca.knn(x, y, 9, batch, by, batch_size=9)
        assert (a == b.new_tensor(want)).all()
    finally:
        pca.set_search_strategy(before)


def test_scripted_wrappers_take_the_id_path():
    x = torch.rand(3000, 3, device=DEV)
    batch = torch.arange(3000, device=DEV) // 1000
    f = torch.jit.script(pca.knn_graph)
    g = torch.jit.script(pca.radius_graph)
    assert (f(x, 4, batch, batch_size=3) == pca.knn_graph(x, 4, batch)).all()
    assert (g(x, 0.1, batch, batch_size=3)
            == pca.radius_graph(x, 0.1, batch)).all()


@pytest.mark.parametrize("strategy", ["scan", "binned"])
def test_batch_size_below_the_ids_in_use(oracle, strategy):
    # a batch_size smaller than the largest id + 1: the reference's lookup
    # (csrc/cuda/utils.cuh:11-19) hands the queries of the examples beyond it
    # to the last example it knows, and the rows of those examples are never
    # searched; the id path does the same, for every kernel that plans its
    # work differently
    rng = np.random.default_rng(31)
    before = pca.get_search_strategy()
    pca.set_search_strategy(strategy)
    try:
        for d, k in ((3, 7), (40, 5), (3, 40)):
            n = 12000
            x = rng.random((n, d)).astype(np.float32)
            ptr = ragged_ptrs(rng, n, 6)
            batch = _ids(ptr)
            y, by = x[::5].copy(), batch[::5].copy()
            xd, yd = dev(x), dev(y)
            bd, byd = dev(batch), dev(by)
            for size in (4, 2):
                got = pca.knn(xd, yd, k, bd, byd, batch_size=size)
                want = oracle.knn(x, y, k, batch, by, batch_size=size)
                assert got.shape == want.shape
                assert (got.cpu().numpy() == want).all()
                got = pca.knn_graph(xd, k, bd, batch_size=size)
                want = oracle.knn_graph(x, k, batch, batch_size=size)
                assert got.shape == want.shape
                assert (got.cpu().numpy() == want).all()
            if d == 3:
                got = pca.radius(xd, yd, 0.05, bd, byd, max_num_neighbors=9,
                                 batch_size=3)
                want = oracle.radius(x, y, 0.05, batch, by,
                                     max_num_neighbors=9, batch_size=3)
                assert got.shape == want.shape
                assert (got.cpu().numpy() == want).all()
    finally:
        pca.set_search_strategy(before)


def test_default_calls_wait_for_the_device_once(oracle):
    # without batch_size the reference reads the number of examples from the
    # device before it starts (two reductions, two waits).  Here the search
    # starts with the number the previous call met and the launch that
    # derives the pointers reports the real one: a call waits for the device
    # once (for its edge count) -- twice when the number grew, and only the
    # first call of a process reads the ids' last entries up front
    waits = torch.ops.pytorch_cluster_amd.host_waits
    rng = np.random.default_rng(41)
    n = 9000
    x = rng.random((n, 3)).astype(np.float32)

    def clouds(count):
        ptr = ragged_ptrs(rng, n, count)
        return _ids(ptr)

    xd = dev(x)
    first = clouds(5)
    pca.knn_graph(xd, 4, dev(first))          # (whatever the process did before)
    for count, expected in ((5, 1), (5, 1), (3, 1), (3, 1), (9, 2), (9, 1),
                            (1, 1), (2, 2)):
        batch = clouds(count)
        bd = dev(batch)
        before = waits()
        got = pca.knn_graph(xd, 6, bd)
        assert waits() - before == expected, (count, waits() - before)
        want = oracle.knn_graph(x, 6, batch)
        assert got.shape == want.shape and (got.cpu().numpy() == want).all()
    # radius_graph, knn and radius share the number
    batch = clouds(4)
    bd = dev(batch)
    pca.knn_graph(xd, 3, bd)
    y, by = x[::3].copy(), batch[::3].copy()
    for call, ref in (
            (lambda: pca.radius_graph(xd, 0.05, bd, max_num_neighbors=7),
             lambda: oracle.radius_graph(x, 0.05, batch, max_num_neighbors=7)),
            (lambda: pca.knn(xd, dev(y), 5, bd, dev(by)),
             lambda: oracle.knn(x, y, 5, batch, by)),
            (lambda: pca.radius(xd, dev(y), 0.04, bd, dev(by),
                                max_num_neighbors=6),
             lambda: oracle.radius(x, y, 0.04, batch, by,
                                   max_num_neighbors=6))):
        before = waits()
        got = call()
        assert waits() - before == 1
        want = ref()
        assert got.shape == want.shape and (got.cpu().numpy() == want).all()
    # the binned searches take the same road
    before_strategy = pca.get_search_strategy()
    pca.set_search_strategy("binned")
    try:
        for count, expected in ((4, 1), (7, 2), (7, 1)):
            batch = clouds(count)
            before = waits()
            got = pca.knn_graph(xd, 6, dev(batch))
            assert waits() - before == expected
            want = oracle.knn_graph(x, 6, batch)
            assert (got.cpu().numpy() == want).all()
    finally:
        pca.set_search_strategy(before_strategy)
