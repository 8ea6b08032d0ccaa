"""CPU-side tests: the C-ABI library loads and exports what the header
declares, argument validation that returns before any GPU work, the Python
entry points' host logic (with the search operator replaced by the oracle),
TorchScript compilation, and loud failure for tensors that are not on a GPU.
"""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

import pytorch_cluster_amd as pca
from pytorch_cluster_amd import _native
from helpers import to_set

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_header_symbols_are_exported():
    header = open(os.path.join(ROOT, "include", "pca_neighbors.h")).read()
    declared = set(re.findall(r"\b(pca_[a-z0-9_]+)\s*\(", header))
    assert declared, "no declarations found"
    lib = ctypes.CDLL(_native.CAPI_PATH)
    for name in sorted(declared):
        assert hasattr(lib, name), "missing export: " + name
    assert declared == set(_native.C_ABI), "ctypes table out of date"
    assert lib.pca_abi_version() == 5


def test_capi_validation_needs_no_gpu():
    capi = _native.capi
    one = ctypes.c_void_p(256)  # never dereferenced on these paths
    # k > 100 -> the reference's message (csrc/cuda/knn_cuda.cu:98)
    rc = capi.pca_knn(one, one, None, None, 10, 10, 3, 1, 101, 0, 0, 0, one, one,
                      None, one, 1 << 20, None)
    assert rc == -2
    assert b"smaller than or equal to 100" in capi.pca_last_error()
    rc = capi.pca_knn(one, one, one, None, 10, 10, 3, 1, 4, 0, 0, 0, one, one,
                      None, one, 1 << 20, None)
    assert rc == -1  # only one ptr given
    rc = capi.pca_knn(one, one, None, None, 10, 10, 3, 1, 4, 0, 0, 0, one, one,
                      None, one, 16, None)
    assert rc == -3  # workspace too small
    rc = capi.pca_knn(one, one, None, None, 10, 10, 3, 1, 4, 0, 7, 0, one, one,
                      None, one, 1 << 20, None)
    assert rc == -5  # no such element type
    rc = capi.pca_knn(one, one, None, None, 10, 10, 3, 1, 4, 0, 1, 0, one, one,
                      one, one, 1 << 20, None)
    assert rc == -5  # distances are written for fp32 points only
    rc = capi.pca_radius(one, one, None, None, 10, 10, 3, 1, 0.5, 0, 0, 0,
                         0, one, one, one, 1 << 20, None)
    assert rc == -1  # max_num_neighbors must be >= 1
    assert capi.pca_knn_workspace_bytes(100, 100, 3, 1, 101, 0) == 0
    assert capi.pca_knn_workspace_bytes(100, 100, 3, 1, 16, 0) > 100 * 16 * 8
    assert capi.pca_radius_slots(10, 32) == 10
    assert capi.pca_radius_slots(100, 32) == 32
    assert capi.pca_status_string(0) == b"ok"


def test_operators_are_registered_and_scriptable():
    assert torch.ops.torch_cluster.cuda_version() > 0
    for fn in (pca.knn, pca.knn_graph, pca.radius, pca.radius_graph):
        torch.jit.script(fn)
    schema = str(torch.ops.torch_cluster.knn.default._schema)
    assert "Tensor? ptr_x" in schema and "bool cosine" in schema
    schema = str(torch.ops.torch_cluster.radius.default._schema)
    assert "float r" in schema and "bool ignore_same_index" in schema


def test_operators_refuse_tensors_of_mixed_devices():
    # (every operator takes CPU tensors; what it refuses is a mix)
    x = torch.rand(8, 3)
    meta = torch.empty(8, 3, device="meta")
    with pytest.raises(RuntimeError):
        torch.ops.torch_cluster.nearest(x, meta, torch.tensor([0, 8]),
                                        torch.tensor([0, 8]))
    # half-precision points are searched in float on the host
    got = torch.ops.torch_cluster.nearest(x.half(), x.half(),
                                          torch.tensor([0, 8]),
                                          torch.tensor([0, 8]))
    assert got.tolist() == list(range(8))


def test_empty_inputs_short_circuit():
    x = torch.rand(0, 3)
    y = torch.rand(4, 3)
    assert pca.knn(x, y, 2).shape == (2, 0)
    assert pca.radius(y, x, 1.0).shape == (2, 0)
    assert pca.knn(x, y, 2).dtype == torch.long


@pytest.fixture
def oracle_ops(monkeypatch, oracle):
    """Replaces the two search operators with the CPU oracle so the host
    logic of the Python entry points can be exercised without a GPU."""
    calls = []

    def fake_knn(x, y, ptr_x, ptr_y, k, cosine, num_workers):
        assert x.is_contiguous() and y.is_contiguous() and x.dim() == 2
        calls.append(("knn", ptr_x, ptr_y, k))
        px = None if ptr_x is None else ptr_x.numpy()
        py = None if ptr_y is None else ptr_y.numpy()
        return torch.from_numpy(oracle.knn_op(x.numpy(), y.numpy(), px, py, k,
                                              cosine))

    def fake_radius(x, y, ptr_x, ptr_y, r, max_nn, num_workers, ignore):
        assert x.is_contiguous() and y.is_contiguous() and x.dim() == 2
        calls.append(("radius", ptr_x, ptr_y, max_nn, ignore))
        px = None if ptr_x is None else ptr_x.numpy()
        py = None if ptr_y is None else ptr_y.numpy()
        return torch.from_numpy(oracle.radius_op(x.numpy(), y.numpy(), px, py,
                                                 r, max_nn, 1, ignore))

    # the variants the graph entry points call: the operator's edges without
    # self-pairs and / or with the x row first
    def finish(edges, drop_self, x_first):
        if drop_self:
            edges = edges[:, edges[0] != edges[1]]
        return edges.flip(0) if x_first else edges

    def fake_knn_edges(x, y, ptr_x, ptr_y, k, cosine, drop_self, x_first):
        return finish(fake_knn(x, y, ptr_x, ptr_y, k, cosine, 1), drop_self,
                      x_first)

    def fake_radius_edges(x, y, ptr_x, ptr_y, r, max_nn, ignore, x_first):
        return finish(fake_radius(x, y, ptr_x, ptr_y, r, max_nn, 1, ignore),
                      False, x_first)

    monkeypatch.setattr(torch.ops.torch_cluster, "knn", fake_knn)
    monkeypatch.setattr(torch.ops.torch_cluster, "radius", fake_radius)
    monkeypatch.setattr(torch.ops.pytorch_cluster_amd, "knn_edges",
                        fake_knn_edges)
    monkeypatch.setattr(torch.ops.pytorch_cluster_amd, "radius_edges",
                        fake_radius_edges)
    return calls


def test_wrappers_match_oracle_entry_points(oracle_ops, oracle):
    g = torch.Generator().manual_seed(0)
    x = torch.rand(600, 3, generator=g)
    y = torch.rand(90, 3, generator=g)
    bx = torch.tensor([0] * 200 + [2] * 150 + [3] * 250)
    by = torch.tensor([0] * 30 + [1] * 10 + [3] * 50)
    for kwargs in ({}, {"batch_size": 4}, {"batch_size": 6}):
        got = pca.knn(x, y, 5, bx, by, **kwargs)
        want = oracle.knn(x.numpy(), y.numpy(), 5, bx.numpy(), by.numpy(),
                          **kwargs)
        assert got.numpy().tolist() == want.tolist()
        got = pca.radius(x, y, 0.2, bx, by, max_num_neighbors=6, **kwargs)
        want = oracle.radius(x.numpy(), y.numpy(), 0.2, bx.numpy(),
                             by.numpy(), max_num_neighbors=6, **kwargs)
        assert got.numpy().tolist() == want.tolist()
    # the pointers handed to the operator: first row of each example id
    name, ptr_x, ptr_y, _k = [c for c in oracle_ops if c[0] == "knn"][0]
    assert ptr_x.tolist() == [0, 200, 200, 350, 600]
    assert ptr_y.tolist() == [0, 30, 40, 40, 90]

    for flow in ("source_to_target", "target_to_source"):
        for loop in (False, True):
            got = pca.knn_graph(x, 4, bx, loop=loop, flow=flow)
            want = oracle.knn_graph(x.numpy(), 4, bx.numpy(), loop=loop,
                                    flow=flow)
            assert got.numpy().tolist() == want.tolist()
            got = pca.radius_graph(x, 0.15, bx, loop=loop, flow=flow,
                                   max_num_neighbors=7)
            want = oracle.radius_graph(x.numpy(), 0.15, bx.numpy(), loop=loop,
                                       flow=flow, max_num_neighbors=7)
            assert got.numpy().tolist() == want.tolist()


def test_wrappers_one_dimensional_and_single_example(oracle_ops):
    x = torch.tensor([0.0, 1.0, 3.0, 7.0])
    e = pca.knn_graph(x, 1)
    assert oracle_ops[-1][1] is None  # no pointers for one example
    assert to_set(e.numpy()) == {(1, 0), (0, 1), (1, 2), (2, 3)}
    # non-contiguous input is made contiguous before the operator sees it
    xt = torch.rand(3, 50).t()
    assert not xt.is_contiguous()
    assert pca.knn(xt, xt, 2).shape == (2, 100)


def test_reference_fixtures_through_wrappers(oracle_ops):
    # test/test_knn.py:57-75 and README.md:188-191 (ordered)
    x = torch.tensor([[-1., -1.], [-1., 1.], [1., -1.], [1., 1.]])
    batch = torch.zeros(4, dtype=torch.long)
    want = [[1, 2, 0, 3, 0, 3, 1, 2], [0, 0, 1, 1, 2, 2, 3, 3]]
    assert pca.knn_graph(x, k=2, batch=batch, loop=False).tolist() == want
    assert pca.radius_graph(x, r=2.5, batch=batch, loop=False).tolist() == want


def test_knn_graph_keeps_k_plus_one_for_duplicates(oracle_ops):
    # reference quirk (torch_cluster/knn.py:132,140-142): a point whose k+1
    # nearest do not include itself keeps k+1 edges
    x = torch.zeros(5, 2)
    e = pca.knn_graph(x, 2, flow="target_to_source")
    counts = np.bincount(e[0].numpy(), minlength=5).tolist()
    assert counts == [2, 2, 2, 3, 3]
