"""The committed golden vectors (tests/golden/) against the oracle (CPU) and
against the HIP path (GPU)."""
import json
import os

import numpy as np
import pytest

from helpers import to_set

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def fixtures():
    with open(os.path.join(GOLDEN, "reference_fixtures.json")) as f:
        return json.load(f)


def ref_vectors():
    return np.load(os.path.join(GOLDEN, "ref_cpu_vectors.npz"))


def arr(v, dtype):
    return None if v is None else np.asarray(v, dtype=dtype)


def check_edges(case, edge_index):
    e = np.asarray(edge_index)
    if case.get("ordered"):
        assert e.tolist() == case["edge_index"], case["source"]
    else:
        assert to_set(e) == {tuple(p) for p in case["edges"]}, case["source"]


# ---- CPU: the oracle ---------------------------------------------------------

def test_oracle_matches_reference_fixtures(oracle):
    fx = fixtures()
    for c in fx["knn"]:
        check_edges(c, oracle.knn(arr(c["x"], np.float32),
                                  arr(c["y"], np.float32), c["k"],
                                  arr(c["batch_x"], np.int64),
                                  arr(c["batch_y"], np.int64),
                                  cosine=c["cosine"]))
    for c in fx["knn_graph"]:
        check_edges(c, oracle.knn_graph(arr(c["x"], np.float32), c["k"],
                                        arr(c["batch"], np.int64),
                                        loop=c["loop"], flow=c["flow"]))
    for c in fx["radius"]:
        check_edges(c, oracle.radius(arr(c["x"], np.float32),
                                     arr(c["y"], np.float32), c["r"],
                                     arr(c["batch_x"], np.int64),
                                     arr(c["batch_y"], np.int64),
                                     max_num_neighbors=c["max_num_neighbors"]))
    for c in fx["radius_graph"]:
        check_edges(c, oracle.radius_graph(arr(c["x"], np.float32), c["r"],
                                           arr(c["batch"], np.int64),
                                           loop=c["loop"], flow=c["flow"]))


@pytest.mark.parametrize("fma_mode", [0, 1])
def test_oracle_matches_reference_cpu_vectors(oracle, fma_mode):
    v = ref_vectors()
    e = oracle.knn_op(v["knn3_x"], v["knn3_y"], v["knn3_ptr_x"],
                      v["knn3_ptr_y"], int(v["knn3_k"]), fma_mode=fma_mode)
    assert (e == v["knn3_edges"]).all()
    e = oracle.knn_op(v["knn16_x"], v["knn16_y"], None, None,
                      int(v["knn16_k"]), fma_mode=fma_mode)
    assert (e == v["knn16_edges"]).all()
    e = oracle.radius_op(v["rad_x"], v["rad_y"], v["rad_ptr_x"],
                         v["rad_ptr_y"], float(v["rad_r"]), int(v["rad_max"]),
                         fma_mode=fma_mode)
    assert (e == v["rad_edges"]).all()


# ---- GPU: the HIP path -------------------------------------------------------

@pytest.mark.gpu
def test_gpu_matches_reference_fixtures():
    import torch
    import pytorch_cluster_amd as pca
    dev = torch.device("cuda:0")

    def t(v, dtype=torch.float32):
        return None if v is None else torch.tensor(v, dtype=dtype, device=dev)

    fx = fixtures()
    for c in fx["knn"]:
        check_edges(c, pca.knn(t(c["x"]), t(c["y"]), c["k"],
                               t(c["batch_x"], torch.long),
                               t(c["batch_y"], torch.long),
                               cosine=c["cosine"]).cpu().numpy())
    for c in fx["knn_graph"]:
        check_edges(c, pca.knn_graph(t(c["x"]), c["k"],
                                     t(c["batch"], torch.long),
                                     loop=c["loop"],
                                     flow=c["flow"]).cpu().numpy())
    for c in fx["radius"]:
        check_edges(c, pca.radius(t(c["x"]), t(c["y"]), c["r"],
                                  t(c["batch_x"], torch.long),
                                  t(c["batch_y"], torch.long),
                                  max_num_neighbors=c["max_num_neighbors"])
                    .cpu().numpy())
    for c in fx["radius_graph"]:
        check_edges(c, pca.radius_graph(t(c["x"]), c["r"],
                                        t(c["batch"], torch.long),
                                        loop=c["loop"],
                                        flow=c["flow"]).cpu().numpy())


@pytest.mark.gpu
def test_gpu_matches_reference_cpu_vectors():
    from gpu_common import gpu_knn, gpu_radius
    v = ref_vectors()
    e, _ = gpu_knn(v["knn3_x"], v["knn3_y"], v["knn3_ptr_x"], v["knn3_ptr_y"],
                   int(v["knn3_k"]))
    assert (e == v["knn3_edges"]).all()
    e, _ = gpu_knn(v["knn16_x"], v["knn16_y"], None, None, int(v["knn16_k"]))
    assert (e == v["knn16_edges"]).all()
    e = gpu_radius(v["rad_x"], v["rad_y"], v["rad_ptr_x"], v["rad_ptr_y"],
                   float(v["rad_r"]), int(v["rad_max"]))
    assert (e == v["rad_edges"]).all()
