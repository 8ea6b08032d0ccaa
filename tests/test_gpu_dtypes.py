"""fp64 / fp16 / bf16 points on the GPU against the oracle, bit-exact, and the
reference's dtype-parametrised fixtures (test/test_knn.py:14,
test/test_radius.py:23 run over half, float, double and, for radius,
bfloat16)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

import pytorch_cluster_amd as pca  # noqa: E402
from pytorch_cluster_amd import capi  # noqa: E402
from gpu_common import DEV, ragged_ptrs  # noqa: E402
from helpers import to_set  # noqa: E402

DTYPES = [torch.float16, torch.bfloat16, torch.float32, torch.float64]


def bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def gpu_knn_t(x, y, ptr_x, ptr_y, k, cosine=False):
    px = None if ptr_x is None else torch.as_tensor(ptr_x).to(DEV)
    py = None if ptr_y is None else torch.as_tensor(ptr_y).to(DEV)
    e, _ = capi.knn_edges(x.to(DEV), y.to(DEV), px, py, k, cosine)
    return e.cpu().numpy()


def gpu_radius_t(x, y, ptr_x, ptr_y, r, cap, ignore=False):
    px = None if ptr_x is None else torch.as_tensor(ptr_x).to(DEV)
    py = None if ptr_y is None else torch.as_tensor(ptr_y).to(DEV)
    e = capi.radius_edges(x.to(DEV), y.to(DEV), px, py, r, cap, ignore)
    return e.cpu().numpy()


@pytest.mark.parametrize("dtype", DTYPES)
def test_reference_fixtures_all_dtypes(dtype):
    x = torch.tensor([[-1, -1], [-1, +1], [+1, +1], [+1, -1],
                      [-1, -1], [-1, +1], [+1, +1], [+1, -1]],
                     dtype=dtype, device=DEV)
    y = torch.tensor([[1, 0], [-1, 0]], dtype=dtype, device=DEV)
    bx = torch.tensor([0, 0, 0, 0, 1, 1, 1, 1], device=DEV)
    by = torch.tensor([0, 1], device=DEV)
    assert to_set(pca.knn(x, y, 2).cpu()) == {(0, 2), (0, 3), (1, 0), (1, 1)}
    assert to_set(pca.knn(x, y, 2, bx, by).cpu()) == \
        {(0, 2), (0, 3), (1, 4), (1, 5)}
    assert to_set(pca.knn(x, y, 2, bx, by, cosine=True).cpu()) == \
        {(0, 2), (0, 3), (1, 4), (1, 5)}
    y = torch.tensor([[0, 0], [0, 1]], dtype=dtype, device=DEV)
    assert to_set(pca.radius(x, y, 2, max_num_neighbors=4).cpu()) == \
        {(0, 0), (0, 1), (0, 2), (0, 3), (1, 1), (1, 2), (1, 5), (1, 6)}
    assert to_set(pca.radius(x, y, 2, bx, by, max_num_neighbors=4).cpu()) == \
        {(0, 0), (0, 1), (0, 2), (0, 3), (1, 5), (1, 6)}
    c = torch.tensor([[-1, -1], [-1, +1], [+1, +1], [+1, -1]], dtype=dtype,
                     device=DEV)
    e = pca.knn_graph(c, k=2, flow='target_to_source')
    assert to_set(e.cpu()) == {(0, 1), (0, 3), (1, 0), (1, 2), (2, 1), (2, 3),
                               (3, 0), (3, 2)}
    e = pca.radius_graph(c, r=2.5, flow='source_to_target')
    assert to_set(e.cpu()) == {(1, 0), (3, 0), (0, 1), (2, 1), (1, 2), (3, 2),
                               (0, 3), (2, 3)}


@pytest.mark.parametrize("d,k", [(3, 7), (2, 16), (5, 40), (40, 9),
                                 (200, 3)])
@pytest.mark.parametrize("cosine", [False, True])
@pytest.mark.parametrize("slices", [1, 6])
def test_knn_fp64_parity(oracle, monkeypatch, d, k, cosine, slices):
    # (slices of every segment's rows, whose lists a second kernel unites)
    monkeypatch.setenv("PCA_KNN_SLICES", str(slices))
    rng = np.random.default_rng(d * 31 + k)
    n, m = 1300, 400
    x = rng.standard_normal((n, d))
    y = rng.standard_normal((m, d))
    ptr_x = ragged_ptrs(rng, n, 4)
    ptr_y = ragged_ptrs(rng, m, 4)
    got = gpu_knn_t(torch.from_numpy(x), torch.from_numpy(y), ptr_x, ptr_y, k,
                    cosine)
    want = oracle.knn_op(x, y, ptr_x, ptr_y, k, cosine, fma_mode=1)
    assert got.shape == want.shape
    assert (got == want).all()


@pytest.mark.parametrize("dtype,kind", [(torch.float16, 0),
                                        (torch.bfloat16, 1)])
@pytest.mark.parametrize("d,k", [(3, 7), (2, 16), (6, 40), (40, 9)])
@pytest.mark.parametrize("cosine", [False, True])
@pytest.mark.parametrize("slices", [1, 5])
def test_knn_16bit_parity(oracle, monkeypatch, dtype, kind, d, k, cosine,
                          slices):
    monkeypatch.setenv("PCA_KNN_SLICES", str(slices))
    rng = np.random.default_rng(d * 17 + k + kind)
    n, m = 1100, 300
    # 16-bit arithmetic produces many exactly equal distances: the order by
    # (distance, row) must still match
    x = torch.from_numpy(rng.standard_normal((n, d))).to(dtype)
    y = torch.from_numpy(rng.standard_normal((m, d))).to(dtype)
    ptr_x = ragged_ptrs(rng, n, 3)
    ptr_y = ragged_ptrs(rng, m, 3)
    got = gpu_knn_t(x, y, ptr_x, ptr_y, k, cosine)
    want, _ = oracle.knn_op16(bits(x), bits(y), ptr_x, ptr_y, k, cosine, kind)
    assert got.shape == want.shape
    assert (got == want).all()


def test_knn_fp64_large_cloud_default_slices(oracle):
    # enough rows that the library slices on its own; duplicated rows, so that
    # equal distances meet across slice borders
    rng = np.random.default_rng(77)
    base = rng.standard_normal((6000, 3))
    x = np.concatenate([base, base[:3000], base[:1500]])
    y = base[::40] + 0.0
    got = gpu_knn_t(torch.from_numpy(x), torch.from_numpy(y), None, None, 12)
    want = oracle.knn_op(x, y, None, None, 12, False, fma_mode=1)
    assert (got == want).all()


def test_knn_fp16_overflowing_distances(oracle):
    # squared distances beyond 65504 are +inf in fp16 and never returned
    x = torch.tensor([[0.0], [10.0], [300.0], [-400.0]], dtype=torch.float16)
    y = torch.tensor([[0.0]], dtype=torch.float16)
    got = gpu_knn_t(x, y, None, None, 4)
    want, _ = oracle.knn_op16(bits(x), bits(y), None, None, 4, False, 0)
    assert got.tolist() == want.tolist() == [[0, 0], [0, 1]]


@pytest.mark.parametrize("dtype", [torch.float64, torch.float16,
                                   torch.bfloat16])
@pytest.mark.parametrize("d,cap,ignore", [(3, 8, True), (2, 64, False),
                                          (10, 5, False)])
def test_radius_other_dtypes_parity(oracle, dtype, d, cap, ignore):
    rng = np.random.default_rng(d + cap)
    n = 1500
    x = torch.from_numpy(rng.random((n, d))).to(dtype)
    ptr = ragged_ptrs(rng, n, 5)
    r = 0.5 * (40.0 / n) ** (1.0 / d)
    got = gpu_radius_t(x, x, ptr, ptr, r, cap, ignore)
    if dtype == torch.float64:
        want = oracle.radius_op(x.numpy(), x.numpy(), ptr, ptr, r, cap, 1,
                                ignore, fma_mode=1)
    else:
        kind = 0 if dtype == torch.float16 else 1
        want = oracle.radius_op16(bits(x), bits(x), ptr, ptr, r, cap, ignore,
                                  kind)
    assert got.shape == want.shape
    assert (got == want).all()


def test_distances_only_for_fp32():
    x = torch.rand(10, 3, dtype=torch.float64, device=DEV)
    with pytest.raises(capi.PcaError, match="fp32 points only"):
        capi.knn_edges(x, x, None, None, 2, want_dist=True)
