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
@pytest.mark.parametrize("slices", [1, 5, "filter"])
def test_knn_16bit_parity(oracle, monkeypatch, dtype, kind, d, k, cosine,
                          slices):
    # the exhaustive 16-bit kernel in one slice and in five, and what runs by
    # default (Euclidean: the matrix-core filter in front of the same chain)
    if slices == "filter":
        if cosine:
            pytest.skip("the cosine distance of 16-bit rows has no filter")
    else:
        monkeypatch.setenv("PCA_KNN_SLICES", str(slices))
        monkeypatch.setenv("PCA_KNN_FEAT_16BIT", "0")
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


def _knn16_case(rng, kind, n, m, d, dtype):
    x = rng.standard_normal((n, d))
    y = rng.standard_normal((m, d))
    if kind == "rows_as_queries":
        y[: m // 2] = x[rng.integers(0, n, m // 2)]
    elif kind == "duplicates":
        x = x[rng.integers(0, 40, n)]
        y = x[rng.integers(0, n, m)] + 0.0
    elif kind == "one_large_component":
        # sums that stop growing: the first term is worth hundreds of the rest
        x[:, 0] *= 60.0
        y[:, 0] *= 60.0
    elif kind == "overflow":
        # squared distances around and beyond the largest fp16 number
        x *= 25.0
        y *= 25.0
    elif kind == "tiny":
        x *= 2e-4
        y *= 2e-4
    elif kind == "large_rows_and_queries":
        x[rng.integers(0, n, 5)] *= 300.0
        y[[0, m - 1]] *= 500.0
    elif kind == "not_finite":
        x[3, 1] = np.nan
        x[n // 2] = np.inf
        y[5, 0] = np.nan
        y[6, 2] = -np.inf
    elif kind == "grid":
        x = np.round(x)
        y = np.round(y)
    return (torch.from_numpy(x).to(dtype), torch.from_numpy(y).to(dtype))


@pytest.mark.parametrize("dtype,kind16", [(torch.float16, 0),
                                          (torch.bfloat16, 1)])
@pytest.mark.parametrize("kind", ["plain", "rows_as_queries", "duplicates",
                                  "one_large_component", "overflow", "tiny",
                                  "large_rows_and_queries", "not_finite",
                                  "grid"])
def test_knn_16bit_feature_space_parity(oracle, dtype, kind16, kind):
    # 16-bit rows of 9 to 128 components: the matrix-core filter in
    # front of the exact 16-bit chain (knn_feat_small_impl.hpp), against the
    # checker's chain; the 16-bit sums produce many equal distances
    rng = np.random.default_rng(len(kind) * 7 + kind16)
    dims = (9, 20, 64, 100, 128) if kind16 == 0 else (9, 33, 64, 100, 128)
    for d in dims:
        n, m = 2600, 420
        x, y = _knn16_case(rng, kind, n, m, d, dtype)
        ptr_x = np.array([0, 40, 40, 1500, n])
        ptr_y = np.array([0, 30, 50, 300, m])
        for k in ((1, 20, 41) if d % 2 else (8, 32, 48)):
            got = gpu_knn_t(x, y, ptr_x, ptr_y, k)
            want, _ = oracle.knn_op16(bits(x), bits(y), ptr_x, ptr_y, k, False,
                                      kind16)
            assert got.shape == want.shape, (d, k)
            assert (got == want).all(), (d, k)


def test_knn_16bit_feature_space_same_edges_without_the_filter(monkeypatch):
    # one larger call against the exhaustive 16-bit scan of the library itself
    g = torch.Generator().manual_seed(5)
    x = torch.randn(24 * 900, 64, generator=g).to(torch.float16)
    ptr = np.arange(25) * 900
    with_filter = gpu_knn_t(x, x, ptr, ptr, 21)
    monkeypatch.setenv("PCA_KNN_FEAT_16BIT", "0")
    without = gpu_knn_t(x, x, ptr, ptr, 21)
    assert with_filter.shape == without.shape == (2, 24 * 900 * 21)
    assert (with_filter == without).all()


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


@pytest.mark.parametrize("dtype,kind16", [(torch.float16, 0),
                                          (torch.bfloat16, 1)])
@pytest.mark.parametrize("kind", ["plain", "rows_as_queries", "duplicates",
                                  "one_large_component", "overflow", "tiny",
                                  "large_rows_and_queries", "not_finite",
                                  "grid"])
def test_radius_16bit_feature_space_parity(oracle, monkeypatch, dtype, kind16,
                                           kind):
    # the radius search on 16-bit rows of 9 to 128 components
    # through the matrix-core filter, against the checker's 16-bit chain:
    # radii around the typical distance, so that both "fewer than the limit"
    # and "the first 32 in row order" occur
    monkeypatch.setenv("PCA_RADIUS_FEAT", "1")
    rng = np.random.default_rng(len(kind) * 5 + kind16)
    dims = (9, 20, 64, 100, 128) if kind16 == 0 else (9, 33, 64, 100, 128)
    for d in dims:
        n, m = 2600, 420
        x, y = _knn16_case(rng, kind, n, m, d, dtype)
        ptr_x = np.array([0, 40, 40, 1500, n])
        ptr_y = np.array([0, 30, 50, 300, m])
        scale = {"one_large_component": 60.0, "overflow": 25.0,
                 "tiny": 2e-4}.get(kind, 1.0)
        base = scale * float(np.sqrt(2.0 * d))
        if kind == "one_large_component":
            base = scale * 1.0
        for r, cap, ignore in ((0.8 * base, 32, False), (1.05 * base, 9, True),
                               (0.9 * base, 1, False)):
            got = gpu_radius_t(x, y, ptr_x, ptr_y, r, cap, ignore)
            want = oracle.radius_op16(bits(x), bits(y), ptr_x, ptr_y, r, cap,
                                      ignore, kind16)
            assert got.shape == want.shape, (d, r, cap)
            assert (got == want).all(), (d, r, cap)


def test_distances_only_for_fp32():
    x = torch.rand(10, 3, dtype=torch.float64, device=DEV)
    with pytest.raises(capi.PcaError, match="fp32 points only"):
        capi.knn_edges(x, x, None, None, 2, want_dist=True)


def test_bf16_rounding_of_every_float():
    """The 16-bit searches round to bfloat16 with the device's conversion
    instruction; c10::BFloat16 (torch/headeronly/util/BFloat16.h,
    round_to_nearest_even) is an integer formula.  The probe library compares
    the two on all 2^32 bit patterns, NaNs included."""
    import ctypes
    import os
    lib = ctypes.CDLL(os.path.join(os.path.dirname(pca.__file__),
                                   "libpca_probe.so"))
    out = (ctypes.c_ulonglong * 2)()
    assert lib.pca_probe_bf16_rounding(out) == 0
    assert out[0] == 0, "differs on %d floats, first 0x%08x" % (out[0], out[1])
