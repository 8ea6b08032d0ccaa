"""GPU parity of `fps` (pca_fps through the C ABI, the TorchScript operator
and the Python entry point) against the oracle's play-through of the reference
kernel (csrc/cuda/fps_cuda.cu:10-66).  The sampled rows and their order must
be identical, ties and the 5e4 clipping included."""
import numpy as np
import pytest
import torch
from torch import Tensor

pytestmark = pytest.mark.gpu

import pytorch_cluster_amd as pca  # noqa: E402
from pytorch_cluster_amd import capi  # noqa: E402
from gpu_common import DEV, dev  # noqa: E402

TORCH_DTYPE = {np.float32: torch.float32, np.float64: torch.float64,
               np.float16: torch.float16}


def gpu_fps(oracle, x, ptr, ratio, start=None, max_rows=None):
    """pca_fps through the C ABI with the oracle's output positions."""
    dt = x.dtype.type
    out_ptr = oracle.fps_out_ptr(ptr, ratio, dt)
    if max_rows is None:
        max_rows = int(np.diff(ptr).max())
    out, _ws = capi.fps_launch(dev(x), dev(ptr, torch.long),
                               dev(out_ptr, torch.long), int(out_ptr[-1]),
                               dev(start, torch.long), max_rows)
    torch.cuda.synchronize()
    return out.cpu().numpy()


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.float16])
@pytest.mark.parametrize("d", [1, 2, 3, 4, 5, 33])
def test_random_points(oracle, dtype, d):
    rng = np.random.default_rng(100 * d)
    ptr = np.array([0, 900, 900, 3000, 8000], dtype=np.int64)
    x = rng.standard_normal((8000, d)).astype(dtype)
    ratio = np.array([0.1, 0.5, 0.05, 0.02])
    got = gpu_fps(oracle, x, ptr, ratio)
    want = oracle.fps_op(x, ptr, ratio)
    assert (got == want).all()


@pytest.mark.parametrize("dtype,d", [(np.float32, 3), (np.float32, 2),
                                     (np.float32, 7), (np.float64, 3),
                                     (np.float16, 3)])
def test_ties_and_clipping_follow_the_reference_block(oracle, dtype, d):
    rng = np.random.default_rng(23 + d)
    ptr = np.array([0, 900, 1500, 6000], dtype=np.int64)
    x = rng.integers(0, 5, (6000, d)).astype(dtype)
    x[900:1500] *= 60  # most running minima stay at the 5e4 they start from
    ratio = np.array([0.05, 0.1, 0.01])
    got = gpu_fps(oracle, x, ptr, ratio)
    want = oracle.fps_op(x, ptr, ratio)
    assert (got == want).all()


@pytest.mark.parametrize("rows", [1, 200, 256, 257, 512, 1000, 1024, 2047,
                                  2048, 3000, 4096, 4097, 8192, 8193, 12000,
                                  16384])
@pytest.mark.parametrize("d", [2, 3, 4])
def test_every_register_shape_resolves_ties_like_the_reference(oracle, rows, d):
    """The register kernel's launch shape follows the largest example; points
    on a coarse integer grid make most maxima ties, which go by
    (row - start) % 256 first and the row second."""
    rng = np.random.default_rng(rows + d)
    small = max(1, rows // 3)
    ptr = np.array([0, small, small + rows], dtype=np.int64)
    x = rng.integers(0, 4, (ptr[-1], d)).astype(np.float32)
    ratio = np.array([0.5, min(1.0, 150.0 / rows)])
    start = np.array([small - 1, rows // 2], dtype=np.int64)
    got = gpu_fps(oracle, x, ptr, ratio, start)
    want = oracle.fps_op(x, ptr, ratio, start)
    assert (got == want).all()


def test_register_and_streaming_kernels_agree(oracle):
    """Examples of up to 4,096 / 16,384 rows are sampled from registers,
    larger ones (or an unknown bound) from memory: same samples."""
    rng = np.random.default_rng(5)
    for n_big in (4096, 16384, 16385, 30000):
        ptr = np.array([0, 1000, 1000 + n_big], dtype=np.int64)
        x = rng.standard_normal((ptr[-1], 3)).astype(np.float32)
        ratio = np.array([0.2, 300.0 / n_big])
        want = oracle.fps_op(x, ptr, ratio)
        assert (gpu_fps(oracle, x, ptr, ratio) == want).all()
        assert (gpu_fps(oracle, x, ptr, ratio, max_rows=0) == want).all()


def test_start_offsets_nan_rows_and_oversampling(oracle):
    rng = np.random.default_rng(6)
    x = rng.standard_normal((700, 3)).astype(np.float32)
    ptr = np.array([0, 300, 700], dtype=np.int64)
    got = gpu_fps(oracle, x, ptr, 0.1, start=np.array([17, 250]))
    assert (got == oracle.fps_op(x, ptr, 0.1, start=[17, 250])).all()
    # rows with NaN coordinates keep the value they start from
    x[5] = np.nan
    x[400, 1] = np.nan
    for max_rows in (None, 0):
        got = gpu_fps(oracle, x, ptr, 0.2, max_rows=max_rows)
        assert (got == oracle.fps_op(x, ptr, 0.2)).all()
    # more samples than rows: the arg-max over zeros follows the tie rule
    y = rng.standard_normal((40, 2)).astype(np.float32)
    p = np.array([0, 40], dtype=np.int64)
    for max_rows in (None, 0):
        got = gpu_fps(oracle, y, p, 1.5, max_rows=max_rows)
        assert (got == oracle.fps_op(y, p, 1.5)).all()
    # every value NaN: the reference's index 0
    z = np.full((10, 3), np.nan, dtype=np.float32)
    p = np.array([0, 4, 10], dtype=np.int64)
    for max_rows in (None, 0):
        got = gpu_fps(oracle, z, p, 0.5, max_rows=max_rows)
        assert (got == oracle.fps_op(z, p, 0.5)).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.float16])
def test_entry_point_fixture(dtype):
    # test/test_fps.py:16-63 of the reference
    x = torch.tensor([[-1, -1], [-1, +1], [+1, +1], [+1, -1],
                      [-2, -2], [-2, +2], [+2, +2], [+2, -2]],
                     dtype=dtype, device=DEV)
    batch = torch.tensor([0, 0, 0, 0, 1, 1, 1, 1], device=DEV)
    ptr_list = [0, 4, 8]
    ptr = torch.tensor(ptr_list, device=DEV)
    out = pca.fps(x, batch, random_start=False)
    assert out.dtype == torch.long and out.device == x.device
    assert out.tolist() == [0, 2, 4, 6]
    assert pca.fps(x, batch, ratio=0.5,
                   random_start=False).tolist() == [0, 2, 4, 6]
    ratio = torch.tensor(0.5, device=DEV)
    assert pca.fps(x, batch, ratio=ratio,
                   random_start=False).tolist() == [0, 2, 4, 6]
    assert pca.fps(x, ptr=ptr_list, ratio=0.5,
                   random_start=False).tolist() == [0, 2, 4, 6]
    assert pca.fps(x, ptr=ptr, ratio=0.5,
                   random_start=False).tolist() == [0, 2, 4, 6]
    ratio = torch.tensor([0.5, 0.5], device=DEV)
    assert pca.fps(x, batch, ratio=ratio,
                   random_start=False).tolist() == [0, 2, 4, 6]
    assert sorted(pca.fps(x, random_start=False).tolist()) == [0, 5, 6, 7]
    assert sorted(pca.fps(x, ratio=0.5,
                          random_start=False).tolist()) == [0, 5, 6, 7]
    assert sorted(pca.fps(x, ratio=torch.tensor([0.5], device=DEV),
                          random_start=False).tolist()) == [0, 5, 6, 7]

    @torch.jit.script
    def fps2(x: Tensor, ratio: Tensor) -> Tensor:
        return pca.fps(x, None, ratio, False)

    out = fps2(x, torch.tensor([0.5], device=DEV))
    assert sorted(out.tolist()) == [0, 5, 6, 7]


def test_random_start():
    # test/test_fps.py:66-75 of the reference
    N = 1024
    for _ in range(5):
        pos = torch.randn((2 * N, 3), device=DEV)
        batch = torch.cat([torch.zeros(N, dtype=torch.long, device=DEV),
                           torch.ones(N, dtype=torch.long, device=DEV)])
        idx = pca.fps(pos, batch, ratio=0.5)
        assert idx.numel() == N
        assert idx.min() >= 0 and idx.max() < 2 * N
        assert (idx[:N // 2] < N).all() and (idx[N // 2:] >= N).all()
        assert idx.unique().numel() == N


def test_operator_against_oracle_with_ratio_types(oracle):
    """The sample counts come from ceil(deg * ratio) in the ratio's type."""
    rng = np.random.default_rng(9)
    x = rng.standard_normal((3013, 3)).astype(np.float32)
    ptr = np.array([0, 10, 13, 3013], dtype=np.int64)
    for ratio in (0.3, 0.001):
        got = torch.ops.torch_cluster.fps(
            dev(x), dev(ptr, torch.long),
            torch.tensor(ratio, dtype=torch.float32, device=DEV), False)
        want = oracle.fps_op(x, ptr, ratio)
        assert got.cpu().numpy().tolist() == want.tolist()
    with pytest.raises(RuntimeError, match="BFloat16"):
        pca.fps(dev(x).to(torch.bfloat16), random_start=False)


def test_set_abstraction_sizes(oracle):
    """16 clouds of 4,096 points, a quarter sampled (the step that precedes
    radius / knn in a PointNet++ layer): every cloud against the oracle."""
    g = torch.Generator().manual_seed(0)
    x = torch.rand(16 * 4096, 3, generator=g)
    ptr = torch.arange(17) * 4096
    out = torch.ops.torch_cluster.fps(
        x.to(DEV), ptr.to(DEV), torch.tensor(0.25, device=DEV), False)
    want = oracle.fps_op(x.numpy(), ptr.numpy(), 0.25)
    assert out.cpu().numpy().tolist() == want.tolist()
