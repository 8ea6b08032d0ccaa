"""Seeded random cases across the operators, point kinds, segment layouts and
search strategies, each against the oracle: a net under the targeted parity
tests (shapes and combinations nobody thought of), small enough to run in a
few seconds."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from pytorch_cluster_amd import capi  # noqa: E402
from gpu_common import dev, oracle_knn_edges, ragged_ptrs  # noqa: E402


def _points(rng, n, d, kind):
    if kind == 0:
        return rng.random((n, d)).astype(np.float32)
    if kind == 1:  # a small grid: exact ties everywhere
        return rng.integers(0, 6, (n, d)).astype(np.float32)
    if kind == 2:  # very small, ordinary or very large coordinates
        scale = rng.choice([1e-3, 1.0, 1e3])
        return (rng.standard_normal((n, d)) * scale).astype(np.float32)
    centres = rng.random((8, d))
    return (centres[rng.integers(0, 8, n)]
            + 0.01 * rng.standard_normal((n, d))).astype(np.float32)


@pytest.mark.parametrize("seed", [11, 12, 13, 14])
def test_random_cases_against_the_oracle(oracle, seed):
    rng = np.random.default_rng(seed)
    for case in range(120):
        op = rng.choice(["knn", "knn", "radius", "nearest"])
        d = int(rng.choice([1, 2, 3, 3, 3, 4, 8, 12, 33, 64, 130]))
        n = int(rng.integers(1, 6000))
        m = int(rng.integers(1, 3000))
        segments = int(rng.choice([1, 1, 3, 9]))
        kind = int(rng.integers(0, 4))
        x = _points(rng, n, d, kind)
        y = (x[:m].copy() if m <= n and rng.random() < 0.3
             else _points(rng, m, d, kind))
        ptr_x = ragged_ptrs(rng, n, segments)
        ptr_y = ragged_ptrs(rng, len(y), segments)
        binned = bool(d <= 3 and rng.random() < 0.5)
        px, py = dev(ptr_x, torch.long), dev(ptr_y, torch.long)
        what = dict(seed=seed, case=case, op=str(op), d=d, n=n, m=len(y),
                    segments=segments, kind=kind, binned=binned)
        if op == "knn":
            k = int(rng.choice([1, 3, 8, 16, 17, 32, 50, 64, 100]))
            k = min(k, 64) if binned else k
            cosine = bool(d > 3 and rng.random() < 0.2)
            what.update(k=k, cosine=cosine)
            got = capi.knn_edges(dev(x), dev(y), px, py, k, cosine, False,
                                 binned=binned)[0]
            torch.cuda.synchronize()
            got = got.cpu().numpy()
            want, _ = oracle_knn_edges(oracle, x, y, ptr_x, ptr_y, k, cosine)
        elif op == "radius":
            r = float(rng.choice([0.05, 0.2, 0.7, 1.5]))
            cap = int(rng.choice([1, 5, 32, 64]))
            ignore = bool(rng.random() < 0.5)
            what.update(r=r, cap=cap, ignore=ignore)
            got = capi.radius_edges(dev(x), dev(y), px, py, r, cap, ignore,
                                    binned=binned)
            torch.cuda.synchronize()
            got = got.cpu().numpy()
            want = oracle.radius_op(x, y, ptr_x, ptr_y, r, cap, 1, ignore)
        else:  # the rows of y look for their nearest row of x
            got = capi.nearest_rows(dev(y), dev(x), py, px, binned=binned)
            torch.cuda.synchronize()
            got = got.cpu().numpy()
            want = oracle.nearest_op(y, x, ptr_y, ptr_x)
        assert got.shape == want.shape and (got == want).all(), what
