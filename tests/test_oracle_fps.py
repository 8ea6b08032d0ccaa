"""Pins of the oracle's `fps` (a play-through of the reference's block of 256
threads, csrc/cuda/fps_cuda.cu:10-66) and of the Python entry point's host
logic.

What pins it: the reference's fixture (test/test_fps.py:16-63), float64
brute-force farthest point sampling on data without ties, the reference's own
compiled CPU operator (csrc/cpu/fps_cpu.cpp, oracle/_ref) on such data, numpy
float16 arithmetic for the fp16 operation order, and a closed form of the tie
rule written independently of the play-through: largest clipped running
minimum, then smallest (row - start) % 256, then smallest row.
"""
import numpy as np
import pytest
import torch
from torch import Tensor

import pytorch_cluster_amd as pca

X_FIX = [[-1, -1], [-1, +1], [+1, +1], [+1, -1],
         [-2, -2], [-2, +2], [+2, +2], [+2, -2]]


def closed_form_fps(x, ptr, counts, dist_fn, limit=5e4, lowest_row=False):
    """Per example: start at its first row; the running minima start at
    `limit`; next = arg max by (value, -(rel % 256), -rel) -- or, with
    `lowest_row`, the rule the reference does NOT follow: (value, -rel)."""
    out = []
    for b in range(len(ptr) - 1):
        s, e = ptr[b], ptr[b + 1]
        if counts[b] == 0:
            continue
        pts = x[s:e]
        rel = np.arange(e - s)
        mind = np.full(e - s, limit, dtype=np.float64)
        cur = 0
        out.append(s + cur)
        for _ in range(counts[b] - 1):
            with np.errstate(over="ignore"):
                mind = np.minimum(mind, dist_fn(pts, pts[cur]))
            cand = rel[mind == mind.max()]
            slot = cand % 256
            cur = cand.min() if lowest_row else cand[slot == slot.min()].min()
            out.append(s + cur)
    return np.array(out, dtype=np.int64)


def dist_f32_fma(pts, p):
    d = np.zeros(len(pts), dtype=np.float32)
    for c in range(pts.shape[1]):
        diff = (p[c] - pts[:, c]).astype(np.float32)
        d = (diff.astype(np.float64) ** 2 + d.astype(np.float64)).astype(
            np.float32)
    return d.astype(np.float64)


def dist_f16(pts, p):
    d = np.zeros(len(pts), dtype=np.float16)
    for c in range(pts.shape[1]):
        diff = p[c] - pts[:, c]
        d = d + diff * diff
    return d.astype(np.float64)


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.float16])
def test_reference_fixture(oracle, dtype):
    x = np.array(X_FIX, dtype=dtype)
    batch = [0, 0, 0, 0, 1, 1, 1, 1]
    assert oracle.fps(x, batch, random_start=False).tolist() == [0, 2, 4, 6]
    assert oracle.fps(x, batch, ratio=0.5,
                      random_start=False).tolist() == [0, 2, 4, 6]
    assert oracle.fps(x, ptr=[0, 4, 8], ratio=0.5,
                      random_start=False).tolist() == [0, 2, 4, 6]
    assert oracle.fps(x, batch, ratio=np.array([0.5, 0.5]),
                      random_start=False).tolist() == [0, 2, 4, 6]
    assert sorted(oracle.fps(x, random_start=False).tolist()) == [0, 5, 6, 7]


@pytest.mark.parametrize("d", [1, 2, 3, 5, 40])
def test_matches_float64_brute_force(oracle, d):
    rng = np.random.default_rng(d)
    x = rng.standard_normal((2500, d))
    ptr = np.array([0, 700, 700, 2500])
    got = oracle.fps_op(x, ptr, 0.2)

    def exact(pts, p):
        return ((pts - p) ** 2).sum(1)
    counts = np.diff(oracle.fps_out_ptr(ptr, 0.2, np.float64))
    want = closed_form_fps(x, ptr, counts, exact)
    assert (got == want).all()
    got32 = oracle.fps_op(x.astype(np.float32), ptr, 0.2)
    assert (got32 == want).mean() > 0.99  # float32 may flip a near-tie


def test_matches_reference_cpu_operator(ref):
    rng = np.random.default_rng(3)
    x = rng.standard_normal((6000, 3)).astype(np.float32)
    ptr = np.array([0, 1000, 3500, 6000])  # (it fails on an empty example)
    got = ref.fps_op(x, ptr, 0.25, fma_mode=0)
    want = ref.ref_fps(x, ptr, 0.25)
    assert got.shape == want.shape
    # (the CPU operator sums the squares in another order: a near-tie may
    # flip, after which the two sequences are different samplings)
    first_diff = np.flatnonzero(got != want)
    assert first_diff.size == 0 or first_diff[0] > 200


def test_sample_counts_follow_the_ratio_type(oracle):
    # ceil(deg * ratio) in the ratio's element type
    # (csrc/cuda/fps_cuda.cu:80-83), checked against torch's own arithmetic
    ptr = np.array([0, 10, 13, 3013, 3020])
    deg = torch.from_numpy(np.diff(ptr))
    for np_t, th_t in ((np.float32, torch.float32), (np.float64, torch.float64),
                       (np.float16, torch.float16)):
        for ratio in (0.3, 0.5, 0.001, 1.0, [0.5, 1.0, 0.001, 0.3]):
            r = torch.tensor(ratio, dtype=th_t)
            want = (deg.to(th_t) * r).ceil().to(torch.long).cumsum(0)
            got = oracle.fps_out_ptr(ptr, ratio, np_t)
            assert got[0] == 0 and got[1:].tolist() == want.tolist()
    # the element type matters: 3000 * 0.3 is 900.00006 in float32
    assert oracle.fps_out_ptr(ptr, 0.3, np.float32)[3] == 905
    assert oracle.fps_out_ptr(ptr, 0.3, np.float64)[3] == 904


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_tie_rule_and_clipping(oracle, dtype):
    """Integer grids (exact ties), examples longer than one pass of the 256
    threads, and coordinates so far apart that the running minima stay at
    the 5e4 they start from."""
    rng = np.random.default_rng(17)
    ptr = np.array([0, 900, 1500, 2300])
    x = rng.integers(0, 5, (2300, 3)).astype(dtype)
    x[1500:] *= 60  # squared distances of 3600 .. 1.7e5: many clip at 5e4
    counts = [40, 30, 50]
    out_ptr = np.concatenate([[0], np.cumsum(counts)])
    ratio = np.array(counts) / np.diff(ptr)
    got = oracle.fps_op(x, ptr, ratio.astype(np.float64)
                        if dtype != np.float16 else ratio)
    if len(got) != out_ptr[-1]:
        pytest.skip("ratio rounding changed the sample counts")
    fn = dist_f16 if dtype == np.float16 else dist_f32_fma
    limit = float(np.float16(5e4)) if dtype == np.float16 else 5e4
    want = closed_form_fps(x, ptr, counts, fn, limit)
    assert (got == want).all()
    # the rule is not "lowest row among the farthest": the test sees that
    lowest = closed_form_fps(x, ptr, counts, fn, limit, lowest_row=True)
    assert (lowest != want).any()


def test_fp16_operation_order(oracle):
    rng = np.random.default_rng(2)
    x = (rng.standard_normal((1800, 4)) * 3).astype(np.float16)
    ptr = np.array([0, 800, 1800])
    got = oracle.fps_op(x, ptr, np.float16(0.1))
    counts = np.diff(oracle.fps_out_ptr(ptr, 0.1, np.float16))
    want = closed_form_fps(x, ptr, counts, dist_f16, float(np.float16(5e4)))
    assert (got == want).all()


def test_start_offsets(oracle):
    rng = np.random.default_rng(4)
    x = rng.standard_normal((600, 3)).astype(np.float32)
    ptr = np.array([0, 200, 600])
    got = oracle.fps_op(x, ptr, 0.1, start=[7, 130])
    assert got[0] == 7 and got[20] == 200 + 130
    assert len(set(got.tolist())) == len(got)


# ---- host logic of the Python entry point, operator replaced by the oracle --

@pytest.fixture
def oracle_fps_op(monkeypatch, oracle):
    calls = []

    def fake(src, ptr, ratio, random_start):
        assert not random_start
        calls.append((ptr.tolist(), ratio.dtype, ratio.tolist()))
        return torch.from_numpy(oracle.fps_op(src.numpy(), ptr.numpy(),
                                              ratio.numpy()))
    monkeypatch.setattr(torch.ops.torch_cluster, "fps", fake)
    return calls


def test_wrapper_fixture(oracle_fps_op):
    # test/test_fps.py:16-63
    x = torch.tensor(X_FIX, dtype=torch.float)
    batch = torch.tensor([0, 0, 0, 0, 1, 1, 1, 1])
    ptr_list = [0, 4, 8]
    ptr = torch.tensor(ptr_list)
    assert pca.fps(x, batch, random_start=False).tolist() == [0, 2, 4, 6]
    assert oracle_fps_op[-1] == ([0, 4, 8], torch.float32, 0.5)
    assert pca.fps(x, batch, ratio=0.5,
                   random_start=False).tolist() == [0, 2, 4, 6]
    assert pca.fps(x, batch, ratio=torch.tensor(0.5),
                   random_start=False).tolist() == [0, 2, 4, 6]
    assert pca.fps(x, ptr=ptr_list, ratio=0.5,
                   random_start=False).tolist() == [0, 2, 4, 6]
    assert pca.fps(x, ptr=ptr, ratio=0.5,
                   random_start=False).tolist() == [0, 2, 4, 6]
    assert pca.fps(x, batch, ratio=torch.tensor([0.5, 0.5]),
                   random_start=False).tolist() == [0, 2, 4, 6]
    assert sorted(pca.fps(x, random_start=False).tolist()) == [0, 5, 6, 7]
    assert sorted(pca.fps(x, ratio=torch.tensor([0.5]),
                          random_start=False).tolist()) == [0, 5, 6, 7]
    assert pca.fps(x, batch, batch_size=2,
                   random_start=False).tolist() == [0, 2, 4, 6]


def test_entry_point_is_scriptable_and_takes_cpu_tensors():
    @torch.jit.script
    def fps2(x: Tensor, ratio: Tensor) -> Tensor:
        return pca.fps(x, None, ratio, False)

    x = torch.rand(16, 3)
    assert torch.equal(fps2(x, torch.tensor([0.5])),
                       pca.fps(x, random_start=False))
    assert pca.fps(x, random_start=False).numel() == 8
    schema = str(torch.ops.torch_cluster.fps.default._schema)
    assert "Tensor ratio, bool random_start" in schema
