"""Feature-space kNN with the fp16 matrix-core filter.  Every test runs with
each of the three searches behind it: the four-wave first stage
(knn_feat_impl.hpp), the eight-wave first stage (knn_feat_wide_impl.hpp, up to
128 components), and the one-kernel search for examples of moderate size
(knn_feat_small_impl.hpp: up to 128 components, k <= 48; other
calls fall through to the stages).  Parity with the CPU checker where the
mechanisms of that path are exercised -- lists that overflow (near-duplicates:
the flagged queries go through the second pass), rows and queries the filter
cannot represent, 129-512 components, every list width (k up to 100), scales
at both ends of fp32.  Bit-exact edges and distances, as everywhere.
"""
import numpy as np
import pytest
import torch

import zlib

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True,
                params=["four_waves", "eight_waves", "one_kernel"])
def first_stage(request, monkeypatch):
    """Which search serves the calls of a test: the four-wave kernel with its
    register lists, (where the shape fits: up to 128 components) the
    eight-wave kernel with candidate buffers, or (up to 128 components,
    k <= 48) the one kernel that needs no second stage.  Left to
    itself the library takes the last one for examples of up to 2,048 rows on
    average (up to 8,192 while its workgroups fit the device at once), else
    the eight-wave stage from 4,096 queries on."""
    if request.param == "one_kernel":
        monkeypatch.setenv("PCA_KNN_FEAT_SMALL", "1")
        monkeypatch.delenv("PCA_KNN_FEAT_WIDE", raising=False)
    else:
        monkeypatch.setenv("PCA_KNN_FEAT_SMALL", "0")
        monkeypatch.setenv("PCA_KNN_FEAT_WIDE",
                           "1" if request.param == "eight_waves" else "0")
    return request.param


def _only_once_beyond_128(first_stage, d):
    if d > 128 and first_stage != "four_waves":
        pytest.skip("more than 128 components: the four-wave kernel either way")


def _one_kernel(first_stage, d, k, cosine=False):
    """Whether the one-kernel search serves such a call: it keeps no
    candidate lists, so nothing is ever handed to a second pass."""
    return first_stage == "one_kernel" and d <= 128 and k <= 48


def _seed(*parts):
    """The same seed in every process (str hashes are salted per run)."""
    return zlib.crc32(repr(parts).encode())


def _run(oracle, x, y, ptr_x, ptr_y, k, cosine=False):
    from gpu_common import gpu_knn, oracle_knn_edges
    got, gd = gpu_knn(x, y, ptr_x, ptr_y, k, cosine=cosine)
    want, wd = oracle_knn_edges(oracle, x, y, ptr_x, ptr_y, k, cosine=cosine)
    assert got.shape == want.shape
    assert (got == want).all()
    assert (gd == wd).all()


def _flagged_queries(x, y, k, cosine=False):
    """Number of queries the filter kernel handed to the second pass (read
    from the per-call block at the start of the path's scratch: the workspace
    begins with the [n] row norms, 256-byte aligned)."""
    from gpu_common import dev
    from pytorch_cluster_amd import capi
    xd, yd = dev(x), dev(y)
    _e, _n, _d, ws = capi.knn_launch(xd, yd, None, None, k, cosine)
    torch.cuda.synchronize()
    off = (4 * x.shape[0] + 255) // 256 * 256
    words = ws[off:off + 16].cpu().view(torch.int32).tolist()
    return words[1], words[2]  # (rows the filter cannot represent, flagged)


@pytest.mark.parametrize("d,k,cosine", [(130, 5, False), (200, 16, False),
                                        (256, 32, False), (256, 32, True),
                                        (129, 48, True), (24, 33, False),
                                        (64, 40, True), (96, 48, False),
                                        (32, 1, False), (48, 8, True)])
def test_parity_wide_rows_and_every_list_width(oracle, first_stage, d, k,
                                                cosine):
    _only_once_beyond_128(first_stage, d)
    rng = np.random.default_rng(d * 11 + k)
    n, m = 3000, 500
    x = rng.standard_normal((n, d)).astype(np.float32)
    y = rng.standard_normal((m, d)).astype(np.float32)
    ptr_x = np.array([0, 70, 70, 1200, 3000])
    ptr_y = np.array([0, 100, 130, 131, 500])
    _run(oracle, x, y, ptr_x, ptr_y, k, cosine)


@pytest.mark.parametrize("d", [20, 128, 200])
@pytest.mark.parametrize("cosine", [False, True])
def test_near_duplicates_go_through_the_second_pass(oracle, first_stage, d,
                                                    cosine):
    _only_once_beyond_128(first_stage, d)
    # 60 copies (equal up to the last bits) of every cluster centre: far more
    # than 16 rows within the filter's rounding margin of the k-th distance,
    # so the lists cannot be shown complete and the queries are searched again
    rng = np.random.default_rng(d)
    centres = rng.standard_normal((40, d)).astype(np.float32)
    x = np.repeat(centres, 60, axis=0)
    x = x * (1.0 + 1e-7 * rng.standard_normal(x.shape)).astype(np.float32)
    x = x[rng.permutation(len(x))].astype(np.float32)
    y = np.concatenate([centres[:25],
                        rng.standard_normal((40, d)).astype(np.float32)])
    odd, flagged = _flagged_queries(x, y, 8, cosine)
    if _one_kernel(first_stage, d, 8, cosine):
        assert odd == 0 and flagged == 0
    else:
        assert odd == 0 and flagged >= 25
    _run(oracle, x, y, None, None, 8, cosine)
    # exact duplicates: ties settled by row number
    x2 = np.repeat(centres, 30, axis=0)
    _run(oracle, x2, y, None, None, 20, cosine)


@pytest.mark.parametrize("d,k,cosine", [(300, 7, False), (512, 3, True),
                                        (128, 65, False), (100, 100, False),
                                        (257, 49, True), (400, 100, False),
                                        (512, 64, True), (20, 80, False),
                                        (9, 100, True), (384, 33, False)])
def test_parity_up_to_512_components_and_100_neighbours(oracle, first_stage,
                                                        d, k, cosine):
    _only_once_beyond_128(first_stage, d)
    rng = np.random.default_rng(d * 13 + k)
    n, m = 2500, 300
    x = rng.standard_normal((n, d)).astype(np.float32)
    y = rng.standard_normal((m, d)).astype(np.float32)
    y[:20] = x[:20]
    ptr_x = np.array([0, 90, 90, 1100, 2500])   # (k > rows of the first segment)
    ptr_y = np.array([0, 60, 80, 81, 300])
    _run(oracle, x, y, ptr_x, ptr_y, k, cosine)
    # the filter kernel served the call: its per-call block was written
    odd, flagged = _flagged_queries(x, y, k, cosine)
    assert odd == 0 and 0 <= flagged <= m


def _unresolved_queries(x, y, k, cosine=False):
    """Flagged queries that the threshold scan could not settle (fourth word
    of the per-call block, see _flagged_queries)."""
    from gpu_common import dev
    from pytorch_cluster_amd import capi
    _e, _n, _d, ws = capi.knn_launch(dev(x), dev(y), None, None, k, cosine)
    torch.cuda.synchronize()
    off = (4 * x.shape[0] + 255) // 256 * 256
    return ws[off:off + 16].cpu().view(torch.int32).tolist()[3]


@pytest.mark.parametrize("d", [40, 160])
def test_flagged_queries_beyond_what_the_threshold_scan_holds(oracle,
                                                              first_stage, d):
    _only_once_beyond_128(first_stage, d)
    rng = np.random.default_rng(d + 5)
    # (a) 400 exact copies of one row: more rows at the k-th distance than a
    # hit list holds, the query goes on to the full second pass
    centres = rng.standard_normal((6, d)).astype(np.float32)
    x = np.concatenate([np.repeat(centres[:1], 400, axis=0),
                        np.repeat(centres[1:], 40, axis=0),
                        rng.standard_normal((500, d)).astype(np.float32)])
    x = x[rng.permutation(len(x))]
    y = np.concatenate([centres, rng.standard_normal((30, d)).astype(np.float32)])
    lists = not _one_kernel(first_stage, d, 8)
    if lists:
        assert _unresolved_queries(x, y, 8) >= 1
    _run(oracle, x, y, None, None, 8)
    _run(oracle, x, y, None, None, 8, cosine=True)
    # (b) more flagged queries than the scan's queue takes (8,192 here)
    centres = rng.standard_normal((30, d)).astype(np.float32)
    x = np.repeat(centres, 40, axis=0)
    x = x * (1.0 + 1e-7 * rng.standard_normal(x.shape)).astype(np.float32)
    x = x.astype(np.float32)
    y = np.repeat(centres, 300, axis=0)
    odd, flagged = _flagged_queries(x, y, 6)
    if lists:
        assert flagged > 8192 and _unresolved_queries(x, y, 6) == flagged - 8192
    else:
        assert flagged == 0
    ptr_x = np.array([0, 600, 1200])
    ptr_y = np.array([0, 4200, 9000])
    _run(oracle, x, y, ptr_x, ptr_y, 6)


def test_rows_and_queries_the_filter_cannot_represent(oracle, first_stage):
    rng = np.random.default_rng(3)
    d = 40
    # (the one-kernel search hands nothing on: lanes the filter cannot serve
    # evaluate every row themselves)
    lists = not _one_kernel(first_stage, d, 12)
    x = rng.standard_normal((2000, d)).astype(np.float32)
    y = rng.standard_normal((300, d)).astype(np.float32)
    # NaN and infinite components: never neighbours, the filter skips them
    xa = x.copy()
    xa[5, 3] = np.nan
    xa[700] = np.inf
    xa[900, 0] = -np.inf
    ya = y.copy()
    ya[7, 1] = np.nan      # no neighbours at all
    ya[8] = np.inf
    odd, flagged = _flagged_queries(xa, ya, 12)
    assert odd == 0
    _run(oracle, xa, ya, None, None, 12)
    _run(oracle, xa, ya, None, None, 12, cosine=True)
    # finite rows whose squared norm overflows: everything takes the second
    # pass (such a row can be the duplicate of an equally large query)
    xb = x.copy()
    xb[11] = 3e19
    yb = y.copy()
    yb[4] = 3e19
    odd, flagged = _flagged_queries(xb, yb, 12)
    assert odd == 1 and flagged == (len(yb) if lists else 0)
    _run(oracle, xb, yb, None, None, 12)
    _run(oracle, xb, yb, None, None, 12, cosine=True)
    # a query of that kind alone: only its tile is searched again
    odd, flagged = _flagged_queries(x, yb, 12)
    assert odd == 0 and flagged == (1 if lists else 0)
    _run(oracle, x, yb, None, None, 12)


@pytest.mark.parametrize("case", ["rows", "queries", "both", "one_of_each"])
def test_cosine_norms_that_underflow_to_zero(oracle, case):
    # components below 1e-23: every square underflows, the norm is exactly
    # zero, yet the dot product with an ordinary vector is not -- the
    # reference divides it by that zero and returns the rows with a positive
    # dot product at distance -inf.  Vectors of zeros have no neighbours.
    rng = np.random.default_rng(_seed("lost norms", case))
    d, n, m, k = 40, 2500, 300, 12
    x = rng.standard_normal((n, d)).astype(np.float32)
    y = rng.standard_normal((m, d)).astype(np.float32)
    if case in ("rows", "both"):
        x *= np.float32(1e-25)
    if case in ("queries", "both"):
        y *= np.float32(1e-25)
    if case == "one_of_each":
        x[17] *= np.float32(1e-25)
        y[5] *= np.float32(1e-25)
    x[3] = 0.0
    y[8] = 0.0
    ptr_x = np.array([0, 1200, n])
    ptr_y = np.array([0, 100, m])
    _run(oracle, x, y, ptr_x, ptr_y, k, cosine=True)


@pytest.mark.parametrize("d,k", [(9, 1), (12, 8), (40, 20)])
def test_cosine_norms_in_the_denormal_range_of_their_squares(oracle, d, k):
    # components around 1e-21: squares and products are denormal numbers of a
    # few bits, the reference's distance strays from the cosine by per cents,
    # and only an evaluation in its own arithmetic finds its neighbours (a
    # filter with any margin made for normal numbers does not)
    rng = np.random.default_rng(_seed("denormal squares", d, k))
    n, m = 6000, 500
    centres = rng.standard_normal((60, d))
    x = centres[rng.integers(0, 60, n)] + 0.05 * rng.standard_normal((n, d))
    y = centres[rng.integers(0, 60, m)] + 0.05 * rng.standard_normal((m, d))
    x = (x * 1e-21).astype(np.float32)
    y = (y * 1e-21).astype(np.float32)
    _run(oracle, x, y, None, None, k, cosine=True)
    _run(oracle, x, y, np.array([0, 2500, n]), np.array([0, 200, m]), k,
         cosine=True)


@pytest.mark.parametrize("case", ["tiny", "huge", "mixed", "outlier",
                                  "zeros", "sparse"])
def test_scales_at_both_ends(oracle, case):
    # one power of two scales all rows into the fp16 range: rows far below the
    # largest one lose their bits there, and the lists must notice
    rng = np.random.default_rng(_seed("scales", case))
    d, n, m, k = 72, 4000, 400, 16
    x = rng.standard_normal((n, d))
    y = rng.standard_normal((m, d))
    if case == "tiny":
        x, y = 1e-30 * x, 1e-30 * y
    elif case == "huge":
        x, y = 1e15 * x, 1e15 * y
        y[:40] = x[:40]
    elif case == "mixed":
        x = x * 10.0 ** rng.integers(-5, 6, (n, 1))
        y = y * 10.0 ** rng.integers(-5, 6, (m, 1))
    elif case == "outlier":
        x[17] *= 1e9   # one row sets the scale, all others are tiny beside it
    elif case == "zeros":
        x[:] = 0.0
        x[100:110] = 1.0
        y[:5] = 0.0
    else:
        x = x * (rng.random((n, d)) < 0.05)
        y = y * (rng.random((m, d)) < 0.05)
    x = x.astype(np.float32)
    y = y.astype(np.float32)
    ptr_x = np.array([0, 1500, 4000])
    ptr_y = np.array([0, 150, 400])
    _run(oracle, x, y, ptr_x, ptr_y, k)
    if case not in ("zeros",):
        _run(oracle, x, y, ptr_x, ptr_y, k, cosine=True)


@pytest.mark.parametrize("case", ["one_row", "eight_rows", "nine_rows",
                                  "queries_too", "only_four_times",
                                  "neighbour_of_a_query", "small_segment"])
def test_rows_far_larger_than_the_rest(oracle, case):
    # up to 8 rows of x (and 8 of y) at least four times larger than all
    # others do not set the fp16 scale: they stay out of the filter, every
    # query evaluates them exactly, and the other rows keep their bits --
    # same edges, and (almost) no query is handed to the second pass
    rng = np.random.default_rng(_seed("outliers", case))
    d, n, m, k = 72, 6000, 500, 16
    x = rng.standard_normal((n, d)).astype(np.float32)
    y = rng.standard_normal((m, d)).astype(np.float32)
    ptr_x = np.array([0, 2500, 6000])
    ptr_y = np.array([0, 200, 500])
    few_flagged = True
    if case == "one_row":
        x[17] *= 1e6
    elif case == "eight_rows":
        x[rng.choice(n, 8, replace=False)] *= 3e4
    elif case == "nine_rows":
        # one too many: the scale is made for them, as before
        x[rng.choice(n, 9, replace=False)] *= 3e4
        few_flagged = False
    elif case == "queries_too":
        x[4000] *= 1e5
        y[[3, 250, 499]] *= 1e7
    elif case == "only_four_times":
        x[100] *= 40.0   # (largest components 4 x 40 / 4: three binades up)
    elif case == "neighbour_of_a_query":
        x[[10, 3000]] *= 1e5
        y[0] = x[10]            # the large row is this query's nearest row
        y[1] = x[10] * (1 + 1e-3)
        y[300] = x[3000]
    else:
        # a segment of 40 rows: the large row is one of many in the call
        ptr_x = np.array([0, 40, 6000])
        x[5] *= 1e6
    odd, flagged = _flagged_queries(x, y, k)
    assert odd == 0
    if few_flagged:
        assert flagged <= 8, flagged
    _run(oracle, x, y, ptr_x, ptr_y, k)
    _run(oracle, x, y, ptr_x, ptr_y, k, cosine=True)
    _run(oracle, x, y, None, None, 40)


@pytest.mark.parametrize("d", [9, 12, 17, 32, 63, 64, 65, 100, 127, 128])
def test_one_kernel_search_shapes(oracle, first_stage, d):
    if first_stage != "one_kernel":
        pytest.skip("the one-kernel search only")
    # examples of 0, 1, 31, 32, 33 rows, of more rows than the bound samples
    # (64 steps of 32), of exactly a number of steps, with no queries, with
    # fewer rows than k; queries that do not fill a workgroup; every list
    # width; components that are and are not a multiple of four
    rng = np.random.default_rng(_seed("one_kernel", d))
    sizes_x = [0, 1, 31, 32, 33, 2500, 512, 40, 1024, 7]
    sizes_y = [3, 5, 130, 0, 129, 300, 128, 1, 257, 20]
    ptr_x = np.concatenate([[0], np.cumsum(sizes_x)])
    ptr_y = np.concatenate([[0], np.cumsum(sizes_y)])
    x = rng.standard_normal((ptr_x[-1], d)).astype(np.float32)
    y = rng.standard_normal((ptr_y[-1], d)).astype(np.float32)
    y[:200] = x[rng.integers(0, len(x), 200)]      # distance zero, ties
    x[3000:3040] = x[2990]                         # equal rows: row numbers
    for k in (1, 7, 8, 9, 16, 20, 24, 25, 32, 33, 41, 48):
        _run(oracle, x, y, ptr_x, ptr_y, k)
    # rows far larger than the rest, one in an example too short for a bound
    # (every row of it is evaluated; the large one must not be listed twice)
    x[[1000, 3120]] *= 1e5
    for k in (5, 20, 32, 47):
        _run(oracle, x, y, ptr_x, ptr_y, k)


def test_one_kernel_search_is_the_default_for_small_examples(oracle,
                                                             first_stage,
                                                             monkeypatch):
    if first_stage != "one_kernel":
        pytest.skip("once is enough")
    monkeypatch.delenv("PCA_KNN_FEAT_SMALL", raising=False)
    # 24 examples of 700 rows searched in themselves, as a dynamic graph
    # layer does; no query is handed on, the per-call block says so
    rng = np.random.default_rng(77)
    x = rng.standard_normal((24 * 700, 64)).astype(np.float32)
    ptr = np.arange(25) * 700
    _run(oracle, x, x, ptr, ptr, 21)
    odd, flagged = _flagged_queries(x, x, 21)
    assert odd == 0 and flagged == 0
    # the same tensor on both sides (a graph of the cloud in itself): the
    # preparation goes over the rows once
    from gpu_common import dev
    from pytorch_cluster_amd import capi
    xd, pd = dev(x), dev(ptr)
    for t in (xd, xd.half(), xd[:, :40].contiguous().bfloat16()):
        one, _ = capi.knn_edges(t, t, pd, pd, 21)
        two, _ = capi.knn_edges(t, t.clone(), pd, pd, 21)
        assert one.shape == two.shape == (2, 24 * 700 * 21)
        assert bool((one == two).all())


def test_many_slices_share_their_bounds(oracle, monkeypatch):
    rng = np.random.default_rng(9)
    x = rng.standard_normal((20000, 64)).astype(np.float32)
    y = rng.standard_normal((300, 64)).astype(np.float32)
    for slices in ("1", "3", "16"):
        monkeypatch.setenv("PCA_KNN_SLICES", slices)
        _run(oracle, x, y, None, None, 24)
        _run(oracle, x, y, None, None, 24, cosine=True)


def test_pieces_of_the_eight_wave_stage(oracle, monkeypatch):
    # the eight-wave stage cuts the (tile of 512 queries, 64 rows) pairs of a
    # call into as many stretches as it has workgroups: one workgroup that
    # walks through every tile, pieces of a few rows, several pieces per tile,
    # and the buffers at their smallest (a checkpoint tidies them more often)
    monkeypatch.setenv("PCA_KNN_FEAT_WIDE", "1")
    monkeypatch.setenv("PCA_KNN_FEAT_SMALL", "0")
    rng = np.random.default_rng(21)
    x = rng.standard_normal((9000, 48)).astype(np.float32)
    y = rng.standard_normal((1500, 48)).astype(np.float32)
    ptr_x = np.array([0, 3000, 3000, 3100, 9000])
    ptr_y = np.array([0, 700, 800, 900, 1500])
    for grid, cap in (("1", "192"), ("7", "8192"), ("64", "192"),
                      ("200", "256")):
        monkeypatch.setenv("PCA_FEAT_WIDE_GRID", grid)
        monkeypatch.setenv("PCA_FEAT_WIDE_CAP", cap)
        _run(oracle, x, y, ptr_x, ptr_y, 20)
        _run(oracle, x, y, None, None, 70, cosine=True)
    # rows that arrive ever closer to the queries: every row passes the cut of
    # its time, the buffers fill up between the scheduled checkpoints
    monkeypatch.setenv("PCA_FEAT_WIDE_GRID", "2")
    monkeypatch.setenv("PCA_FEAT_WIDE_CAP", "192")
    centre = rng.standard_normal(48)
    radius = np.linspace(30.0, 0.5, 6000)[:, None]
    xs = (centre + radius * rng.standard_normal((6000, 48))
          / np.sqrt(48)).astype(np.float32)
    ys = (centre + 0.01 * rng.standard_normal((600, 48))).astype(np.float32)
    _run(oracle, xs, ys, None, None, 16)


def test_queries_enough_for_the_eight_wave_stage_by_default(oracle,
                                                            monkeypatch):
    # from 4,096 queries on the library takes the eight-wave stage by itself
    monkeypatch.delenv("PCA_KNN_FEAT_WIDE", raising=False)
    monkeypatch.setenv("PCA_KNN_FEAT_SMALL", "0")
    rng = np.random.default_rng(22)
    x = rng.standard_normal((12000, 96)).astype(np.float32)
    y = rng.standard_normal((5000, 96)).astype(np.float32)
    _run(oracle, x, y, np.array([0, 5000, 12000]), np.array([0, 2100, 5000]),
         20)


def test_feature_space_knn_256_full_size_properties(oracle, first_stage):
    _only_once_beyond_128(first_stage, 256)
    # 50,000 rows of 256 components onto themselves, k = 32: every 400th query
    # exactly, all of them by the properties the result must have
    from gpu_common import dev
    from pytorch_cluster_amd import capi
    g = torch.Generator().manual_seed(0)
    x = torch.randn(50000, 256, generator=g)
    e, dist = capi.knn_edges(dev(x.numpy()), dev(x.numpy()), None, None, 32,
                             want_dist=True)
    torch.cuda.synchronize()
    e, dist = e.cpu().numpy(), dist.cpu().numpy()
    assert e.shape == (2, 50000 * 32)
    rows = e[0].reshape(50000, 32)
    cols = e[1].reshape(50000, 32)
    dd = dist.reshape(50000, 32)
    assert (rows == np.arange(50000)[:, None]).all()
    assert (cols[:, 0] == np.arange(50000)).all() and (dd[:, 0] == 0).all()
    assert (np.diff(dd, axis=1) >= 0).all()
    sample = np.arange(0, 50000, 400)
    xs = x.numpy()
    _, col, d_ref = oracle.knn_dense(xs, xs[sample], None, None, 32)
    assert (cols[sample] == col).all()
    assert (dd[sample] == d_ref).all()
