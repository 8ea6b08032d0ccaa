#!/usr/bin/env python3
"""Benchmark of the kNN hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one `knn(x, y, k=16, batch_x, batch_y)` call over the ragged
LiDAR-like workload (8 scans, ~1.03 M points, every 4th point a query), inputs
resident in HBM.  Prints ONE JSON line with whole-job queries/s, the roofline
of the dominant kernel (brute-force distance tiles: algorithmic fp32 flops
against the fp32 peak, which is the same figure for the vector and the matrix
units) measured with HIP events around that kernel inside the timed region,
and the reference's CPU path timed on this host beside it.
"""
import argparse
import ctypes
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

K = 16
PEAK_FP32_TFLOPS = 157.3  # MI355X fp32, vector (packed) = matrix
FLOP_PER_PAIR = 9         # 3-D: 3 subtractions + 3 multiply-adds


class HipEvents:
    """hipEvent_t pairs through the HIP runtime PyTorch has loaded."""

    def __init__(self, torch):
        lib_dir = os.path.join(os.path.dirname(torch.__file__), "lib")
        self.hip = ctypes.CDLL(os.path.join(lib_dir, "libamdhip64.so"))

    def create(self):
        ev = ctypes.c_void_p()
        rc = self.hip.hipEventCreate(ctypes.byref(ev))
        assert rc == 0, "hipEventCreate failed: %d" % rc
        return ev

    def elapsed_ms(self, start, stop):
        ms = ctypes.c_float()
        rc = self.hip.hipEventElapsedTime(ctypes.byref(ms), start, stop)
        assert rc == 0, "hipEventElapsedTime failed: %d" % rc
        return ms.value

    def destroy(self, ev):
        self.hip.hipEventDestroy(ev)


def cpu_build_baseline(pca, data):
    """This package's own CPU path (the operators called with CPU tensors:
    k-d trees searched on all host threads) on the full workload."""
    import torch
    x, y = data["x"], data["y"]
    bx, by = data["batch_x"], data["batch_y"]
    times = []
    for _ in range(4):
        t0 = time.perf_counter()
        e = pca.knn(x, y, K, bx, by, batch_size=data["batch_size"])
        times.append(time.perf_counter() - t0)
    assert e.shape[1] == y.shape[0] * K
    return {"value": y.shape[0] / statistics.median(times[1:]),
            "unit": "queries/s", "cores": torch.get_num_threads(),
            "kind": "build",
            "sample": "full workload (%d queries over %d points), median of "
                      "3 calls after one untimed; pytorch_cluster_amd.knn on "
                      "CPU tensors (k-d tree per scan, queries spread over "
                      "the host threads)" % (y.shape[0], x.shape[0])}


def cpu_baseline(data, ptr_x, ptr_y):
    """The reference's CPU operator (nanoflann KD-tree; single-threaded by
    construction, `num_workers` is never read) on the same inputs, or the
    brute-force port on a sample of the queries when it is not available."""
    import numpy as np
    import oracle

    x = data["x"].numpy()
    y = data["y"].numpy()
    px, py = ptr_x.numpy(), ptr_y.numpy()
    m = y.shape[0]
    if oracle.have_ref():
        times = []
        for _ in range(3):
            t0 = time.perf_counter()
            e = oracle.ref_knn(x, y, px, py, K)
            times.append(time.perf_counter() - t0)
        assert e.shape[1] == m * K
        return {"value": m / statistics.median(times), "unit": "queries/s",
                "cores": 1, "kind": "reference",
                "sample": "full workload (%d queries over %d points), median "
                          "of 3 runs; nanoflann KD-tree operator of the "
                          "reference, single-threaded by construction"
                          % (m, x.shape[0])}
    stride = 64
    sample = np.arange(0, m, stride)
    ys = np.ascontiguousarray(y[sample])
    pys = np.searchsorted(sample, py)
    t0 = time.perf_counter()
    oracle.knn_op(x, ys, px, pys, K)
    dt = time.perf_counter() - t0
    return {"value": len(sample) / dt, "unit": "queries/s",
            "cores": os.cpu_count(), "kind": "port",
            "sample": "every %dth query (%d queries), brute-force C port with "
                      "OpenMP" % (stride, len(sample))}


PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 / fp16 matrix peak
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E

# Pairs the reference's radius kernel has to look at on configs[2] (seed 0):
# for every query the scan position of its 32nd hit, or the segment length
# (csrc/cuda/radius_cuda.cu:26-41).  tests/test_bench_constants.py recomputes
# it with the CPU checker.
C3_REQUIRED_PAIRS = 255153263


def _median_ms(torch, fn, reps):
    fn()
    torch.cuda.synchronize()
    times = []
    out = None
    for _ in range(reps):
        t0 = time.perf_counter()
        out = fn()
        torch.cuda.synchronize()
        times.append((time.perf_counter() - t0) * 1e3)
    return statistics.median(times), out


def _search_ms(torch, capi, events, fn, reps=3):
    """Average duration of the search kernel of `fn` (HIP events recorded by
    the library immediately around that kernel, on its launch stream)."""
    total = 0.0
    for _ in range(reps):
        start, stop = events.create(), events.create()
        capi.pca_time_next_search(start, stop)
        fn()
        torch.cuda.synchronize()
        total += events.elapsed_ms(start, stop)
        events.destroy(start)
        events.destroy(stop)
    return total / reps


def _roofline(kernel, kernel_ms, flop, peak_tflops, bound, detail):
    achieved = flop / kernel_ms / 1e9
    return {"bound": bound, "bound_detail": detail, "kernel": kernel,
            "kernel_ms": kernel_ms, "flop_per_launch": flop,
            "achieved": achieved, "peak": peak_tflops, "unit": "TFLOP/s",
            "frac": achieved / peak_tflops}


def _hbm_roofline(kernel, kernel_ms, nbytes, detail):
    achieved = nbytes / kernel_ms / 1e6
    return {"bound": "hbm", "bound_detail": detail, "kernel": kernel,
            "kernel_ms": kernel_ms, "bytes_per_launch": nbytes,
            "achieved": achieved, "peak": PEAK_HBM_GBS, "unit": "GB/s",
            "frac": achieved / PEAK_HBM_GBS}


def _search_bytes(n, m, d, slots, elem=4):
    """Bytes a neighbour search has to move: every point and query once, and
    the [2, m * slots] int64 edge list."""
    return (n + m) * d * elem + m * slots * 16


def _feat_shape(d, k):
    """(16-component blocks per row incl. the one that carries |x|^2, list
    width) of the feature-space kernel that serves (d, k)."""
    blocks = next(b for b in (3, 5, 9, 17, 33) if 16 * (b - 1) >= d)
    width = next(w for w in (24, 32, 48, 64, 80, 116) if w >= k + 16)
    return blocks, width


class Cases:
    """The benchmark configurations beside the headline one, by name; each
    returns its report (whole-call time, rate, roofline of its search
    kernel)."""

    def __init__(self, torch, pca, testing, dev):
        from pytorch_cluster_amd._native import capi
        self.torch, self.pca, self.testing, self.dev = torch, pca, testing, dev
        self.capi = capi
        self.events = HipEvents(torch)

    def names(self):
        return ["c1", "c2", "c3", "c4", "c4cos", "d256", "clouds64",
                "nearest_points", "nearest_codes", "fps", "strategies"]

    def run(self, name, reps=None):
        return getattr(self, "case_" + name)(reps)

    # configs[0]: the plumbing case, on the GPU here (CPU tensors take the
    # package's CPU path: see cpu_build_baseline)
    def case_c1(self, reps):
        t, pca = self.torch, self.pca
        x = self.testing.uniform_cloud(0)["x"].to(self.dev)
        pca.set_search_strategy("scan")
        fn = lambda: pca.knn_graph(x, 16)  # noqa: E731
        ms, out = _median_ms(t, fn, reps or 10)
        kms = _search_ms(t, self.capi, self.events, fn)
        pairs = x.shape[0] * x.shape[0]
        return {"configs[0] knn_graph 1024 k=16": {
            "ms": ms, "queries_per_s": x.shape[0] / ms * 1e3,
            "edges": int(out.shape[1]),
            "roofline": _roofline(
                "knn_lowd_mc_kernel<3,24>", kms, 9 * pairs, PEAK_FP32_TFLOPS,
                "mfma", "algorithmic 3*D flop per pair against the fp32 "
                "peak; 8 workgroups: a launch-latency case")}}

    def case_c2(self, reps):
        t, pca = self.torch, self.pca
        c2 = self.testing.uniform_batched(0)
        x, b = c2["x"].to(self.dev), c2["batch"].to(self.dev)
        pca.set_search_strategy("scan")
        fn = lambda: pca.knn_graph(x, 20, b, batch_size=16)  # noqa: E731
        ms, out = _median_ms(t, fn, reps or 10)
        kms = _search_ms(t, self.capi, self.events, fn)
        pairs = 16 * 4096 * 4096
        return {"configs[1] knn_graph 16x4096 k=20": {
            "ms": ms, "queries_per_s": x.shape[0] / ms * 1e3,
            "edges": int(out.shape[1]),
            "roofline": _roofline(
                "knn_lowd_mc_kernel<3,24>", kms, 9 * pairs, PEAK_FP32_TFLOPS,
                "mfma", "algorithmic 3*D flop per pair against the fp32 peak "
                "(vector = matrix)")}}

    def case_c3(self, reps):
        t, pca = self.torch, self.pca
        c3 = self.testing.gaussian_mixture_batched(0)
        x, b = c3["x"].to(self.dev), c3["batch"].to(self.dev)
        pca.set_search_strategy("scan")
        fn = lambda: pca.radius_graph(  # noqa: E731
            x, 0.05, b, max_num_neighbors=32, batch_size=8)
        ms, out = _median_ms(t, fn, reps or 10)
        kms = _search_ms(t, self.capi, self.events, fn)
        full = 8 * 16384 * 16384
        detail = ("algorithmic 3*D flop per pair against the fp32 peak; the "
                  "kernel stops a query at its 32nd hit")
        return {"configs[2] radius_graph 8x16384 r=0.05 max 32": {
            "ms": ms, "edges_per_s": out.shape[1] / ms * 1e3,
            "edges": int(out.shape[1]),
            "roofline": _roofline(
                "radius_mc_kernel<3>", kms, 9 * C3_REQUIRED_PAIRS,
                PEAK_FP32_TFLOPS, "mfma", detail + "; pairs = those the "
                "reference's scan has to look at (position of the 32nd hit)"),
            "roofline_all_pairs": _roofline(
                "radius_mc_kernel<3>", kms, 9 * full, PEAK_FP32_TFLOPS,
                "mfma", detail + "; pairs = all pairs of a segment")}}

    def _feature_case(self, label, n, m, d, k, cosine, reps):
        t, pca = self.torch, self.pca
        c = self.testing.feature_space(0, n, m, d)
        x, y = c["x"].to(self.dev), c["y"].to(self.dev)
        fn = lambda: pca.knn(x, y, k, cosine=cosine)  # noqa: E731
        ms, out = _median_ms(t, fn, reps or 3)
        kms = _search_ms(t, self.capi, self.events, fn)
        flop = 2 * d * n * m
        if d > 512:
            kernel = "knn_generic_kernel"
            issued = None
        else:
            blocks, width = _feat_shape(d, k)
            # up to 128 components and from 4,096 queries on: the eight-wave
            # first stage (queries in tiles of 512, lists of the k smallest
            # values); else the four-wave one (tiles of 128, lists of k + 16)
            wide = d <= 128 and m >= 4096
            if wide:
                kernel = "knn_feat_wide_kernel<%d,%d,%s>" % (
                    blocks, next(w for w in (16, 32, 64, 100) if w >= k),
                    "true" if cosine else "false")
            else:
                kernel = "knn_feat_kernel<%d,%d,%s>" % (
                    blocks, width, "true" if cosine else "false")
            # one v_mfma_f32_32x32x16_f16 (32,768 flop) per block and 32 x 32
            # pairs; rows in tiles of 64 (32 from 144 components on)
            tile = 64 if blocks <= 9 else 32
            qtile = 512 if wide else 128
            issued = (-(-n // tile) * tile) * (-(-m // qtile) * qtile) \
                // 1024 * blocks * 32768
        roof = _roofline(
            kernel, kms, flop, PEAK_BF16_TFLOPS, "mfma",
            "algorithmic 2*D flop per pair against the dense fp16 / bf16 "
            "matrix peak; the kernel forms one fp16 product per pair and "
            "component on the matrix cores (a proven lower bound of the "
            "distance), keeps the k + 16 rows per query with the smallest "
            "bounds, and a second kernel evaluates those exactly in fp32")
        if issued is not None:
            roof["issued_flop_per_launch"] = issued
            roof["issued_frac"] = issued / kms / 1e9 / PEAK_BF16_TFLOPS
        return {label: {
            "ms": ms, "queries_per_s": m / ms * 1e3,
            "edges": int(out.shape[1]), "roofline": roof}}

    def case_c4(self, reps):
        return self._feature_case(
            "configs[3] knn 200000x128 / 50000x128 k=32 cosine=False",
            200000, 50000, 128, 32, False, reps)

    def case_c4cos(self, reps):
        return self._feature_case(
            "configs[3] knn 200000x128 / 50000x128 k=32 cosine=True",
            200000, 50000, 128, 32, True, reps)

    def case_d256(self, reps):
        report = self._feature_case(
            "knn 50000x256 onto themselves k=32", 50000, 50000, 256, 32,
            False, reps)
        report.update(self._feature_case(
            "knn 50000x256 onto themselves k=64", 50000, 50000, 256, 64,
            False, reps))
        return report

    # the shape of a dynamic-graph layer of a point-cloud network: many small
    # clouds searched in themselves in feature space (one kernel that needs
    # no second stage: examples of moderate length, d <= 128, k <= 48)
    def case_clouds64(self, reps):
        t, pca = self.torch, self.pca
        clouds, points, d, k = 32, 1024, 64, 20
        x = self.testing.feature_space(0, clouds * points, 1, d)["x"].to(
            self.dev)
        b = t.arange(clouds, device=self.dev).repeat_interleave(points)
        fn = lambda: pca.knn_graph(x, k, b, batch_size=clouds)  # noqa: E731
        ms, out = _median_ms(t, fn, reps or 10)
        kms = _search_ms(t, self.capi, self.events, fn)
        blocks = _feat_shape(d, k)[0]
        flop = 2 * d * clouds * points * points
        detail = ("algorithmic 2*D flop per pair against the dense fp16 "
                  "matrix peak; one workgroup per 128 queries goes over its "
                  "cloud (twice for kNN: bound, then search) with one wave "
                  "per SIMD: a latency case, 4 GFLOP per call")
        report = {"knn_graph 32x1024 points x 64 features k=20": {
            "ms": ms, "queries_per_s": x.shape[0] / ms * 1e3,
            "edges": int(out.shape[1]),
            "roofline": _roofline(
                "knn_feat_small_kernel<%d,24>" % blocks, kms, flop,
                PEAK_BF16_TFLOPS, "mfma", detail)}}
        # the same clouds: rows in fp16 (the reference's 16-bit arithmetic
        # behind the same filter), cosine distance, radius search
        variants = (
            ("knn_graph 32x1024 points x 64 features k=20, fp16 rows",
             "knn_feat_small_kernel<%d,24,1>" % blocks,
             lambda h=x.half(): pca.knn_graph(h, k, b, batch_size=clouds)),
            ("knn_graph 32x1024 points x 64 features k=20, cosine",
             "knn_feat_small_kernel<%d,24,3>" % blocks,
             lambda: pca.knn_graph(x, k, b, batch_size=clouds, cosine=True)),
            ("radius_graph 32x1024 points x 64 features r=9 max 32",
             "knn_feat_small_kernel<%d,32,0,true>" % blocks,
             lambda: pca.radius_graph(x, 9.0, b, max_num_neighbors=32,
                                      batch_size=clouds)))
        for label, kernel, call in variants:
            ms, out = _median_ms(t, call, reps or 10)
            kms = _search_ms(t, self.capi, self.events, call)
            report[label] = {
                "ms": ms, "queries_per_s": x.shape[0] / ms * 1e3,
                "edges": int(out.shape[1]),
                "roofline": _roofline(kernel, kms, flop, PEAK_BF16_TFLOPS,
                                      "mfma", detail)}
        return report

    # nearest: every point of the LiDAR-like scans looks for the nearest of
    # its scan's every-8th point (the operator that follows the neighbour
    # searches in the reference's list; 3 * D flop per pair as above)
    def case_nearest_points(self, reps):
        t, pca = self.torch, self.pca
        lidar = self.testing.lidar_scans(0, query_stride=8)
        x, y = lidar["x"].to(self.dev), lidar["y"].to(self.dev)
        bx, by = lidar["batch_x"].to(self.dev), lidar["batch_y"].to(self.dev)
        sizes_x = t.bincount(lidar["batch_x"])
        sizes_y = t.bincount(lidar["batch_y"])
        pairs = int((sizes_x * sizes_y).sum())
        pca.set_search_strategy("scan")
        fn = lambda: pca.nearest(x, y, bx, by)  # noqa: E731
        ms, _ = _median_ms(t, fn, reps or 10)
        kms = _search_ms(t, self.capi, self.events, fn)
        return {"nearest: %d scan points -> their scan's every 8th point (%d)"
                % (x.shape[0], y.shape[0]): {
            "ms": ms, "rows_per_s": x.shape[0] / ms * 1e3,
            "roofline": _roofline(
                "knn_lowd_mc_kernel<3,1,nearest>", kms, 9 * pairs,
                PEAK_FP32_TFLOPS, "mfma",
                "algorithmic 3*D flop per pair against the fp32 peak")}}

    # nearest in feature space: a code-book assignment (1M rows of 64
    # components to 4,096 code vectors, one segment; 2 * D flop per pair)
    def case_nearest_codes(self, reps):
        t, pca = self.torch, self.pca
        g = t.Generator().manual_seed(0)
        codes = t.randn(4096, 64, generator=g)
        feats = (codes[t.randint(0, 4096, (1 << 20,), generator=g)]
                 + 0.5 * t.randn(1 << 20, 64, generator=g)).to(self.dev)
        codes = codes.to(self.dev)
        fn = lambda: pca.nearest(feats, codes)  # noqa: E731
        ms, _ = _median_ms(t, fn, reps or 5)
        kms = _search_ms(t, self.capi, self.events, fn)
        return {"nearest: 1048576 x 64 features -> 4096 code vectors": {
            "ms": ms, "rows_per_s": feats.shape[0] / ms * 1e3,
            "roofline": _roofline(
                "knn_mfma_kernel<5,8,nearest>", kms,
                2 * 64 * feats.shape[0] * 4096, PEAK_BF16_TFLOPS, "mfma",
                "algorithmic 2*D flop per pair against the dense bf16 "
                "matrix peak (this kernel forms three split-bf16 products "
                "per pair and component)")}}

    # fps: the sampling step that precedes radius / knn in a set-abstraction
    # layer; a quarter of every cloud, first row as start
    def case_fps(self, reps):
        t = self.torch
        report = {}
        for clouds, points in ((16, 4096), (8, 16384)):
            pts = self.testing.uniform_batched(0, clouds, points)["x"]
            pts = pts.to(self.dev)
            ptr = (t.arange(clouds + 1) * points).to(self.dev)
            ratio = t.tensor(0.25, device=self.dev)
            ms, out = _median_ms(
                t, lambda: t.ops.torch_cluster.fps(pts, ptr, ratio, False),
                reps or 5)
            # A sample step depends on the one before it, and a cloud is
            # one workgroup's (its running minima stay in that compute
            # unit's registers), so the floor is latency, not bandwidth:
            # per step and row 3 subtractions, 3 multiply-adds, the minimum
            # and two compare/selects for the running maximum = 9 vector
            # instructions, 4 cycles each per wave of 64 on one of the
            # unit's 4 SIMDs at 2.4 GHz; the two reductions across the
            # workgroup come on top.
            step_us = ms * 1e3 / (points // 4)
            floor_us = points / 64.0 * 9 * 4 / 4 / 2400.0
            report["fps %dx%d ratio 0.25" % (clouds, points)] = {
                "ms": ms, "samples": int(out.numel()),
                "us_per_sample_step": step_us,
                "roofline": {
                    "bound": "valu-latency", "unit": "us/step",
                    "floor": floor_us, "achieved": step_us,
                    "frac": floor_us / step_us,
                    "note": "vector-ALU time of one compute unit per "
                            "sample step (9 instructions per row); "
                            "clouds run side by side, %d of the chip's "
                            "256 units busy" % clouds}}
        return report

    # "auto" against the clock: whole calls of knn / radius / nearest on
    # uniform clouds of growing size under both strategies, with what the
    # cost model of "auto" picks for that size (`--case crossover`; not part
    # of the default line).  `auto_is_faster_or_within` is the time auto's
    # pick loses against the better strategy, as a fraction of that one.
    def case_crossover(self, reps):
        t, pca = self.torch, self.pca
        pick = t.ops.pytorch_cluster_amd.strategy_for
        report = {}
        before = pca.get_search_strategy()
        try:
            for segments in (1, 8):
                for n in (2048, 4096, 8192, 16384, 32768, 65536, 131072,
                          262144):
                    g = t.Generator().manual_seed(n + segments)
                    x = t.rand(n * segments, 3, generator=g).to(self.dev)
                    b = (t.arange(n * segments) // n).to(self.dev)
                    xq, bq = x[::3].contiguous(), b[::3].contiguous()
                    r = 0.6 * n ** (-1.0 / 3.0)
                    calls = {
                        "knn": lambda: pca.knn(x, x, 16, b, b,
                                               batch_size=segments),
                        "radius": lambda: pca.radius(
                            x, x, r, b, b, max_num_neighbors=32,
                            batch_size=segments),
                        "nearest": lambda: pca.nearest(x, xq, b, bq)}
                    for op, call in calls.items():
                        ms = {}
                        for strategy in ("scan", "binned"):
                            pca.set_search_strategy(strategy)
                            ms[strategy], _ = _median_ms(t, call, reps or 5)
                        pca.set_search_strategy("auto")
                        if op == "nearest":
                            picked = pick(op, xq.shape[0], x.shape[0],
                                          segments)
                        else:
                            picked = pick(op, x.shape[0], x.shape[0],
                                          segments)
                        best = min(ms.values())
                        report["%s %d x %d" % (op, segments, n)] = {
                            "scan_ms": ms["scan"], "binned_ms": ms["binned"],
                            "auto_picks": picked,
                            "auto_loses": ms[picked] / best - 1.0}
        finally:
            pca.set_search_strategy(before)
        return report

    # the headline workload and large clouds through both search strategies
    # (binned: rows ordered along a space-filling curve, exact pruning by tile
    # boxes; same edges as the scan); `search_ms` covers binning and search
    def case_strategies(self, reps):
        t, pca = self.torch, self.pca
        report = {}
        lidar = self.testing.lidar_scans(0)
        x, y = lidar["x"].to(self.dev), lidar["y"].to(self.dev)
        bx, by = lidar["batch_x"].to(self.dev), lidar["batch_y"].to(self.dev)
        big = t.rand(1000000, 3, generator=t.Generator().manual_seed(1))
        big = big.to(self.dev)
        c3 = self.testing.gaussian_mixture_batched(0)
        x3, b3 = c3["x"].to(self.dev), c3["batch"].to(self.dev)
        lidar8 = self.testing.lidar_scans(0, query_stride=8)
        nx, ny = lidar8["x"].to(self.dev), lidar8["y"].to(self.dev)
        nbx = lidar8["batch_x"].to(self.dev)
        nby = lidar8["batch_y"].to(self.dev)
        N, M = x.shape[0], y.shape[0]
        cases = (("configs[4] ragged LiDAR-like knn k=16",
                  lambda: pca.knn(x, y, 16, bx, by, batch_size=8),
                  M, _search_bytes(N, M, 3, 16)),
                 ("knn 1000000 uniform points onto themselves k=16",
                  lambda: pca.knn(big, big, 16), big.shape[0],
                  _search_bytes(big.shape[0], big.shape[0], 3, 16)),
                 ("configs[2] radius_graph 8x16384 r=0.05 max 32",
                  lambda: pca.radius_graph(x3, 0.05, b3, max_num_neighbors=32,
                                           batch_size=8), x3.shape[0], None),
                 ("radius 1000000 uniform points onto themselves r=0.01 "
                  "max 32",
                  lambda: pca.radius(big, big, 0.01, max_num_neighbors=32),
                  big.shape[0], None),
                 ("nearest on the LiDAR-like points",
                  lambda: pca.nearest(nx, ny, nbx, nby), nx.shape[0],
                  (nx.shape[0] + ny.shape[0]) * 12 + nx.shape[0] * 8))
        for name, fn, queries, nbytes in cases:
            for strategy in ("scan", "binned"):
                pca.set_search_strategy(strategy)
                try:
                    ms, out = _median_ms(t, fn, reps or 5)
                    search_ms = _search_ms(t, self.capi, self.events, fn, 1)
                finally:
                    pca.set_search_strategy("scan")
                entry = {
                    "ms": ms, "queries_per_s": queries / ms * 1e3,
                    "search_ms": search_ms,
                    "edges": int(out.shape[1]) if out.dim() == 2 else None}
                if nbytes is None and strategy == "binned":
                    # radius: the edge list actually written
                    nbytes = (2 * queries * 12 + int(out.shape[1]) * 16)
                if strategy == "binned":
                    entry["roofline"] = _hbm_roofline(
                        "binning passes + binned search kernel", search_ms,
                        nbytes, "bytes a search has to move (points and "
                        "queries once, the int64 edge list once) over the "
                        "time from the first binning pass to the end of the "
                        "search kernel, against the HBM peak")
                report["%s, strategy %s" % (name, strategy)] = entry
        return report


def other_configs(torch, pca, testing, dev, only=None):
    """End-to-end times and search-kernel rooflines of the other benchmark
    configurations (median of a few calls, inputs resident in HBM); reported
    beside the headline number, they are parity-test cases, not the
    benchmark."""
    cases = Cases(torch, pca, testing, dev)
    report = {}
    before = pca.get_search_strategy()
    try:
        for name in (only or cases.names()):
            report.update(cases.run(name))
    finally:
        pca.set_search_strategy(before)
    return report


def measured_traffic():
    """HBM bytes per launch of the dominant kernel from the committed rocprof
    counter summary, and the commit that summary was measured at, if there is
    one: (bytes, commit)."""
    import re
    path = os.path.join(ROOT, "profiles", "knn_lowd_lidar_traffic.md")
    try:
        with open(path) as f:
            text = f.read()
    except OSError:
        return None, None
    found = re.search(r"hbm_bytes_per_launch:\s*(\d+)", text)
    commit = re.search(r"[Mm]easured at commit\s+([0-9a-f]{7,40})", text)
    return (int(found.group(1)) if found else None,
            commit.group(1) if commit else None)


def built_commit():
    """The commit the native libraries were built from (written by
    pytorch_cluster_amd/build.py; "+" marks a tree with local changes)."""
    path = os.path.join(ROOT, "pytorch_cluster_amd", "build_commit.txt")
    try:
        with open(path) as f:
            return f.read().strip() or None
    except OSError:
        return None


def probe_feat_loop(reps):
    """pytorch_cluster_amd/csrc/probes/feat_loop_probe.hip: the loop of the
    feature-space filter with everything but the matrix-core chain taken
    away, then put back piece by piece (best of `reps` launches each)."""
    import ctypes
    here = os.path.dirname(os.path.abspath(__file__))
    lib = ctypes.CDLL(os.path.join(here, "pytorch_cluster_amd",
                                   "libpca_probe.so"))
    text = ctypes.create_string_buffer(1 << 16)
    count = lib.pca_probe_feat_loop(ctypes.c_int(reps), text,
                                    ctypes.c_int(len(text)))
    if count < 0:
        sys.exit("bench.py: the probe failed (a HIP call returned an error)")
    sys.stdout.write(text.value.decode())


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the short timings of the other benchmark "
                         "configurations")
    ap.add_argument("--extras-only", action="store_true",
                    help="run only the other benchmark configurations and "
                         "print their timings (for kernel traces of those "
                         "paths)")
    ap.add_argument("--case", action="append", default=None,
                    help="with --extras-only: run only this configuration "
                         "(c1, c2, c3, c4, c4cos, d256, clouds64, "
                         "nearest_points, nearest_codes, fps, strategies, "
                         "crossover; "
                         "repeatable)")
    ap.add_argument("--strategy", choices=("scan", "binned", "auto"),
                    default="scan",
                    help="search strategy of the timed steps: scan (default "
                         "here: the brute-force kernel the metric's roofline "
                         "figure is about), binned or auto (the library's "
                         "default; rows ordered along a space-filling curve, "
                         "exact pruning; same edges)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 1 GiB device copy three times, so "
                         "that a counter profile of this command can scale "
                         "FETCH_SIZE / WRITE_SIZE by a kernel of known traffic")
    ap.add_argument("--probe", choices=("feat_loop",), default=None,
                    help="run a measurement aid instead of the benchmark: "
                         "feat_loop = the stripped matrix-core loop of the "
                         "feature-space filter, variant by variant (one JSON "
                         "line each)")
    args = ap.parse_args()
    if args.probe == "feat_loop":
        return probe_feat_loop(max(args.steps // 4, 3))
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus %d is not "
                 "supported (the path would shard by segment, without "
                 "communication)" % args.gpus)

    import torch
    import pytorch_cluster_amd as pca
    from pytorch_cluster_amd import testing
    from pytorch_cluster_amd._native import capi

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    if args.extras_only:
        print(json.dumps({"other_configs":
                          other_configs(torch, pca, testing, dev,
                                        args.case)}))
        return
    data = testing.lidar_scans(0)
    B = data["batch_size"]
    ptr_x = testing.pointers(data["batch_x"], B)
    ptr_y = testing.pointers(data["batch_y"], B)
    x, y = data["x"].to(dev), data["y"].to(dev)
    bx, by = data["batch_x"].to(dev), data["batch_y"].to(dev)
    n, m = x.shape[0], y.shape[0]
    pairs = int(((ptr_x[1:] - ptr_x[:-1]) * (ptr_y[1:] - ptr_y[:-1])).sum())

    pca.set_search_strategy(args.strategy)
    binned = args.strategy != "scan"

    def step():
        return pca.knn(x, y, K, bx, by, batch_size=B)

    for _ in range(args.warmup):
        out = step()
    torch.cuda.synchronize()
    assert out.shape == (2, m * K)

    events = HipEvents(torch)
    pairs_of_events = [(events.create(), events.create())
                       for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for start, stop in pairs_of_events:
        capi.pca_time_next_search(start, stop)
        out = step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0

    kernel_ms = [events.elapsed_ms(a, b) for a, b in pairs_of_events]
    for a, b in pairs_of_events:
        events.destroy(a)
        events.destroy(b)
    kernel_s = sum(kernel_ms) / len(kernel_ms) / 1e3
    flops = FLOP_PER_PAIR * pairs
    achieved = flops / kernel_s / 1e12

    result = {
        "metric": "kNN queries/sec (k=16, 3D, 1M pts)",
        "value": m * args.steps / elapsed,
        "unit": "queries/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": elapsed / args.steps * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "configs[4]: ragged LiDAR-like knn(x, y, k=16, "
                        "batch_x, batch_y), 8 scans of 60k-200k points, "
                        "y = every 4th point",
            "strategy": args.strategy,
            "points": n, "queries": m, "k": K, "dim": 3, "segments": B,
            "pairs": pairs, "seed": 0,
        },
        "edges_per_s": m * K * args.steps / elapsed,
        "roofline": {
            "bound": "mfma",
            "bound_detail": "fp32 peak (vector = matrix, 157.3 TFLOP/s); the "
                            "distance filter runs on the matrix cores as "
                            "split-bf16 products, every kept distance is "
                            "exact fp32; flops counted are the algorithmic "
                            "3*D per pair",
            "kernel": "knn_lowd_mc_kernel<3,16>",
            "achieved": achieved,
            "peak": PEAK_FP32_TFLOPS,
            "unit": "TFLOP/s",
            "frac": achieved / PEAK_FP32_TFLOPS,
            "kernel_ms": kernel_s * 1e3,
            "flop_per_launch": flops,
            "traffic": measured_traffic()[0],
            "traffic_commit": measured_traffic()[1],
        },
        "commit": built_commit(),
    }
    if binned:
        # the events bracket binning + search here, and the work is not the
        # 9 flop x all pairs the roofline figure prices: no roofline claim
        result["roofline"] = None
        result["search_ms"] = kernel_s * 1e3
    if not binned:
        # the same steps with the binned search (same edges; the library's
        # default stays the scan, which the roofline figure is about)
        pca.set_search_strategy("binned")
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        result["with_binned_strategy"] = {
            "value": m * args.steps / dt, "unit": "queries/s",
            "ms_per_step": dt / args.steps * 1e3}
    if not args.no_extras:
        result["other_configs"] = other_configs(torch, pca, testing, dev)
    if args.copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).fill_(1.0)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(data, ptr_x, ptr_y)
        result["cpu_baseline"]["build"] = cpu_build_baseline(pca, data)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
