"""CPU model of the fp16 matrix-core filter of the feature-space kNN
(pytorch_cluster_amd/csrc/knn_feat_impl.hpp): the value l the filter derives
for a (row, query) pair must never exceed the distance e the reference's
scalar loop computes (csrc/cuda/knn_cuda.cu:61-64), and F(l) must never fall
below it -- on random rows and on rows built to make the fp16 roundings add up
(every component at a rounding midpoint, query equal to the row, mixed scales,
values at the flush-to-zero limit).

The model rounds exactly as the kernels do (numpy float16, the same flush and
the same truncated parts of W) and sums the products in float64, i.e. without
the matrix cores' own accumulation error; the test therefore demands that the
roundings alone leave the share of the budget that the header of
knn_feat_impl.hpp reserves for accumulation (2^-22 x 2.01 of |X|^2 + |Y|^2 per
term of the chain: 0.13 x 2^-10 at 256 components, 0.26 x 2^-10 at 512) unused.
"""
import math

import numpy as np
import pytest

from helpers import stable_seed

def rho_of(d):
    """2^-9 up to 256 components, 2^-8 beyond (feat_rho)."""
    return 1.0 / 512.0 if d <= 256 else 1.0 / 256.0


def inv_sigma(max_abs):
    if max_abs == 0:
        return 1.0
    bits = np.float32(max_abs).view(np.uint32)
    e = 137 - int((bits >> 23) & 0xff)
    return float(2.0 ** max(-100, min(100, e)))


def h(v):
    """fp16 nearest-even, magnitudes below 2^-14 flushed to zero."""
    v = np.asarray(v, dtype=np.float32)
    out = v.astype(np.float16).astype(np.float64)
    out[np.abs(v) < 2.0 ** -14] = 0.0
    return out


def h_down(v):
    """Largest flushed fp16 <= v (v >= 0)."""
    r = np.float16(np.float32(v))
    if float(r) > v:
        r = np.nextafter(r, np.float16(0))
    if v >= 65504.0:
        r = np.float16(65504.0)
    return 0.0 if float(r) < 2.0 ** -14 else float(r)


def w_parts(w):
    a1 = h_down(w / 32768.0)
    r1 = w - a1 * 32768.0
    a2 = h_down(r1 / 16.0)
    r2 = r1 - a2 * 16.0
    a3 = h_down(r2 * 128.0)
    return a1 * 32768.0 + a2 * 16.0 + a3 / 128.0


def reference_distances(x, y):
    """e[j, i]: one fused multiply-add per component in ascending order, in
    fp32 (float64 holds the exact product and sum of two fp32 numbers'
    product and a third before the one rounding)."""
    e = np.zeros((len(y), len(x)), dtype=np.float32)
    for c in range(x.shape[1]):
        diff = (x[None, :, c] - y[:, None, c]).astype(np.float32)
        e = (diff.astype(np.float64) ** 2 + e.astype(np.float64)).astype(
            np.float32)
    return e.astype(np.float64)


def check(x, y):
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.ascontiguousarray(y, dtype=np.float32)
    d = x.shape[1]
    RHO = rho_of(d)
    GROW = 1.0 + 4.1 * RHO
    inv = inv_sigma(max(np.abs(x).max(), np.abs(y).max()))
    scale2 = inv * inv
    c0 = d / 4096.0 + d * 2.0 ** -149 * scale2
    xs = (x * np.float32(inv)).astype(np.float32)
    ys = (y * np.float32(inv)).astype(np.float32)
    hx = h(xs)
    hy = h(-2.0 * ys.astype(np.float64))
    xsq32 = np.zeros(len(x), dtype=np.float32)
    for c in range(d):  # (any fp32 summation order serves)
        xsq32 = (x[:, c].astype(np.float64) ** 2 + xsq32).astype(np.float32)
    w = np.array([w_parts(float(v) * scale2 * (1.0 - RHO)) for v in xsq32])
    s = w[None, :] + hy @ hx.T
    ysq = (ys.astype(np.float64) ** 2).sum(1)
    shift = ysq * (1.0 - RHO) - c0
    widen = 6.0 * RHO * ysq + 2.0 * c0
    lower = s + shift[:, None]
    upper = (lower + widen[:, None]) * GROW
    e = reference_distances(x, y) * scale2
    norms = (xs.astype(np.float64) ** 2).sum(1)[None, :] + ysq[:, None]
    # what accumulation may still take (2^-22 x 2.01 per term of the chain)
    room = max(0.15, (d + 16) * 2.01 / 4096.0) * 2.0 ** -10 * norms
    assert (lower + room <= e + 1e-300).all(), \
        "lower bound above the reference's distance"
    assert (e <= upper - room).all(), "upper bound below it"
    return float(np.max((lower - (e - RHO * norms - c0))
                        / (RHO * norms + c0)))


def midpoint_rows(rng, n, d, exponents, side):
    # every component sits just below (side = -1) or just above (+1) the
    # middle between two fp16 numbers (odd multiples of 2^-11 of its power of
    # two), all with one sign: every rounding goes the same way by nearly the
    # largest amount, and in a row times itself the errors add up
    frac = 1.0 + (2 * rng.integers(0, 1024, (n, d)) + 1) * 2.0 ** -11
    frac = frac + side * 2.0 ** -21
    return (frac * 2.0 ** exponents).astype(np.float32)


@pytest.mark.parametrize("d", [9, 64, 128, 256, 300, 512])
def test_random_rows(d):
    rng = np.random.default_rng(d)
    x = rng.standard_normal((400, d))
    y = rng.standard_normal((60, d))
    check(x, y)
    check(x, x[:60])  # queries that are rows: distance zero


@pytest.mark.parametrize("d", [16, 128, 256, 512])
def test_rounding_midpoints_with_one_sign(d):
    rng = np.random.default_rng(d + 1)
    used = []
    for side in (-1, 1):
        x = midpoint_rows(rng, 300, d, 0, side)
        used.append(check(x, x[:50]))
        y = midpoint_rows(rng, 50, d, 0, side)
        used.append(check(x, y))
    # rounding down in a row times itself takes about half of the budget (the
    # products are 2^-10 too small, and rho = 2 x 2^-10): the case is as hard
    # as it is meant to be
    # (a quarter where rho is 2^-8)
    assert 0.3 <= max(used) * (rho_of(d) * 512.0) <= 0.7


@pytest.mark.parametrize("case", ["mixed", "flush_limit", "tiny", "huge",
                                  "outlier", "near_duplicates"])
def test_scales(case):
    rng = np.random.default_rng(stable_seed(case))
    d = 96
    if case == "mixed":
        x = midpoint_rows(rng, 300, d, rng.integers(-12, 1, (300, 1)), -1)
        y = midpoint_rows(rng, 40, d, rng.integers(-12, 1, (40, 1)), -1)
    elif case == "flush_limit":
        # after scaling most components lie around 2^-14, where fp16 flushes
        x = rng.standard_normal((300, d)) * 2.0 ** -24
        x[0] = 1.0
        y = rng.standard_normal((40, d)) * 2.0 ** -24
    elif case == "tiny":
        x = rng.standard_normal((300, d)) * 1e-21
        y = rng.standard_normal((40, d)) * 1e-21
    elif case == "huge":
        x = rng.standard_normal((300, d)) * 1e16
        y = rng.standard_normal((40, d)) * 1e16
    elif case == "outlier":
        x = rng.standard_normal((300, d))
        x[5] *= 1e6
        y = rng.standard_normal((40, d))
    else:
        base = rng.standard_normal((10, d))
        x = np.repeat(base, 30, 0) * (1 + 1e-6 * rng.standard_normal((300, d)))
        y = base * (1 + 1e-6 * rng.standard_normal((10, d)))
    check(x, y)


# ---- the cut inside the matrix product (knn_feat_wide_impl.hpp) --------------
# The eight-wave first stage lets the chain of matrix instructions subtract the
# cut: the query's operand carries -c_rep as three fp16 numbers, the packed
# rows the powers of two 2^15, 2^5, 2^-5.  Checked here, with the chain
# modelled as fp32 additions in several orders: c_rep is what its parts say
# and lies above the cut by the rounding the three extra terms can add, D(c);
# every pair the plain test `s < cut` must flag comes out negative; and the
# value kept for a flagged pair, acc + float_below(c_rep - D), stays within
# [S - room - 2 D, S + room] of the exact sum S.

def h_down_any(v):
    """h_down() for the kernel's feat_h_down (v >= 0)."""
    return h_down(v)


def cut_parts(c):
    """wide_cut_parts: (p0, p1, p2) as fp16 values with sign, and rep."""
    neg = c < 0.0
    a = -c if neg else c
    if not a < 2.0e9:
        return None
    a0 = h_down_any(a / 32768.0)
    r0 = a - a0 * 32768.0
    a1 = h_down_any(r0 / 32.0)
    r1 = r0 - a1 * 32.0
    a2 = h_down_any(r1 * 32.0)
    r2 = r1 - a2 / 32.0
    if not neg and r2 > 0.0:
        a2 = 2.0 ** -14 if a2 == 0.0 else float(
            np.nextafter(np.float16(a2), np.float16(np.inf)))
        if a2 > 65504.0:
            return None
        r2 = r1 - a2 / 32.0
    mag = a - r2
    sign = -1.0 if neg else 1.0
    return (sign * a0, sign * a1, sign * a2), sign * mag


def fold_err(d, c):
    return (d + 23) * 2.0 ** -22 * abs(c)


def float_below(v):
    f = np.float32(v)
    if float(f) > v:
        f = np.nextafter(f, np.float32(-np.inf))
    return f


def chain(terms, order):
    acc = np.float32(0.0)
    for i in order:
        acc = np.float32(acc + np.float32(terms[i]))  # (terms are fp32-exact)
    return acc


@pytest.mark.parametrize("d", [16, 64, 128])
def test_cut_inside_the_product(d):
    rng = np.random.default_rng(stable_seed("fold", d))
    RHO = rho_of(d)
    x = rng.standard_normal((40, d)).astype(np.float32)
    x[:8] *= 10.0 ** rng.integers(-4, 1, (8, 1))
    y = (x[:6] + 0.05 * rng.standard_normal((6, d))).astype(np.float32)
    inv = inv_sigma(max(np.abs(x).max(), np.abs(y).max()))
    scale2 = inv * inv
    xs = (x * np.float32(inv)).astype(np.float32)
    ys = (y * np.float32(inv)).astype(np.float32)
    hx = h(xs)
    hy = h(-2.0 * ys.astype(np.float64))
    xsq = (x.astype(np.float64) ** 2).sum(1)
    ysq = (ys.astype(np.float64) ** 2).sum(1)
    checked = 0
    for j in range(len(y)):
        for i in range(len(x)):
            w = float(xsq[i]) * scale2 * (1.0 - RHO)
            a1 = h_down(w / 32768.0)
            r1 = w - a1 * 32768.0
            a2 = h_down(r1 / 16.0)
            r2 = r1 - a2 * 16.0
            a3 = h_down(r2 * 128.0)
            base = [a1 * 32768.0, a2 * 16.0, a3 / 128.0] + list(hx[i] * hy[j])
            total = float(np.sum(np.array(base, dtype=np.float64)))
            norms = float((xs[i].astype(np.float64) ** 2).sum() + ysq[j])
            room = max(0.15, (d + 16) * 2.01 / 4096.0) * 2.0 ** -10 * norms
            # cuts around the pair's own value, far above, below, negative
            for c0 in (total + room * 1.0001 + 1e-6, total * 1.5 + 3.0,
                       total - abs(total) * 0.01 - 1.0, abs(total) * 40.0 + 7.0,
                       -abs(total) * 0.3 - 0.125, 2.0 ** -20):
                c0 = float(np.float32(c0))
                got = cut_parts(c0 + fold_err(d, c0) * 1.002 + 1e-30)
                if got is None:
                    # beyond the parts' range: the kernel works without a cut
                    assert abs(c0) > 1.9e9
                    checked += 1
                    continue
                (p0, p1, p2), rep = got
                for part in (p0, p1, p2):
                    assert float(np.float16(part)) == part
                    assert part == 0.0 or abs(part) >= 2.0 ** -14
                assert rep == p0 * 32768.0 + p1 * 32.0 + p2 / 32.0
                err = fold_err(d, rep)
                assert rep >= c0 + err
                recon = float_below(rep - err)
                terms = base + [-p0 * 32768.0, -p1 * 32.0, -p2 / 32.0]
                n = len(terms)
                orders = [list(range(n)), list(range(n))[::-1],
                          list(rng.permutation(n)),
                          # the cut first, then the rest
                          [n - 3, n - 2, n - 1] + list(range(n - 3))]
                for order in orders:
                    acc = chain(terms, order)
                    bound = (d + 22) * 2.0 ** -22 * (2.01 * norms + abs(rep))
                    assert abs(float(acc) - (total - rep)) <= bound
                    if total + room <= c0:
                        assert acc < 0.0, "a pair the plain test flags got away"
                    key = float(np.float32(acc + recon))
                    assert key <= total + room
                    assert key >= total - room - 2.0 * err - 1e-30
                checked += 1
    assert checked == 40 * 6 * 6


# ---- the split-bf16 filter of the exact matrix-core kernel --------------------
# (pytorch_cluster_amd/csrc/knn_mfma_impl.hpp): t = w - 2 x.y from the
# products hi*hi + hi*lo + lo*hi of operands split into two bf16 numbers,
# w = fl(|x|^2) (1 - eps), cut = thresh (1 + eps) - fl(|y|^2) (1 - eps).  A pair
# whose exact distance is below thresh must come out with t < cut.

def bf16(v):
    """fp32 -> bf16, nearest-even, as fp32 values."""
    u = np.asarray(v, dtype=np.float32).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7fff + ((u >> 16) & 1)) >> 16) << 16
    return r.astype(np.uint32).view(np.float32)


def split(v):
    hi = bf16(v)
    lo = bf16((np.asarray(v, dtype=np.float32) - hi).astype(np.float32))
    return hi.astype(np.float64), lo.astype(np.float64)


def mfma_eps(d):
    return 2.0 ** -14 + (3 * d + 8) * 2.0 ** -21


def worst_split_mantissas(count):
    """fp32 numbers in [1, 2) whose split loses the most in a product with
    themselves: v^2 - (hi^2 + 2 hi lo) largest."""
    m = np.arange(0, 1 << 23, 7, dtype=np.uint32)
    v = (m | np.uint32(0x3f800000)).view(np.float32)
    hi, lo = split(v)
    loss = v.astype(np.float64) ** 2 - (hi * hi + 2.0 * hi * lo)
    return v[np.argsort(loss / v.astype(np.float64) ** 2)[-count:]]


@pytest.mark.parametrize("d", [9, 16, 40, 128])
def test_split_bf16_filter_keeps_near_duplicates(d):
    rng = np.random.default_rng(d)
    worst = worst_split_mantissas(4096)
    n = 200
    x = rng.choice(worst, (n, d)) * 2.0 ** rng.integers(-3, 4, (n, 1))
    x = x.astype(np.float32)
    # queries: the rows themselves, and rows a few ulps away
    y = np.concatenate([x[:50], np.nextafter(x[50:100], np.float32(4.0))])
    eps = mfma_eps(d)
    e = reference_distances(x, y)                         # [m, n]
    xsq = np.zeros(n, dtype=np.float32)
    for c in range(d):
        xsq = (x[:, c].astype(np.float64) ** 2 + xsq).astype(np.float32)
    ysq = np.zeros(len(y), dtype=np.float32)
    for c in range(d):
        ysq = (y[:, c].astype(np.float64) ** 2 + ysq).astype(np.float32)
    w = (xsq * np.float32(1.0 - eps)).astype(np.float32)
    wh, wl = split(w)
    xh, xl = split(x)
    yh, yl = split((-2.0 * y).astype(np.float32))
    # exact sums of the products the matrix cores form (no accumulation error)
    t = (wh + wl)[None, :] + yh @ xh.T + yh @ xl.T + yl @ xh.T
    # thresh just above the exact distance: the pair must be looked at
    thresh = np.nextafter(e.astype(np.float32), np.float32(np.inf)).astype(
        np.float64)
    cut = thresh * (1.0 + eps) - ysq.astype(np.float64)[:, None] * (1.0 - eps)
    scale = xsq.astype(np.float64)[None, :] + ysq.astype(np.float64)[:, None] \
        + thresh
    # what fp32 accumulation of the 3 d + 4 terms may still add
    room = (3 * d + 4) * 2.0 ** -22 * scale
    assert (t + room < cut).all()
    # and the case is as hard as meant: for y = x the split alone takes more
    # than half of the 2^-15 (|x|^2 + |y|^2) its analysis allows
    used = (t - (e - ysq.astype(np.float64)[:, None]
                 - eps * xsq.astype(np.float64)[None, :])) / (2.0 ** -15 * scale)
    assert 0.5 < used[:50, :50].diagonal().max() <= 1.0


# ---- 16-bit rows: what the reference's chain can lose (knn_feat_small_impl.hpp)

def _round16(v, bf16):
    """float32 array -> nearest fp16 / bf16 number (ties to even) as float32."""
    v = np.asarray(v, dtype=np.float32)
    if not bf16:
        return v.astype(np.float16).astype(np.float32)
    bits = v.view(np.uint32).astype(np.uint64)
    bits = (bits + 0x7fff + ((bits >> 16) & 1)) & 0xffff0000
    return bits.astype(np.uint32).view(np.float32)


def _chain16(x, y, bf16):
    """The reference's scalar loop in c10::Half / c10::BFloat16 arithmetic
    (csrc/cuda/knn_cuda.cu:61-64): every operator works in fp32 and rounds to
    16 bits.  x: [rows, d], y: [d]."""
    acc = np.zeros(len(x), dtype=np.float32)
    for c in range(x.shape[1]):
        diff = _round16(x[:, c] - y[c], bf16)
        sq = _round16(diff * diff, bf16)
        acc = _round16(acc + sq, bf16)
    return acc


def _chain_keep(bf16, sums):
    """kChainKeep.s[bf16][sums] of csrc/device_utils.hpp, restated: the square
    root of (1 - u)^(3 + sums), rounded down to 13 (bf16: 16) bits behind the
    point."""
    u = (2.0 ** -8 if bf16 else 2.0 ** -11) + 2.0 ** -23
    root = math.sqrt((1.0 - u) ** (3 + sums)) * (1.0 - 2.0 ** -30)
    unit = 65536.0 if bf16 else 8192.0
    return math.floor(root * unit) / unit


@pytest.mark.parametrize("bf16", [False, True])
def test_chain_keep_factors(bf16):
    # below what the roundings leave of a term (in exact arithmetic), and
    # short enough for a 16-bit number times the factor to be exact in fp32
    from fractions import Fraction
    u = (Fraction(1, 256) if bf16 else Fraction(1, 2048)) + Fraction(1, 2 ** 23)
    rng = np.random.default_rng(stable_seed("keep", bf16))
    v16 = _round16(rng.standard_normal(2000) *
                   10.0 ** rng.integers(-6, 4, 2000), bf16)
    for sums in range(0, 129):
        s = _chain_keep(bf16, sums)
        unit = 65536.0 if bf16 else 8192.0
        assert 0.5 <= s < 1.0 and s * unit == int(s * unit)
        assert Fraction(s) ** 2 <= (1 - u) ** (3 + sums)
        # (not more than one part in 1,000 below it: the bound stays tight)
        assert Fraction(s) ** 2 >= (1 - u) ** (3 + sums) * Fraction(999, 1000)
        prod32 = (v16.astype(np.float32) * np.float32(s)).astype(np.float64)
        assert (prod32 == v16.astype(np.float64) * s).all()


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("kind", ["normal", "first_term_large",
                                  "last_term_large", "tiny",
                                  "mixed_scales", "grid", "decreasing"])
def test_16bit_chain_against_the_real_distance(bf16, kind):
    # the filter of the one-kernel search sees rows and queries with component
    # j (of d) times chain_keep(d - j) and admits a row whenever that scaled
    # distance D' satisfies D' < h + d t: every row whose chain value H is
    # below h must do so, i.e. H >= D' - d t
    rng = np.random.default_rng(stable_seed("chain16", bf16, kind))
    u = (2.0 ** -8 if bf16 else 2.0 ** -11) + 2.0 ** -23
    t = 2.0 ** -126 if bf16 else 2.0 ** -24
    for d in (9, 33, 64, 128):
        x = rng.standard_normal((4000, d))
        y = rng.standard_normal(d)
        if kind == "first_term_large":
            x[:, 0] *= 40.0
            y[0] *= -40.0
        elif kind == "last_term_large":
            x[:, -1] *= 40.0
            y[-1] *= -40.0
        elif kind == "tiny":
            x *= 3e-4
            y *= 3e-4
        elif kind == "mixed_scales":
            x *= 10.0 ** rng.integers(-4, 2, (4000, 1))
        elif kind == "grid":
            x, y = np.round(2 * x) / 2, np.round(2 * y) / 2
        elif kind == "decreasing":
            # the sum stops growing: later terms fall below half a unit of it
            scale = 30.0 * 0.8 ** np.arange(d)
            x *= scale
            y *= scale
        x16 = _round16(x, bf16)
        y16 = _round16(y, bf16)
        H = _chain16(x16, y16, bf16).astype(np.float64)
        keep = np.array([_chain_keep(bf16, d - j) for j in range(d)])
        diff = x16.astype(np.float64) - y16.astype(np.float64)
        D = (diff ** 2).sum(1)
        scaled = ((keep * diff) ** 2).sum(1)
        finite = np.isfinite(H)
        assert finite.any()
        assert (H[finite] >= scaled[finite] - d * t).all(), (d, kind)
        # the scaled distance is the tighter of the two bounds (but for the
        # bits the factors were cut to)
        assert (scaled >= D * (1.0 - u) ** (d + 3) * (1.0 - 2.0 ** -11)).all()
        # and the bound is not vacuous: the chain does lose something
        if kind in ("normal", "decreasing"):
            assert (H[finite] < D[finite]).any()
