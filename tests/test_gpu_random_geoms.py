"""GPU parity on seeded random geometries: the dispatch picks one of several kernels per layer
shape (direct, row-gather, tiled, streaming, staged, register-resident ...), and the boundaries
between them are where a wrong condition would hide.  Every case is compared bit for bit with
the CPU oracle; the shapes are small enough for the oracle to take milliseconds."""
import numpy as np
import pytest

import oracle
from gpu_helpers import assert_same, conv, depthwise_generic, depthwise_hwc, linear, rand_s8, rand_u8, rng_for
from pulp_nn_amd import PulpNNError

pytestmark = pytest.mark.gpu


def _bn(r, n, bn_bits):
    if bn_bits == 32:
        return r.integers(2 ** 10, 2 ** 13 + 1, n), r.integers(-2 ** 16, 2 ** 16 + 1, n), 18
    return r.integers(2 ** 20, 2 ** 24 + 1, n), r.integers(-2 ** 36, 2 ** 36 + 1, n), 34


def _flags(r):
    return [(1, 1), (1, 0), (0, 0), (0, 1)][int(r.integers(0, 4))]


def _conv_cases(n, seed):
    r = rng_for(seed)
    cases = []
    while len(cases) < n:
        ci = int(r.choice([1, 2, 3, 4, 5, 8, 12, 16, 24, 32, 64, 128]))
        co = int(r.choice([1, 5, 8, 16, 17, 24, 32, 33, 64, 96, 130]))
        ky, kx = int(r.integers(1, 4)), int(r.integers(1, 4))
        h, w = int(r.integers(ky, 15)), int(r.integers(kx, 15))
        pads = tuple(int(v) for v in (r.integers(0, ky), r.integers(0, ky), r.integers(0, kx), r.integers(0, kx)))
        s = int(r.integers(1, 3))
        b = int(r.integers(1, 4))
        if (h + pads[0] + pads[1] - ky) // s + 1 < 1 or (w + pads[2] + pads[3] - kx) // s + 1 < 1:
            continue
        cases.append((b, h, w, ci, co, ky, kx, pads, (s, s)))
    return cases


@pytest.mark.parametrize("bn_bits", [32, 64])
@pytest.mark.parametrize("case", _conv_cases(40, 9001), ids=lambda c: "x".join(map(str, c[:7])) + "p%d%d%d%ds%d" % (c[7] + (c[8][0],)))
def test_random_conv(case, bn_bits):
    B, H, W, Ci, Co, ky, kx, pads, strides = case
    r = rng_for(hash(case) % (2 ** 31) + bn_bits)
    relu, bn = _flags(r)
    x, w, b = rand_u8(r, (B, H, W, Ci)), rand_s8(r, (Co, ky, kx, Ci)), rand_s8(r, (Co,))
    k, lam, bshift = _bn(r, Co, bn_bits)
    K = ky * kx * Ci
    lg = int(np.log2(max(K, 2) ** 0.5 * 128 * 74))
    shift = bshift if (relu and bn) else ((lg + 3) if relu == 1 else max(lg - 7, 0))
    mult = int(r.integers(64, 1025))
    want = oracle.conv(x, w, b, k, lam, mult, shift, pads, strides, relu, bn, bn_bits)
    got = conv(x, w, b, k, lam, mult, shift, pads, strides, relu, bn, bn_bits)
    assert_same(got, want, "conv %s" % (case,))


def _dw_cases(n, seed):
    r = rng_for(seed)
    cases = []
    while len(cases) < n:
        ch = int(r.choice([4, 8, 16, 32, 64, 128, 5, 70]))
        w = int(r.choice([4, 8, 16, 32, 64, 12, 20, 9]))
        h = w if r.random() < 0.5 else int(r.integers(3, 20))
        s = int(r.integers(1, 3))
        # (left padding 0 with right padding 1 is left out: there the reference pads a wrong count,
        # a documented deviation)
        lr = [(1, 1), (1, 0), (0, 0)][int(r.integers(0, 3))]
        pads = (1, 1, 1, 1) if r.random() < 0.7 else (int(r.integers(0, 2)), int(r.integers(0, 2))) + lr
        b = int(r.choice([1, 2, 4, 8, 16]))
        if (h + pads[0] + pads[1] - 3) // s + 1 < 1 or (w + pads[2] + pads[3] - 3) // s + 1 < 1:
            continue
        cases.append((b, ch, h, w, pads, s))
    return cases


@pytest.mark.parametrize("bn_bits", [32, 64])
@pytest.mark.parametrize("case", _dw_cases(40, 9002), ids=lambda c: "x".join(map(str, c[:4])) + "p%d%d%d%ds%d" % (c[4] + (c[5],)))
def test_random_depthwise(case, bn_bits):
    B, CH, H, W, pads, s = case
    r = rng_for(hash(case) % (2 ** 31) + bn_bits)
    relu, bn = _flags(r)
    x, wt, b = rand_u8(r, (B, CH, H, W)), rand_s8(r, (CH, 3, 3)), rand_s8(r, (CH,))
    if bn_bits == 32:
        k, lam, bshift = r.integers(2 ** 12, 2 ** 14 + 1, CH), r.integers(-2 ** 16, 2 ** 16 + 1, CH), 16
    else:
        k, lam, bshift = r.integers(2 ** 20, 2 ** 24 + 1, CH), r.integers(-2 ** 36, 2 ** 36 + 1, CH), 28
    shift = bshift if (relu and bn) else (14 if relu else 6)
    want = oracle.depthwise_generic(x, wt, b, k, lam, 900, shift, pads, (s, s), relu, bn, bn_bits)
    got = depthwise_generic(x, wt, b, k, lam, 900, shift, pads, (s, s), relu, bn, bn_bits)
    assert_same(got, want, "depthwise %s" % (case,))
    if pads == (1, 1, 1, 1):
        # the fused HWC entry point: either the same bytes or a clean refusal
        x_hwc = np.ascontiguousarray(x.transpose(0, 2, 3, 1))
        try:
            got2 = depthwise_hwc(x_hwc, wt, b, k, lam, 900, shift, s, relu, bn, bn_bits)
        except PulpNNError as err:
            assert err.code == 2
        else:
            assert_same(got2, want, "depthwise_hwc %s" % (case,))


def _dw_group_cases(n, seed):
    """Whole 64-channel groups with rows of whole dwords and output columns in whole groups of four: the shapes whose
    bands are staged by LDS-direct loads (16-byte pieces that may straddle the image's first and last row)."""
    r = rng_for(seed)
    cases = []
    while len(cases) < n:
        ch = int(r.choice([64, 128, 192]))
        w = 4 * int(r.integers(2, 16))
        h = int(r.integers(3, 41))
        s = int(r.integers(1, 3))
        pads = (int(r.integers(0, 2)), int(r.integers(0, 2))) + [(1, 1), (1, 0), (0, 0)][int(r.integers(0, 3))]
        ho, wo = (h + pads[0] + pads[1] - 3) // s + 1, (w + pads[2] + pads[3] - 3) // s + 1
        if ho < 1 or wo < 1 or wo % 4:
            continue
        cases.append((int(r.choice([1, 2, 5])), ch, h, w, pads, s))
    return cases


@pytest.mark.parametrize("bn_bits", [32, 64])
@pytest.mark.parametrize("case", _dw_group_cases(40, 9102), ids=lambda c: "x".join(map(str, c[:4])) + "p%d%d%d%ds%d" % (c[4] + (c[5],)))
def test_random_depthwise_whole_groups(case, bn_bits):
    B, CH, H, W, pads, s = case
    r = rng_for(hash(case) % (2 ** 31) + bn_bits)
    relu, bn = _flags(r)
    x, wt, b = rand_u8(r, (B, CH, H, W)), rand_s8(r, (CH, 3, 3)), rand_s8(r, (CH,))
    if bn_bits == 32:
        k, lam, bshift = r.integers(2 ** 12, 2 ** 14 + 1, CH), r.integers(-2 ** 16, 2 ** 16 + 1, CH), 16
    else:
        k, lam, bshift = r.integers(2 ** 20, 2 ** 24 + 1, CH), r.integers(-2 ** 36, 2 ** 36 + 1, CH), 28
    shift = bshift if (relu and bn) else (14 if relu else 6)
    want = oracle.depthwise_generic(x, wt, b, k, lam, 900, shift, pads, (s, s), relu, bn, bn_bits)
    got = depthwise_generic(x, wt, b, k, lam, 900, shift, pads, (s, s), relu, bn, bn_bits)
    assert_same(got, want, "depthwise %s" % (case,))


def _linear_cases(n, seed):
    r = rng_for(seed)
    return [(int(r.choice([1, 2, 7, 64, 65, 130, 256, 257, 300])), int(r.choice([16, 32, 48, 100, 256, 1000, 37])),
             int(r.choice([1, 10, 16, 17, 100, 257]))) for _ in range(n)]


@pytest.mark.parametrize("bn_bits", [32, 64])
@pytest.mark.parametrize("case", _linear_cases(24, 9003), ids=lambda c: "x".join(map(str, c)))
def test_random_linear(case, bn_bits):
    B, K, N = case
    r = rng_for(hash(case) % (2 ** 31) + bn_bits)
    relu, bn = _flags(r)
    x, w, b = rand_u8(r, (B, K)), rand_s8(r, (N, K)), rand_s8(r, (N,))
    k, lam, bshift = _bn(r, N, bn_bits)
    lg = int(np.log2(max(K, 2) ** 0.5 * 128 * 74))
    shift = bshift if (relu and bn) else ((lg + 3) if relu == 1 else max(lg - 7, 0))
    mult = int(r.integers(64, 1025))
    want = oracle.linear(x, w, b, k, lam, mult, shift, relu, bn, bn_bits)
    got = linear(x, w, b, k, lam, mult, shift, relu, bn, bn_bits)
    assert_same(got, want, "linear %s" % (case,))


def _pw_cases(n, seed):
    """Pixel counts on both sides of the streaming kernel's threshold, channel counts on and off its list."""
    r = rng_for(seed)
    px = [(1, 45, 45), (2, 32, 32), (4, 64, 64), (7, 68, 68), (8, 64, 64), (5, 81, 81), (3, 100, 110)]
    return [px[int(r.integers(0, len(px)))] + (int(r.choice([16, 48, 64, 128, 200, 256])),
                                              int(r.choice([16, 32, 64, 100, 128, 192, 256]))) for _ in range(n)]


@pytest.mark.parametrize("bn_bits", [32, 64])
@pytest.mark.parametrize("case", _pw_cases(20, 9004), ids=lambda c: "x".join(map(str, c)))
def test_random_pointwise(case, bn_bits):
    B, H, W, Ci, Co = case
    r = rng_for(hash(case) % (2 ** 31) + bn_bits)
    relu, bn = _flags(r)
    x, w, b = rand_u8(r, (B, H, W, Ci)), rand_s8(r, (Co, 1, 1, Ci)), rand_s8(r, (Co,))
    k, lam, bshift = _bn(r, Co, bn_bits)
    lg = int(np.log2(max(Ci, 2) ** 0.5 * 128 * 74))
    shift = bshift if (relu and bn) else ((lg + 3) if relu == 1 else max(lg - 7, 0))
    mult = int(r.integers(64, 1025))
    want = oracle.pointwise(x, w, b, k, lam, mult, shift, relu, bn, bn_bits)
    got = conv(x, w, b, k, lam, mult, shift, (0, 0, 0, 0), (1, 1), relu, bn, bn_bits, out_hw=(H, W),
               fn="pulp_nn_pointwise_HoWo_parallel")
    assert_same(got, want, "pointwise %s" % (case,))
