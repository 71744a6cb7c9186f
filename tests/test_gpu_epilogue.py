"""GPU parity of the requantisation epilogue's rarely taken branches.

Two kinds of test, all through the C ABI:

  * the hand-derived known answers of tests/golden/epilogue_kats.json, driven through real
    layers: the weights of a linear / pointwise layer are chosen so that the accumulator of
    channel c equals the vector's `phi` exactly, so the byte that comes back is the vector's
    `out` (no oracle involved);
  * seeded random layers against the oracle with parameters that force the slow forms of the
    device epilogue: batch-norm multipliers that do not fit 24 bits (32-bit build) or 32 bits
    (64-bit build), wrapping 32-bit products, multiplier-branch shifts below 16 (the int16
    narrowing then changes values), multipliers >= 32768 (negative as int16), shift 0 and a
    uint16 shift above 127.
"""
import json
import os

import numpy as np
import pytest

import oracle
from gpu_helpers import (assert_same, conv, depthwise_3x3_s1, depthwise_generic, depthwise_hwc, linear, nn, rand_s8,
                         rand_u8, rng_for)

pytestmark = pytest.mark.gpu

KATS = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "epilogue_kats.json")))


# ---- layers whose accumulators are prescribed ---------------------------------------------

def x_and_weights_for(phis, K):
    """One activation vector x (u8, K long) and one weight row per phi with w . x == phi.
    x = 255 everywhere but 1 in the last two places; phi = 255*A + r with |r| <= 127."""
    x = np.full(K, 255, np.uint8)
    x[K - 2:] = 1
    w = np.zeros((len(phis), K), np.int8)
    for c, phi in enumerate(phis):
        A = int(round(phi / 255))
        r = phi - 255 * A
        assert abs(r) <= 127 and abs(A) <= 127 * (K - 2), phi
        j = 0
        while A != 0:
            step = max(-127, min(127, A))
            w[c, j] = step
            A -= step
            j += 1
        w[c, K - 2] = r
        assert int(w[c].astype(np.int64) @ x.astype(np.int64)) == phi
    return x, w


def groups(vectors, key):
    out = {}
    for v in vectors:
        out.setdefault(key(v), []).append(v)
    return sorted(out.items())


def run_layer(path, x, w, k, lam, mult, shift, relu, bn, bn_bits):
    """Outputs (one per weight row) of one pixel / one input vector through the named path."""
    N, K = w.shape
    if path == "linear":                      # skinny kernel (K % 16 == 0) or the tiled one
        return linear(x[None], w, None, k, lam, mult, shift, relu, bn, bn_bits)[0]
    if path == "pointwise":                   # a 3-pixel image: the tiled kernel
        img = np.broadcast_to(x, (1, 1, 3, K)).copy()
        got = conv(img, w.reshape(N, 1, 1, K), None, k, lam, mult, shift, (0, 0, 0, 0), (1, 1), relu, bn, bn_bits,
                   fn="pulp_nn_pointwise_HoWo_parallel")
        assert (got[0, 0] == got[0, 0, 0]).all()
        return got[0, 0, 0]
    if path == "stream":                      # 32768 pixels, 16 channels: the weights-stationary streaming kernel
        reps = -(-16 // N)
        w16 = np.tile(w, (reps, 1))[:16]
        k16 = None if k is None else np.tile(np.asarray(k), reps)[:16]
        l16 = None if lam is None else np.tile(np.asarray(lam), reps)[:16]
        img = np.broadcast_to(x, (2, 128, 128, K)).copy()
        got = conv(img, w16.reshape(16, 1, 1, K), None, k16, l16, mult, shift, (0, 0, 0, 0), (1, 1), relu, bn,
                   bn_bits, fn="pulp_nn_pointwise_Ho_parallel")
        flat = got.reshape(-1, 16)
        assert (flat == flat[0]).all()
        return flat[0, :N]
    raise ValueError(path)


PATHS = ["linear", "pointwise", "stream"]


@pytest.mark.parametrize("path", PATHS)
@pytest.mark.parametrize("K", [80, 96])
@pytest.mark.parametrize("bn_bits", [32, 64])
def test_bn_known_answers(bn_bits, K, path):
    for d, vs in groups([v for v in KATS["bn"] if v["bits"] == bn_bits], lambda v: v["d"]):
        x, w = x_and_weights_for([v["phi"] for v in vs], K)
        k, lam = [v["k"] for v in vs], [v["lambda"] for v in vs]
        got = run_layer(path, x, w, k, lam, 0, d, 1, 1, bn_bits)
        want = np.array([v["out"] for v in vs], np.uint8)
        assert_same(got, want, "bn KATs d=%d via %s" % (d, path))


@pytest.mark.parametrize("path", PATHS)
@pytest.mark.parametrize("bn_bits", [32, 64])
def test_quant_known_answers(bn_bits, path):
    for (m, d), vs in groups(KATS["quant"], lambda v: (v["m"], v["d"])):
        x, w = x_and_weights_for([v["phi"] for v in vs], 80)
        got = run_layer(path, x, w, None, None, m, d, 1, 0, bn_bits)
        assert_same(got, np.array([v["out"] for v in vs], np.uint8), "quant KATs m=%d d=%d via %s" % (m, d, path))


@pytest.mark.parametrize("bn_bits", [32, 64])
def test_branch_known_answers(bn_bits):
    """Branch selection by the flags; flag_relu is tested with == 1 by conv / pointwise / linear and for
    truth by depthwise_generic; out_shift 257 reaches the quantiser as int8 1 (uint16 entry points)."""
    for v in KATS["branch"]:
        k, lam = [v["k"]], [v["lambda"]]
        if v["relu_eq1"]:
            x, w = x_and_weights_for([v["acc"]], 80)
            got = run_layer("pointwise", x, w, k, lam, v["mult"], v["shift"], v["relu"], v["bn"], bn_bits)[0]
        else:
            # depthwise 1x1: acc = w * x with w = 1
            assert 0 <= v["acc"] <= 255
            img = np.full((1, 1, 2, 2), v["acc"], np.uint8)
            got = depthwise_generic(img, np.ones((1, 1, 1), np.int8), None, k, lam, v["mult"], v["shift"],
                                    (0, 0, 0, 0), (1, 1), v["relu"], v["bn"], bn_bits)[0, 0, 0, 0]
        assert int(got) == v["out"], (v, int(got))


# ---- random layers with parameters outside the fast forms' preconditions ------------------

def wild_bn(r, n, bn_bits):
    """k, lambda, shift: full-range multipliers (wraps in the 32-bit tree, |k| >= 2^32 in the 64-bit one)."""
    if bn_bits == 32:
        k = r.integers(-2 ** 31, 2 ** 31, n)
        lam = r.integers(-2 ** 31, 2 ** 31, n)
        k[: n // 4] = r.integers(2 ** 23, 2 ** 26, n // 4)        # just past the 24-bit form
        return k, lam, int(r.integers(0, 32))
    k = r.integers(-2 ** 44, 2 ** 44, n)
    lam = r.integers(-2 ** 52, 2 ** 52, n)
    k[: n // 4] = r.integers(2 ** 32, 2 ** 34, n // 4)            # just past the 32-bit form
    return k, lam, int(r.integers(30, 64))


MULT_CASES = [(700, 12), (3, 0), (40000, 9), (65535, 3), (1000, 15), (32768, 10)]


def epi_cases(r, n, bn_bits):
    """(relu, bn, k, lambda, mult, shift) tuples for one layer with n channels."""
    out = []
    for _ in range(2):
        k, lam, sh = wild_bn(r, n, bn_bits)
        out.append((1, 1, k, lam, 0, sh))
    k, lam, _ = wild_bn(r, n, bn_bits)
    out.append((1, 1, k, lam, 0, 0))                               # batch-norm with shift 0
    for m, d in MULT_CASES:
        out.append((1, 0, None, None, m, d))
    out.append((0, 0, None, None, 0, 0))                           # raw branch, shift 0
    return out


CONV_CASES = [
    # B, H, W, Ci, Co, ky, kx, pads, strides
    (2, 12, 12, 64, 72, 3, 3, (1, 1, 1, 1), (1, 1)),     # scalar tap walk (Ci % 64 == 0), K = 576
    (1, 10, 10, 256, 40, 3, 3, (1, 0, 1, 0), (1, 1)),    # K = 2304: accumulators beyond 24 bits
    (2, 9, 9, 48, 24, 3, 3, (1, 1, 1, 1), (1, 1)),       # 16-byte chunks with per-thread taps
    (3, 9, 7, 5, 6, 3, 3, (1, 1, 1, 1), (1, 1)),         # byte gather
    (2, 16, 16, 3, 16, 3, 3, (1, 1, 1, 1), (2, 2)),      # direct small-filter kernel (rows)
    (2, 9, 10, 8, 32, 2, 2, (0, 0, 0, 0), (1, 1)),       # direct small-filter kernel (bytes)
    (2, 16, 16, 32, 64, 3, 3, (1, 1, 1, 1), (1, 1)),     # config 0 geometry
]


@pytest.mark.parametrize("bn_bits", [32, 64])
@pytest.mark.parametrize("geom", CONV_CASES, ids=lambda g: "x".join(map(str, g[:7])))
def test_conv_slow_epilogues(geom, bn_bits):
    B, H, W, Ci, Co, ky, kx, pads, strides = geom
    r = rng_for(11000 + Ci + bn_bits)
    x, w, b = rand_u8(r, (B, H, W, Ci)), rand_s8(r, (Co, ky, kx, Ci)), rand_s8(r, (Co,))
    for relu, bn, k, lam, m, d in epi_cases(r, Co, bn_bits):
        want = oracle.conv(x, w, b, k, lam, m, d, pads, strides, relu, bn, bn_bits)
        got = conv(x, w, b, k, lam, m, d, pads, strides, relu, bn, bn_bits)
        assert_same(got, want, "conv relu=%d bn=%d mult=%d shift=%d" % (relu, bn, m, d))


PW_CASES = [
    # B, H, W, Ci, Co
    (8, 64, 64, 64, 64),      # 32768 pixels: streaming kernel, 8-wave shape
    (2, 128, 129, 128, 256),  # streaming kernel, config 1 channels, ragged pixel count
    (13, 128, 128, 32, 16),   # 212992 pixels: streaming kernel, 16-wave shape
    (2, 20, 20, 128, 256),    # tiled kernel
    (1, 9, 9, 512, 70),       # K = 512: accumulators beyond 24 bits
]


@pytest.mark.parametrize("bn_bits", [32, 64])
@pytest.mark.parametrize("geom", PW_CASES, ids=lambda g: "x".join(map(str, g)))
def test_pointwise_slow_epilogues(geom, bn_bits):
    B, H, W, Ci, Co = geom
    r = rng_for(12000 + Ci + bn_bits)
    x, w, b = rand_u8(r, (B, H, W, Ci)), rand_s8(r, (Co, 1, 1, Ci)), rand_s8(r, (Co,))
    for relu, bn, k, lam, m, d in epi_cases(r, Co, bn_bits):
        want = oracle.pointwise(x, w, b, k, lam, m, d, relu, bn, bn_bits)
        got = conv(x, w, b, k, lam, m, d, (0, 0, 0, 0), (1, 1), relu, bn, bn_bits,
                   fn="pulp_nn_pointwise_HoWo_parallel")
        assert_same(got, want, "pointwise relu=%d bn=%d mult=%d shift=%d" % (relu, bn, m, d))


def test_pointwise_uint16_shift_is_taken_as_int8():
    """out_shift = 257 on a uint16_t entry point is the quantiser's int8_t 1 (pulp_nn_utils.c:35, 148)."""
    r = rng_for(12500)
    x, w = rand_u8(r, (1, 4, 4, 16)), rand_s8(r, (8, 1, 1, 16))
    w[:] = np.sign(w)                                   # small accumulators, so that >> 1 leaves something to see
    k, lam = r.integers(1, 4, 8), r.integers(-50, 50, 8)
    for relu, bn in [(1, 1), (1, 0)]:
        want = oracle.pointwise(x, w, None, k, lam, 1, 1, relu, bn)
        assert want.max() > 0
        got = conv(x, w, None, k, lam, 1, 257, (0, 0, 0, 0), (1, 1), relu, bn, fn="pulp_nn_pointwise_HoWo_parallel")
        assert_same(got, want, "shift 257")
        assert_same(oracle.pointwise(x, w, None, k, lam, 1, 257, relu, bn), want, "oracle shift 257")


@pytest.mark.parametrize("bn_bits", [32, 64])
@pytest.mark.parametrize("dims", [(64, 1024, 96), (7, 80, 33), (300, 64, 64), (5, 100, 70)])
def test_linear_slow_epilogues(dims, bn_bits):
    B, K, N = dims
    r = rng_for(13000 + K + bn_bits)
    x, w, b = rand_u8(r, (B, K)), rand_s8(r, (N, K)), rand_s8(r, (N,))
    for relu, bn, k, lam, m, d in epi_cases(r, N, bn_bits):
        want = oracle.linear(x, w, b, k, lam, m, d, relu, bn, bn_bits)
        assert_same(linear(x, w, b, k, lam, m, d, relu, bn, bn_bits), want,
                    "linear relu=%d bn=%d mult=%d shift=%d" % (relu, bn, m, d))


DW_CASES = [
    # B, CH, H, W, ky, kx, pads, strides
    (2, 128, 56, 56, 3, 3, (1, 1, 1, 1), (1, 1)),    # staged kernel, config 2
    (2, 128, 56, 56, 3, 3, (1, 1, 1, 1), (2, 2)),
    (2, 70, 9, 11, 3, 3, (1, 1, 1, 1), (2, 2)),      # staged kernel without the linear copy
    (3, 64, 8, 8, 3, 3, (1, 1, 1, 1), (1, 1)),       # plane in registers
    (5, 192, 4, 4, 3, 3, (1, 1, 1, 1), (1, 1)),
    (4, 16, 64, 64, 3, 3, (1, 1, 1, 1), (1, 1)),     # rows in registers
    (2, 64, 32, 32, 3, 3, (1, 1, 1, 1), (2, 2)),
    (1, 128, 16, 16, 3, 3, (1, 1, 1, 1), (1, 1)),
    (1, 3, 10, 8, 5, 5, (2, 2, 2, 2), (1, 1)),       # generic kernel
]


@pytest.mark.parametrize("bn_bits", [32, 64])
@pytest.mark.parametrize("geom", DW_CASES, ids=lambda g: "x".join(map(str, g[:6])) + "s%d" % g[7][0])
def test_depthwise_slow_epilogues(geom, bn_bits):
    B, CH, H, W, ky, kx, pads, strides = geom
    r = rng_for(14000 + CH + H + bn_bits)
    x, wt, b = rand_u8(r, (B, CH, H, W)), rand_s8(r, (CH, ky, kx)), rand_s8(r, (CH,))
    hwc_ok = (ky, kx, pads) == (3, 3, (1, 1, 1, 1)) and (H, W) in [(8, 8), (4, 4), (64, 64), (32, 32), (16, 16)]
    for relu, bn, k, lam, m, d in epi_cases(r, CH, bn_bits):
        want = oracle.depthwise_generic(x, wt, b, k, lam, m, d, pads, strides, relu, bn, bn_bits)
        got = depthwise_generic(x, wt, b, k, lam, m, d, pads, strides, relu, bn, bn_bits)
        assert_same(got, want, "depthwise relu=%d bn=%d mult=%d shift=%d" % (relu, bn, m, d))
        if hwc_ok:
            x_hwc = np.ascontiguousarray(x.transpose(0, 2, 3, 1))
            got = depthwise_hwc(x_hwc, wt, b, k, lam, m, d, strides[0], relu, bn, bn_bits)
            assert_same(got, want, "depthwise_hwc relu=%d bn=%d mult=%d shift=%d" % (relu, bn, m, d))


@pytest.mark.parametrize("bn_bits", [32, 64])
def test_depthwise_3x3_s1_slow_epilogues(bn_bits):
    r = rng_for(15000 + bn_bits)
    B, CH, H, W = 2, 66, 12, 20
    x, kern = rand_u8(r, (B, CH, H, W)), rand_s8(r, (CH, 3, 3))
    xpad = np.pad(x, ((0, 0), (0, 0), (1, 1), (0, 0)))
    for relu, bn, k, lam, m, d in epi_cases(r, CH, bn_bits):
        want = oracle.depthwise_3x3_s1(xpad, kern, k, lam, m, d, 1, 1, relu, bn, bn_bits)
        got = depthwise_3x3_s1(xpad, kern, k, lam, m, d, relu, bn, bn_bits)
        assert_same(got, want, "depthwise_3x3_s1 relu=%d bn=%d mult=%d shift=%d" % (relu, bn, m, d))


# ---- pulp_nn_matmul: both widths, every flag pair, several geometries ---------------------

@pytest.mark.parametrize("bn_bits", [32, 64])
@pytest.mark.parametrize("dims", [(27, 7), (288, 64), (128, 256), (2304, 40), (5, 3)])
def test_matmul_flags_and_widths(dims, bn_bits):
    import torch
    from gpu_helpers import bn_dev, dev
    K, Co = dims
    r = rng_for(16000 + K + bn_bits)
    w, cols, b = rand_s8(r, (Co, K)), rand_u8(r, (2, K)), rand_s8(r, (Co,))
    if bn_bits == 32:
        k, lam, bshift = r.integers(256, 1025, Co), r.integers(-2 ** 16, 2 ** 16, Co), 12
    else:
        k, lam, bshift = r.integers(2 ** 20, 2 ** 24, Co), r.integers(-2 ** 36, 2 ** 36, Co), 30
    L = nn(bn_bits)
    for relu, bn in [(1, 1), (1, 0), (0, 0), (0, 1), (2, 0)]:
        shift = bshift if (relu and bn) else (14 if relu == 1 else 6)
        for bias in (b, None):
            w0, w1 = oracle.matmul(w, cols, bias, k, lam, 300, shift, relu, bn, bn_bits)
            out = torch.full((2 * Co + 5,), 0xA5, dtype=torch.uint8, device="cuda")
            ret = L.pulp_nn_matmul(dev(w), dev(cols), Co, K, shift, 300, bn_dev(k, bn_bits), bn_dev(lam, bn_bits),
                                   dev(bias), out, out.data_ptr() + Co, relu, bn)
            L.sync()
            assert ret == out.data_ptr() + 2 * Co
            o = out.cpu().numpy()
            assert_same(o[:Co], w0, "matmul col 0 %s" % ((relu, bn),))
            assert_same(o[Co:2 * Co], w1, "matmul col 1 %s" % ((relu, bn),))
            assert (o[2 * Co:] == 0xA5).all()
