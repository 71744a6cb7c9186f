"""GPU parity: every entry point of the C ABI against the CPU oracle, bit-exact.

All comparisons are integer / byte work, so the bar is equality of every element."""
import numpy as np
import pytest

import oracle
from gpu_helpers import (add, assert_same, avgpool, conv, depthwise_3x3_s1, depthwise_generic, depthwise_hwc, linear,
                         linear_out_32, maxpool, nn, rand_s8, rand_u8, rng_for)
from pulp_nn_amd import PulpNNError

pytestmark = pytest.mark.gpu

CONV_GEOMS = [
    # B, H, W, Ci, Co, ky, kx, pads(t,b,l,r), strides(sx,sy)
    (2, 16, 16, 32, 64, 3, 3, (1, 1, 1, 1), (1, 1)),    # config 0 geometry
    (3, 9, 7, 5, 6, 3, 3, (1, 1, 1, 1), (1, 1)),        # Ci, Co not multiples of anything
    (2, 11, 13, 3, 7, 3, 3, (1, 0, 1, 0), (1, 1)),      # asymmetric padding
    (2, 12, 12, 8, 10, 3, 3, (1, 1, 1, 1), (2, 2)),     # stride 2
    (1, 10, 9, 6, 5, 5, 3, (2, 2, 1, 1), (1, 1)),       # ky != kx
    (2, 16, 16, 3, 16, 3, 3, (1, 1, 1, 1), (2, 2)),     # MobileNet stem style
    (1, 12, 10, 16, 130, 3, 3, (1, 1, 1, 1), (1, 1)),   # Co tail across two 128-wide tiles
    (2, 9, 9, 48, 24, 3, 3, (1, 1, 1, 1), (1, 1)),      # Ci multiple of 16 but K slices straddle taps
    (1, 7, 9, 64, 40, 1, 1, (0, 0, 0, 0), (1, 1)),      # 1x1 through the standard conv entry point
    (1, 20, 20, 256, 32, 3, 3, (1, 0, 1, 0), (1, 1)),   # config 4 style channels, K = 2304
    (3, 33, 31, 3, 16, 3, 3, (1, 1, 1, 1), (2, 2)),     # 27-byte filters, several workgroups with a ragged tail
    (2, 9, 10, 8, 32, 2, 2, (0, 0, 0, 0), (1, 1)),      # filter of exactly 32 bytes, 32 channels
    (2, 8, 9, 2, 24, 3, 3, (1, 1, 1, 1), (1, 1)),       # 18-byte filters, 24 channels (byte stores)
    (1, 6, 5, 2, 5, 1, 2, (0, 0, 0, 0), (1, 1)),        # 4-byte filters, 5 channels
    (2, 8, 8, 4, 40, 3, 3, (1, 1, 1, 1), (1, 1)),       # 36-byte filters: just past the direct kernel
    (2, 8, 9, 4, 20, 3, 3, (1, 1, 1, 1), (1, 1)),       # 12-byte filter rows (RGBA stem), row-gather kernel
    (2, 9, 11, 1, 8, 3, 3, (1, 1, 1, 1), (2, 1)),       # 3-byte filter rows, every alignment of a row start
    (1, 7, 8, 3, 12, 2, 3, (0, 1, 2, 0), (1, 1)),       # two filter rows, two columns of left padding
]
FLAGS = [(1, 1), (1, 0), (0, 0), (0, 1), (2, 0)]


def bn_params(r, n, bn_bits):
    if bn_bits == 32:
        return r.integers(256, 1025, n), r.integers(-2 ** 16, 2 ** 16 + 1, n), 20
    return r.integers(2 ** 20, 2 ** 24 + 1, n), r.integers(-2 ** 36, 2 ** 36 + 1, n), 38


def pick_shift(relu, bn, bn_shift, K):
    if relu and bn:
        return bn_shift
    lg = int(np.log2(max(K, 2) ** 0.5 * 128 * 74))      # typical |acc|
    return (lg + 10 - 7) if relu == 1 else max(lg - 7, 0)


@pytest.mark.parametrize("bn_bits", [32, 64])
@pytest.mark.parametrize("flags", FLAGS)
@pytest.mark.parametrize("geom", CONV_GEOMS, ids=lambda g: "x".join(map(str, g[:7])))
def test_conv(geom, flags, bn_bits):
    B, H, W, Ci, Co, ky, kx, pads, strides = geom
    relu, bn = flags
    r = rng_for(1000 + 17 * relu + bn + bn_bits)
    x, w, b = rand_u8(r, (B, H, W, Ci)), rand_s8(r, (Co, ky, kx, Ci)), rand_s8(r, (Co,))
    k, lam, bshift = bn_params(r, Co, bn_bits)
    mult = int(r.integers(256, 1025))
    shift = pick_shift(relu, bn, bshift, ky * kx * Ci)
    want = oracle.conv(x, w, b, k, lam, mult, shift, pads, strides, relu, bn, bn_bits)
    got = conv(x, w, b, k, lam, mult, shift, pads, strides, relu, bn, bn_bits)
    assert_same(got, want, "conv")
    if ky * kx * Ci >= 16:     # the fixed batch-norm constants are scaled for accumulators of real layers
        assert want.max() > 0 and (want < 255).any(), "degenerate case"


def test_conv_variants_and_null_bias():
    B, H, W, Ci, Co = 2, 10, 12, 32, 20
    r = rng_for(7)
    x, w = rand_u8(r, (B, H, W, Ci)), rand_s8(r, (Co, 3, 3, Ci))
    k, lam = r.integers(256, 1025, Co), r.integers(-2 ** 16, 2 ** 16, Co)
    want = oracle.conv(x, w, None, k, lam, 0, 20, (1, 1, 1, 1), (1, 1), 1, 1)
    for fn in ("pulp_nn_conv_Ho_parallel", "pulp_nn_conv_HoWo_parallel", "pulp_nn_conv_Co_parallel"):
        assert_same(conv(x, w, None, k, lam, 0, 20, (1, 1, 1, 1), (1, 1), 1, 1, fn=fn), want, fn)


PW_GEOMS = [
    # B, H, W, Ci, Co
    (4, 28, 28, 128, 256),   # config 1 geometry, small batch
    (3, 7, 5, 24, 13),
    (2, 8, 8, 16, 32),
    (2, 4, 4, 512, 512),
    (1, 9, 11, 3, 100),
    (5, 3, 3, 70, 64),
    # a few thousand pixels with K, N <= 256: tiled kernel, every tile shape
    (4, 32, 32, 16, 32),     # 16 -> 32 channels (MobileNet block 1), K < 64
    (3, 30, 30, 32, 16),     # N = 16
    (2, 40, 40, 64, 64),
    (2, 33, 35, 64, 128),    # pixel count not a multiple of 64
    # shapes that take the weights-stationary streaming kernel (>= 32768 pixels, K, N <= 256)
    (16, 112, 112, 32, 64),  # 200704 pixels: the 16-wave shape of the streaming kernel, one channel group
    (16, 112, 113, 16, 32),  # ... 32 channels, pixel count not a multiple of 16 per wave
    (8, 64, 64, 64, 128),    # two channel groups
    (8, 64, 65, 128, 256),   # config 1 channels, pixel count not a multiple of 64
    (9, 64, 64, 192, 192),   # K = 192: four K slices, three channel groups
    (8, 64, 66, 256, 16),    # K = 256, N = 16
    (16, 65, 64, 64, 300),   # 66560 pixels x 300 channels: the 256 x 256 tiles of the tiled kernel, channel tail
    (2, 33, 33, 256, 200),   # K = 256, channel tail inside the last group
    (2, 40, 30, 48, 100),    # K and N not multiples of 64
    (3, 33, 33, 192, 256),   # K = 192
    (1, 50, 50, 128, 20),    # N not a multiple of 16
]


@pytest.mark.parametrize("bn_bits", [32, 64])
@pytest.mark.parametrize("flags", FLAGS)
@pytest.mark.parametrize("geom", PW_GEOMS, ids=lambda g: "x".join(map(str, g)))
def test_pointwise(geom, flags, bn_bits):
    B, H, W, Ci, Co = geom
    relu, bn = flags
    r = rng_for(2000 + 17 * relu + bn + bn_bits)
    x, w, b = rand_u8(r, (B, H, W, Ci)), rand_s8(r, (Co, 1, 1, Ci)), rand_s8(r, (Co,))
    k, lam, bshift = bn_params(r, Co, bn_bits)
    mult = int(r.integers(256, 1025))
    shift = pick_shift(relu, bn, bshift, Ci)
    want = oracle.pointwise(x, w, b, k, lam, mult, shift, relu, bn, bn_bits)
    for fn in ("pulp_nn_pointwise_HoWo_parallel", "pulp_nn_pointwise_Ho_parallel", "pulp_nn_pointwise_Co_parallel"):
        # stride / padding / kernel arguments are deliberately nonsense: the reference ignores them
        got = conv(x, w, b, k, lam, mult, shift, (3, 3, 3, 3), (2, 2), relu, bn, bn_bits, out_hw=(H, W), fn=fn)
        assert_same(got, want, fn)


def test_pointwise_output_smaller_than_input():
    r = rng_for(3)
    x, w = rand_u8(r, (2, 6, 8, 16)), rand_s8(r, (3, 1, 1, 16))
    want = oracle.pointwise(x, w, None, None, None, 0, 6, 0, 0, out_hw=(4, 5))
    got = conv(x, w, None, None, None, 0, 6, (0, 0, 0, 0), (1, 1), 0, 0, out_hw=(4, 5),
               fn="pulp_nn_pointwise_HoWo_parallel")
    assert_same(got, want, "pointwise crop")


DW_GEOMS = [
    # B, CH, H, W, ky, kx, pads, strides
    (2, 128, 56, 56, 3, 3, (1, 1, 1, 1), (2, 2)),    # config 2 stride 2
    (2, 8, 12, 12, 3, 3, (1, 1, 1, 1), (1, 1)),
    (2, 70, 9, 11, 3, 3, (1, 1, 1, 1), (2, 2)),      # odd sizes, channel tail
    (1, 16, 64, 64, 3, 3, (1, 1, 1, 1), (1, 1)),     # MobileNet block 1
    (1, 3, 10, 8, 5, 5, (2, 2, 2, 2), (1, 1)),
    (2, 4, 7, 9, 3, 5, (1, 1, 2, 2), (1, 1)),
    (1, 6, 8, 8, 1, 1, (0, 0, 0, 0), (1, 1)),
    (1, 2, 6, 6, 2, 2, (0, 0, 0, 0), (2, 2)),
    (1, 5, 9, 9, 3, 3, (0, 0, 0, 0), (1, 1)),        # no padding: pl = 0 fast path
    (1, 5, 11, 11, 3, 3, (0, 0, 0, 0), (2, 2)),
    (1, 4, 10, 230, 3, 3, (1, 1, 1, 1), (1, 1)),     # wide image: few rows per band
    (8, 16, 16, 16, 3, 3, (1, 1, 1, 1), (1, 1)),     # 16 channels: four images share a workgroup
    (3, 16, 20, 16, 3, 3, (1, 1, 1, 1), (2, 2)),     # ... with a partly filled last group of images
    (5, 32, 12, 24, 3, 3, (1, 1, 1, 1), (2, 2)),     # 32 channels: two images per workgroup, odd batch
    (9, 8, 18, 20, 3, 3, (0, 0, 0, 0), (1, 1)),      # 8 channels: eight images per workgroup, no padding
    (3, 64, 8, 8, 3, 3, (1, 1, 1, 1), (1, 1)),       # 8x8 planes: one plane per lane, in registers
    (2, 128, 8, 8, 3, 3, (1, 1, 1, 1), (2, 2)),      # ... stride 2
    (2, 64, 8, 8, 3, 3, (1, 0, 1, 0), (2, 2)),       # ... stride 2 without bottom / right padding (same output size)
    (5, 192, 4, 4, 3, 3, (1, 1, 1, 1), (1, 1)),      # 4x4 planes
    (4, 16, 64, 64, 3, 3, (1, 1, 1, 1), (1, 1)),     # 64-byte rows, a few rows per lane in registers; 16 channels
    (2, 32, 64, 64, 3, 3, (1, 1, 1, 1), (2, 2)),     # ... stride 2, 32 channels
    (1, 64, 32, 32, 3, 3, (1, 1, 1, 1), (1, 1)),     # 32-byte rows
    (2, 64, 32, 32, 3, 3, (1, 1, 1, 1), (2, 2)),
    (1, 128, 16, 16, 3, 3, (1, 1, 1, 1), (1, 1)),    # 16-byte rows
    (1, 128, 16, 16, 3, 3, (1, 1, 1, 1), (2, 2)),
    (1, 64, 11, 16, 3, 3, (1, 1, 1, 1), (1, 1)),     # ... height not a multiple of the rows per lane
    (2, 32, 9, 32, 3, 3, (1, 1, 1, 1), (2, 2)),      # ... stride 2, odd height
    (1, 64, 12, 16, 3, 3, (1, 0, 1, 1), (1, 1)),     # ... no bottom padding: one output row fewer
    # 512 or more (image, 64 channels) units: whole planes streamed through LDS in chunks of 8 rows (at stride 1
    # only planes of whole chunks)
    (64, 512, 16, 12, 3, 3, (1, 1, 1, 1), (1, 1)),   # two chunks
    (16, 2048, 24, 8, 3, 3, (1, 1, 1, 1), (1, 1)),   # three chunks, two groups of columns (both at an edge)
    (16, 2048, 9, 24, 3, 3, (1, 1, 1, 1), (2, 2)),   # stride 2, odd height: the second chunk is one row
    (64, 512, 8, 12, 3, 3, (0, 1, 0, 2), (1, 1)),    # no top / left padding, two columns of right padding
    (32, 1024, 13, 24, 3, 3, (0, 0, 0, 1), (2, 2)),  # stride 2 without top / left padding
    (64, 512, 16, 12, 3, 3, (2, 0, 1, 1), (1, 1)),   # two rows of top padding, none at the bottom
    (8, 4096, 16, 16, 3, 3, (1, 1, 0, 2), (1, 1)),   # 16-byte rows that the register kernel does not take (pl = 0)
    (64, 512, 12, 12, 3, 3, (1, 1, 1, 1), (1, 1)),   # stride 1, 12 rows: not whole chunks, the band kernel
]


@pytest.mark.parametrize("bn_bits", [32, 64])
@pytest.mark.parametrize("flags", [(1, 1), (1, 0), (0, 0), (2, 0)])
@pytest.mark.parametrize("geom", DW_GEOMS, ids=lambda g: "x".join(map(str, g[:6])) + "s%d" % g[7][0])
def test_depthwise_generic(geom, flags, bn_bits):
    B, CH, H, W, ky, kx, pads, strides = geom
    relu, bn = flags
    r = rng_for(3000 + 17 * relu + bn + bn_bits)
    x, wt, b = rand_u8(r, (B, CH, H, W)), rand_s8(r, (CH, ky, kx)), rand_s8(r, (CH,))
    if bn_bits == 32:
        k, lam, bshift = r.integers(2 ** 12, 2 ** 14 + 1, CH), r.integers(-2 ** 16, 2 ** 16 + 1, CH), 16
    else:
        k, lam, bshift = r.integers(2 ** 20, 2 ** 24 + 1, CH), r.integers(-2 ** 36, 2 ** 36 + 1, CH), 28
    shift = bshift if (relu and bn) else (14 if relu else 6)
    want = oracle.depthwise_generic(x, wt, b, k, lam, 900, shift, pads, strides, relu, bn, bn_bits)
    for fn in ("pulp_nn_depthwise_generic", "pulp_nn_depthwise_generic_less_4_weights"):
        got = depthwise_generic(x, wt, b, k, lam, 900, shift, pads, strides, relu, bn, bn_bits, fn=fn)
        assert_same(got, want, fn)


@pytest.mark.parametrize("bn_bits", [32, 64])
@pytest.mark.parametrize("flags", [(1, 1), (1, 0), (0, 0)])
@pytest.mark.parametrize("shape", [(2, 128, 56, 56), (2, 5, 7, 6), (1, 3, 1, 2), (3, 66, 12, 20), (6, 16, 12, 16),
                                   (3, 32, 9, 20)])
def test_depthwise_3x3_s1(shape, flags, bn_bits):
    B, CH, H, W = shape
    relu, bn = flags
    r = rng_for(4000 + relu + bn)
    x, kern = rand_u8(r, (B, CH, H, W)), rand_s8(r, (CH, 3, 3))
    kern[0] = 127       # same-sign taps drive the 32-bit batch-norm product past 2^31
    k, lam = r.integers(2 ** 12, 2 ** 14 + 1, CH), r.integers(-2 ** 16, 2 ** 16 + 1, CH)
    k[0] = 2 ** 14
    shift = 16 if (relu and bn) else (13 if relu else 5)
    xpad = np.pad(x, ((0, 0), (0, 0), (1, 1), (0, 0)))
    want = oracle.depthwise_3x3_s1(xpad, kern, k, lam, 600, shift, 1, 1, relu, bn, bn_bits)
    got = depthwise_3x3_s1(xpad, kern, k, lam, 600, shift, relu, bn, bn_bits)
    assert_same(got, want, "depthwise_3x3_s1")


DW_HWC_GEOMS = [
    # B, CH, H, W, stride: every kernel shape behind pulp_nn_hip_depthwise_hwc
    (3, 64, 8, 8, 1), (2, 128, 8, 8, 2), (5, 192, 4, 4, 1),
    (4, 16, 64, 64, 1), (2, 32, 64, 64, 2), (1, 64, 32, 32, 1), (2, 64, 32, 32, 2),
    (1, 128, 16, 16, 1), (1, 128, 16, 16, 2), (1, 64, 11, 16, 1), (2, 32, 9, 32, 2), (16, 4, 7, 16, 1),
]


@pytest.mark.parametrize("bn_bits", [32, 64])
@pytest.mark.parametrize("flags", FLAGS)
@pytest.mark.parametrize("geom", DW_HWC_GEOMS, ids=lambda g: "x".join(map(str, g[:4])) + "s%d" % g[4])
def test_depthwise_hwc(geom, flags, bn_bits):
    """The fused layout change + depthwise against the oracle's CHW depthwise on the transposed input."""
    B, CH, H, W, stride = geom
    relu, bn = flags
    r = rng_for(3500 + 17 * relu + bn + bn_bits)
    x_hwc, wt, b = rand_u8(r, (B, H, W, CH)), rand_s8(r, (CH, 3, 3)), rand_s8(r, (CH,))
    if bn_bits == 32:
        k, lam, bshift = r.integers(2 ** 12, 2 ** 14 + 1, CH), r.integers(-2 ** 16, 2 ** 16 + 1, CH), 16
    else:
        k, lam, bshift = r.integers(2 ** 20, 2 ** 24 + 1, CH), r.integers(-2 ** 36, 2 ** 36 + 1, CH), 28
    shift = bshift if (relu and bn) else (14 if relu else 6)
    x_chw = np.ascontiguousarray(x_hwc.transpose(0, 3, 1, 2))
    want = oracle.depthwise_generic(x_chw, wt, b, k, lam, 900, shift, (1, 1, 1, 1), (stride, stride), relu, bn, bn_bits)
    got = depthwise_hwc(x_hwc, wt, b, k, lam, 900, shift, stride, relu, bn, bn_bits)
    assert_same(got, want, "pulp_nn_hip_depthwise_hwc")


def test_depthwise_hwc_unsupported_geometry_is_rejected():
    r = rng_for(3600)
    x_hwc, wt, b = rand_u8(r, (1, 9, 9, 5)), rand_s8(r, (5, 3, 3)), rand_s8(r, (5,))
    k, lam = r.integers(2 ** 12, 2 ** 14 + 1, 5), r.integers(-2 ** 16, 2 ** 16 + 1, 5)
    with pytest.raises(PulpNNError) as ei:
        depthwise_hwc(x_hwc, wt, b, k, lam, 900, 16, 1, 1, 1, 32)
    assert ei.value.code == 2


@pytest.mark.parametrize("bn_bits", [32, 64])
@pytest.mark.parametrize("dims", [(64, 1024, 4096), (256, 512, 1000), (3, 37, 11), (1, 512, 1000), (5, 100, 70),
                                  (70, 48, 30), (130, 256, 132), (300, 64, 64)])
def test_linear(dims, bn_bits):
    B, K, N = dims
    r = rng_for(5000 + K)
    x, w, b = rand_u8(r, (B, K)), rand_s8(r, (N, K)), rand_s8(r, (N,))
    k, lam, bshift = bn_params(r, N, bn_bits)
    for relu, bn in FLAGS:
        shift = pick_shift(relu, bn, bshift, K)
        want = oracle.linear(x, w, b, k, lam, 800, shift, relu, bn, bn_bits)
        assert_same(linear(x, w, b, k, lam, 800, shift, relu, bn, bn_bits), want, "linear %d %d" % (relu, bn))


@pytest.mark.parametrize("dims", [(256, 512, 1000), (3, 37, 11), (2, 1024, 64), (100, 80, 20)])
def test_linear_out_32(dims):
    B, K, N = dims
    r = rng_for(6000 + K)
    x, w = rand_u8(r, (B, K)), rand_s8(r, (N, K))
    b32 = r.integers(-2 ** 31, 2 ** 31, N, dtype=np.int64).astype(np.int32)
    assert_same(linear_out_32(x, w, b32), oracle.linear_out_32(x, w, b32), "linear_out_32")
    assert_same(linear_out_32(x, w, None, 64), oracle.linear_out_32(x, w, None), "linear_out_32 no bias")


def test_matmul_two_columns():
    import torch
    from gpu_helpers import bn_dev, dev
    r = rng_for(8)
    K, Co = 27, 7
    w, cols, b = rand_s8(r, (Co, K)), rand_u8(r, (2, K)), rand_s8(r, (Co,))
    k, lam = r.integers(256, 1025, Co), r.integers(-2 ** 16, 2 ** 16, Co)
    w0, w1 = oracle.matmul(w, cols, b, k, lam, 0, 12, 1, 1)
    L = nn(32)
    out = torch.zeros(2 * Co + 5, dtype=torch.uint8, device="cuda")
    ret = L.pulp_nn_matmul(dev(w), dev(cols), Co, K, 12, 0, bn_dev(k, 32), bn_dev(lam, 32), dev(b), out,
                           out.data_ptr() + Co, 1, 1)
    L.sync()
    assert ret == out.data_ptr() + 2 * Co
    o = out.cpu().numpy()
    assert_same(o[:Co], w0, "matmul col 0")
    assert_same(o[Co:2 * Co], w1, "matmul col 1")
    # separate destinations
    o2 = torch.zeros(64, dtype=torch.uint8, device="cuda")
    L.pulp_nn_matmul(dev(w), dev(cols), Co, K, 12, 0, bn_dev(k, 32), bn_dev(lam, 32), dev(b), o2,
                     o2.data_ptr() + 32, 1, 1)
    L.sync()
    o2 = o2.cpu().numpy()
    assert_same(o2[:Co], w0, "matmul col 0 (split)")
    assert_same(o2[32:32 + Co], w1, "matmul col 1 (split)")


@pytest.mark.parametrize("case", [
    (2, 63, 63, 256, (2, 2), (2, 2), (32, 32)),    # config 4: ceil mode
    (2, 63, 63, 16, (2, 2), (2, 2), (31, 31)),
    (1, 8, 8, 5, (2, 2), (2, 2), (4, 4)),
    (2, 9, 7, 3, (3, 2), (2, 1), (8, 3)),
    (1, 6, 6, 4, (3, 3), (3, 3), (2, 2)),
])
def test_maxpool(case):
    B, H, W, Cc, kernel, strides, out_hw = case
    r = rng_for(7000 + H)
    x = rand_u8(r, (B, H, W, Cc))
    got, xin_after = maxpool(x, kernel, strides, out_hw)
    assert_same(got, oracle.maxpool(x, kernel, strides, out_hw=out_hw), "maxpool")
    assert_same(xin_after, x, "maxpool input must stay intact")


@pytest.mark.parametrize("bn_bits", [32, 64])
def test_avgpool(bn_bits):
    r = rng_for(8000)
    x = rand_u8(r, (3, 4, 4, 512))
    assert_same(avgpool(x, (4, 4), (4, 4), (1, 1), bn_bits=bn_bits),
                oracle.avgpool(x, (4, 4), (4, 4), bn_bits=bn_bits), "global avgpool")
    x2 = rand_u8(r, (2, 9, 7, 6))
    for pads, kernel, strides, out_hw in [((0, 0, 0, 0), (2, 2), (2, 2), (4, 3)), ((1, 1, 1, 1), (3, 3), (1, 1), (9, 7)),
                                          ((1, 0, 0, 1), (3, 2), (2, 1), (8, 3))]:
        for rq, lam, sh, ad in [(0, 0, 0, 0), (1, 3, 2, 20), (1, -1, 22 if bn_bits == 32 else 2, 500)]:
            want = oracle.avgpool(x2, kernel, strides, pads, out_hw, lam, sh, ad, rq, bn_bits)
            got = avgpool(x2, kernel, strides, out_hw, pads, lam, sh, ad, rq, bn_bits)
            assert_same(got, want, "avgpool %s %s" % (pads, (rq, lam)))
    # windows wider than one batch of loads, channel tail
    x3 = rand_u8(r, (2, 7, 7, 22))
    for pads, kernel, strides, out_hw in [((0, 0, 0, 0), (7, 7), (7, 7), (1, 1)), ((2, 2, 2, 2), (5, 5), (1, 1), (7, 7)),
                                          ((0, 0, 0, 0), (6, 5), (1, 2), (2, 2))]:
        want = oracle.avgpool(x3, kernel, strides, pads, out_hw, 0, 0, 0, 0, bn_bits)
        got = avgpool(x3, kernel, strides, out_hw, pads, 0, 0, 0, 0, bn_bits)
        assert_same(got, want, "avgpool %s %s" % (pads, kernel))


def test_add():
    r = rng_for(9000)
    for shape in [(3, 5, 7, 4), (2, 16, 16, 64), (1, 3, 3, 5)]:
        a, b = rand_u8(r, shape), rand_u8(r, shape)
        for m1, m2, d in [(3, 5, 2), (120, 130, 8), (65535, 2, 0), (32767, 32767, 9)]:
            assert_same(add(a, b, m1, m2, d), oracle.add(a, b, m1, m2, d), "add %s" % ((m1, m2, d),))


def test_hwc_to_chw():
    import torch
    from gpu_helpers import dev
    r = rng_for(9100)
    for B, H, W, Cc, pt, pb in [(2, 7, 9, 5, 1, 1), (1, 16, 16, 64, 0, 0), (3, 5, 4, 130, 1, 0)]:
        x = rand_u8(r, (B, H, W, Cc))
        L = nn(32)
        out = torch.full((B, Cc, H + pt + pb, W), 0xA5, dtype=torch.uint8, device="cuda")
        L.set_batch(B)
        L.hwc_to_chw(dev(x), out, W, H, Cc, pt, pb)
        L.sync()
        L.set_batch(1)
        want = np.pad(x.transpose(0, 3, 1, 2), ((0, 0), (0, 0), (pt, pb), (0, 0)))
        assert_same(out.cpu().numpy(), want, "hwc_to_chw")


def test_rejected_calls_report_an_error_and_write_nothing():
    import torch
    from pulp_nn_amd import PulpNNError
    L = nn(32)
    x = torch.zeros(64, dtype=torch.uint8, device="cuda")
    out = torch.full((64,), 0xA5, dtype=torch.uint8, device="cuda")
    w = torch.zeros(64, dtype=torch.int8, device="cuda")
    with pytest.raises(PulpNNError):   # shift 40 is undefined behaviour for a 32-bit accumulator
        L.pulp_nn_pointwise_HoWo_parallel(x, None, None, out, w, None, None, 1, 40, 2, 2, 4, 2, 2, 4, 1, 1,
                                          0, 0, 0, 0, 1, 1, 0, 0)
    with pytest.raises(PulpNNError):   # batch-norm branch without k / lambda
        L.pulp_nn_linear(x, None, out, w, None, None, 1, 3, 8, 4, 1, 1)
    with pytest.raises(PulpNNError):   # p_l = 0: the reference's row pointers drift
        L.pulp_nn_depthwise_3x3_s1(x, out, 4, 4, 1, 0, 1, w, 3, 1, None, None, 0, 0, None)
    L.sync()
    assert int(out.min()) == 0xA5
    assert L.last_error() == 0


@pytest.mark.parametrize("bn_bits", [32, 64])
def test_clock_probe_reads_a_plausible_shader_clock(bn_bits):
    """pulp_nn_hip_clock_probe: 20 us of the 100 MHz wall clock and a shader clock between 0.3 and 3 GHz; a null
    pointer is rejected."""
    import torch
    from pulp_nn_amd import PulpNNError
    L = nn(bn_bits)
    out = torch.zeros(2, dtype=torch.int64, device="cuda")
    L.clock_probe(out)
    L.sync()
    ticks, cycles = (int(v) for v in out.cpu())
    assert 2000 <= ticks < 20000, ticks
    assert 300 <= 100.0 * cycles / ticks <= 3000, (ticks, cycles)
    with pytest.raises(PulpNNError):
        L.clock_probe(None)
