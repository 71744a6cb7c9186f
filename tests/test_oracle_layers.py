"""Pins the oracle's layer functions against independent closed forms and
cross-function invariants:
  * contractions: numpy sliding-window einsum on explicitly zero-padded int64
    arrays, and scipy.signal.correlate2d (a library routine) per channel pair;
  * GEMV: numpy matmul;  pooling: numpy windowed max / sum;
  * invariants: pointwise == 1x1 conv, linear == pointwise on a 1x1 image,
    depthwise_3x3_s1 == depthwise_generic on a row-padded plane, matmul ==
    two pixels of conv, batch == per-image calls.
"""
import numpy as np
import pytest
from scipy.signal import correlate2d

import npref
import oracle


def rng_for(seed):
    return np.random.Generator(np.random.PCG64(seed))


def rand_u8(r, shape):
    return r.integers(0, 256, size=shape, dtype=np.uint8)


def rand_s8(r, shape):
    return r.integers(-128, 128, size=shape, dtype=np.int8)


CONV_GEOMS = [
    # H, W, Ci, Co, ky, kx, pads(t,b,l,r), strides(sx,sy)
    (16, 16, 32, 64, 3, 3, (1, 1, 1, 1), (1, 1)),   # BASELINE config 0
    (9, 7, 5, 6, 3, 3, (1, 1, 1, 1), (1, 1)),       # odd sizes, odd pixel count
    (11, 13, 3, 7, 3, 3, (1, 0, 1, 0), (1, 1)),     # asymmetric padding (config 4 style)
    (12, 12, 8, 10, 3, 3, (1, 1, 1, 1), (2, 2)),    # stride 2
    (10, 9, 6, 5, 5, 3, (2, 2, 1, 1), (1, 1)),      # ky != kx
    (8, 10, 4, 3, 3, 3, (0, 0, 0, 0), (1, 2)),      # no padding, sx != sy
    (7, 7, 3, 16, 3, 3, (1, 1, 1, 1), (2, 2)),      # stem-like, Ci = 3
]


@pytest.mark.parametrize("geom", CONV_GEOMS, ids=lambda g: "x".join(map(str, g[:6])))
def test_conv_acc_matches_numpy_cross_correlation(geom):
    H, W, Ci, Co, ky, kx, pads, strides = geom
    r = rng_for(hash(geom) & 0xFFFF)
    x, w, b = rand_u8(r, (H, W, Ci)), rand_s8(r, (Co, ky, kx, Ci)), rand_s8(r, (Co,))
    np.testing.assert_array_equal(oracle.conv_acc(x, w, b, pads, strides), npref.conv_acc(x, w, b, pads, strides))
    np.testing.assert_array_equal(oracle.conv_acc(x, w, None, pads, strides),
                                  npref.conv_acc(x, w, None, pads, strides))


def test_conv_acc_matches_scipy_correlate2d():
    """Library routine: 'same' cross-correlation per (co, ci) pair, summed over ci."""
    r = rng_for(5)
    H, W, Ci, Co = 9, 8, 3, 4
    x, w = rand_u8(r, (H, W, Ci)), rand_s8(r, (Co, 3, 3, Ci))
    want = np.zeros((H, W, Co), np.int64)
    for co in range(Co):
        for ci in range(Ci):
            want[:, :, co] += correlate2d(x[:, :, ci].astype(np.int64), w[co, :, :, ci].astype(np.int64),
                                          mode="same", boundary="fill", fillvalue=0)
    np.testing.assert_array_equal(oracle.conv_acc(x, w, None, (1, 1, 1, 1), (1, 1)), want)


def test_conv_is_not_transposed_or_flipped():
    """A single non-zero weight tap picks exactly the expected shifted input."""
    r = rng_for(6)
    x = rand_u8(r, (6, 5, 2))
    for fy in range(3):
        for fx in range(3):
            w = np.zeros((1, 3, 3, 2), np.int8)
            w[0, fy, fx, 1] = 1
            acc = oracle.conv_acc(x, w, None, (1, 1, 1, 1), (1, 1))[:, :, 0]
            want = np.pad(x[:, :, 1].astype(np.int64), 1)[fy:fy + 6, fx:fx + 5]
            np.testing.assert_array_equal(acc, want)


FLAGS = [(1, 1), (1, 0), (0, 0), (0, 1), (2, 0)]


@pytest.mark.parametrize("bn_bits", [32, 64])
@pytest.mark.parametrize("flags", FLAGS)
@pytest.mark.parametrize("geom", CONV_GEOMS[:5], ids=lambda g: "x".join(map(str, g[:6])))
def test_conv_full(geom, flags, bn_bits):
    H, W, Ci, Co, ky, kx, pads, strides = geom
    relu, bn = flags
    r = rng_for(100 + bn_bits + 7 * relu + bn)
    x, w, b = rand_u8(r, (H, W, Ci)), rand_s8(r, (Co, ky, kx, Ci)), rand_s8(r, (Co,))
    if bn_bits == 32:
        k, lam, shift = r.integers(256, 1025, Co), r.integers(-2 ** 16, 2 ** 16 + 1, Co), 20
    else:
        k, lam, shift = r.integers(2 ** 20, 2 ** 24 + 1, Co), r.integers(-2 ** 36, 2 ** 36 + 1, Co), 38
    mult = int(r.integers(256, 1025))
    if not (relu and bn):
        shift = 18 if relu == 1 else 9
    got = oracle.conv(x, w, b, k, lam, mult, shift, pads, strides, relu, bn, bn_bits)
    want = npref.epilogue(npref.conv_acc(x, w, b, pads, strides), k, lam, mult, shift, relu, bn, bn_bits)
    np.testing.assert_array_equal(got, want)
    assert got.max() > 0, "degenerate test: all outputs zero"


def test_conv_batch_equals_per_image():
    r = rng_for(7)
    x, w, b = rand_u8(r, (3, 9, 7, 5)), rand_s8(r, (6, 3, 3, 5)), rand_s8(r, (6,))
    k, lam = r.integers(256, 1025, 6), r.integers(-2 ** 16, 2 ** 16, 6)
    full = oracle.conv(x, w, b, k, lam, 0, 14, (1, 1, 1, 1), (1, 1), 1, 1)
    for i in range(3):
        np.testing.assert_array_equal(full[i], oracle.conv(x[i], w, b, k, lam, 0, 14, (1, 1, 1, 1), (1, 1), 1, 1))


@pytest.mark.parametrize("bn_bits", [32, 64])
@pytest.mark.parametrize("flags", FLAGS)
def test_pointwise_equals_1x1_conv_and_numpy(flags, bn_bits):
    relu, bn = flags
    r = rng_for(200 + relu + 3 * bn)
    H, W, Ci, Co = 5, 7, 24, 13
    x, w, b = rand_u8(r, (2, H, W, Ci)), rand_s8(r, (Co, 1, 1, Ci)), rand_s8(r, (Co,))
    k, lam = r.integers(256, 1025, Co), r.integers(-2 ** 16, 2 ** 16, Co)
    mult, shift = 700, (17 if relu else 8)
    got = oracle.pointwise(x, w, b, k, lam, mult, shift, relu, bn, bn_bits)
    via_conv = oracle.conv(x, w, b, k, lam, mult, shift, (0, 0, 0, 0), (1, 1), relu, bn, bn_bits)
    np.testing.assert_array_equal(got, via_conv)
    acc = x.astype(np.int64) @ w.reshape(Co, Ci).astype(np.int64).T + b.astype(np.int64)
    np.testing.assert_array_equal(got, npref.epilogue(acc, k, lam, mult, shift, relu, bn, bn_bits))


def test_pointwise_config1_shape_sample():
    """BASELINE config 1 geometry (28x28x128 -> 256), one image, multiplier branch."""
    r = rng_for(1)
    x, w, b = rand_u8(r, (28, 28, 128)), rand_s8(r, (256, 128)), rand_s8(r, (256,))
    mult = int(r.integers(256, 1025))
    got = oracle.pointwise(x, w, b, None, None, mult, 18, 1, 0)
    acc = x.astype(np.int64) @ w.astype(np.int64).T + b.astype(np.int64)
    np.testing.assert_array_equal(got, npref.epilogue(acc, None, None, mult, 18, 1, 0))
    assert 0 < got.mean() < 255


def test_pointwise_reads_input_with_input_row_stride():
    """Output smaller than input: pixel (y, x) still comes from in[y][x]."""
    r = rng_for(2)
    x, w = rand_u8(r, (6, 8, 4)), rand_s8(r, (3, 4))
    got = oracle.pointwise(x, w, None, None, None, 0, 4, 0, 0, out_hw=(4, 5))
    full = oracle.pointwise(x, w, None, None, None, 0, 4, 0, 0)
    np.testing.assert_array_equal(got, full[:4, :5])


def test_matmul_is_two_pixels_of_conv():
    r = rng_for(3)
    K, Co = 27, 7   # K % 4 != 0 and Co % 4 != 0 exercise the reference's tail loops
    w, cols, b = rand_s8(r, (Co, K)), rand_u8(r, (2, K)), rand_s8(r, (Co,))
    k, lam = r.integers(256, 1025, Co), r.integers(-2 ** 16, 2 ** 16, Co)
    o0, o1 = oracle.matmul(w, cols, b, k, lam, 0, 12, 1, 1)
    acc = cols.astype(np.int64) @ w.astype(np.int64).T + b.astype(np.int64)
    want = npref.epilogue(acc, k, lam, 0, 12, 1, 1)
    np.testing.assert_array_equal(o0, want[0])
    np.testing.assert_array_equal(o1, want[1])


DW_GEOMS = [
    # CH, H, W, ky, kx, pads, strides
    (8, 12, 12, 3, 3, (1, 1, 1, 1), (1, 1)),
    (8, 12, 12, 3, 3, (1, 1, 1, 1), (2, 2)),     # config 2 stride-2 style (right/bottom pad unused)
    (5, 9, 11, 3, 3, (1, 1, 1, 1), (2, 2)),      # odd sizes: right/bottom pad used
    (3, 10, 8, 5, 5, (2, 2, 2, 2), (1, 1)),
    (4, 7, 9, 3, 5, (1, 1, 2, 2), (1, 1)),       # ky != kx
    (6, 8, 8, 1, 1, (0, 0, 0, 0), (1, 1)),       # fewer than 4 weights
    (2, 6, 6, 2, 2, (0, 0, 0, 0), (2, 2)),
]


@pytest.mark.parametrize("bn_bits", [32, 64])
@pytest.mark.parametrize("flags", [(1, 1), (1, 0), (0, 0), (2, 0)])
@pytest.mark.parametrize("geom", DW_GEOMS, ids=lambda g: "x".join(map(str, g[:5])) + "s%d" % g[6][0])
def test_depthwise_generic(geom, flags, bn_bits):
    CH, H, W, ky, kx, pads, strides = geom
    relu, bn = flags
    r = rng_for(300 + relu + 3 * bn + bn_bits)
    x, wt, b = rand_u8(r, (2, CH, H, W)), rand_s8(r, (CH, ky, kx)), rand_s8(r, (CH,))
    k, lam = r.integers(2 ** 12, 2 ** 14 + 1, CH), r.integers(-2 ** 16, 2 ** 16 + 1, CH)
    mult, shift = 900, (16 if (relu and bn) else (14 if relu else 6))
    got = oracle.depthwise_generic(x, wt, b, k, lam, mult, shift, pads, strides, relu, bn, bn_bits)
    for i in range(2):
        acc = npref.depthwise_acc(x[i], wt, b, pads, strides)
        want = npref.epilogue(acc, k, lam, mult, shift, relu, bn, bn_bits, relu_eq1=False)
        np.testing.assert_array_equal(got[i], want)


def test_depthwise_bn32_wrap_events_present_and_matched():
    """Config 2 parameter ranges overflow int32 for some outputs; the oracle must wrap."""
    r = rng_for(4)
    CH, H, W = 16, 20, 20
    x, wt = rand_u8(r, (CH, H, W)), rand_s8(r, (CH, 3, 3))
    k, lam = r.integers(2 ** 12, 2 ** 14 + 1, CH), r.integers(-2 ** 16, 2 ** 16 + 1, CH)
    wt[0], k[0] = 127, 2 ** 14          # same-sign taps: accumulators up to 9*255*127 > 2^31 / 2^14
    wt[1], k[1] = -128, 2 ** 14
    acc = npref.depthwise_acc(x, wt, None, (1, 1, 1, 1), (1, 1))
    exact = acc.astype(object) * k.astype(object) + lam.astype(object)
    assert (np.abs(exact) >= 2 ** 31).any(), "test needs at least one int32 overflow"
    got = oracle.depthwise_generic(x, wt, None, k, lam, 0, 16, (1, 1, 1, 1), (1, 1), 1, 1, 32)
    np.testing.assert_array_equal(got, npref.epilogue(acc, k, lam, 0, 16, 1, 1, 32))
    unwrapped = np.clip(exact >> 16, 0, 255).astype(np.uint8)
    assert (got != unwrapped).any(), "wrap must change at least one output"


@pytest.mark.parametrize("bn_bits", [32, 64])
@pytest.mark.parametrize("flags", [(1, 1), (1, 0), (0, 0)])
@pytest.mark.parametrize("shape", [(128, 10, 56), (5, 7, 6), (3, 3, 2), (4, 12, 20)])
def test_depthwise_3x3_s1_equals_generic_on_row_padded_plane(shape, flags, bn_bits):
    CH, H, W = shape
    relu, bn = flags
    r = rng_for(400 + relu + bn)
    x, kern = rand_u8(r, (2, CH, H, W)), rand_s8(r, (CH, 3, 3))
    k, lam = r.integers(2 ** 12, 2 ** 14 + 1, CH), r.integers(-2 ** 16, 2 ** 16 + 1, CH)
    mult, shift = 600, (16 if (relu and bn) else (13 if relu else 5))
    xpad = np.pad(x, ((0, 0), (0, 0), (1, 1), (0, 0)))     # the caller supplies the zero rows
    got = oracle.depthwise_3x3_s1(xpad, kern, k, lam, mult, shift, 1, 1, relu, bn, bn_bits)
    want = oracle.depthwise_generic(x, kern, None, k, lam, mult, shift, (1, 1, 1, 1), (1, 1), relu, bn, bn_bits)
    np.testing.assert_array_equal(got, want)
    acc = npref.depthwise_acc(x[0], kern, None, (1, 1, 1, 1), (1, 1))
    np.testing.assert_array_equal(got[0], npref.epilogue(acc, k, lam, mult, shift, relu, bn, bn_bits))


@pytest.mark.parametrize("bn_bits", [32, 64])
@pytest.mark.parametrize("dims", [(512, 1000), (1024, 4096), (37, 11)])
def test_linear(dims, bn_bits):
    K, N = dims
    r = rng_for(500 + K)
    x, w, b = rand_u8(r, (3, K)), rand_s8(r, (N, K)), rand_s8(r, (N,))
    k, lam = r.integers(256, 1025, N), r.integers(-2 ** 16, 2 ** 16, N)
    acc = x.astype(np.int64) @ w.astype(np.int64).T + b.astype(np.int64)
    for relu, bn, shift in [(1, 1, 21), (1, 0, 19), (0, 0, 11), (0, 1, 11)]:
        got = oracle.linear(x, w, b, k, lam, 800, shift, relu, bn, bn_bits)
        np.testing.assert_array_equal(got, npref.epilogue(acc, k, lam, 800, shift, relu, bn, bn_bits))
    # invariant: a linear layer is a pointwise conv on a 1x1 image
    pw = oracle.pointwise(x.reshape(3, 1, 1, K), w, b, k, lam, 800, 21, 1, 1, bn_bits)
    np.testing.assert_array_equal(pw.reshape(3, N), oracle.linear(x, w, b, k, lam, 800, 21, 1, 1, bn_bits))


def test_linear_out_32():
    r = rng_for(6)
    K, N = 512, 1000
    x, w = rand_u8(r, (4, K)), rand_s8(r, (N, K))
    b32 = r.integers(-2 ** 31, 2 ** 31, N, dtype=np.int64).astype(np.int32)
    acc = x.astype(np.int64) @ w.astype(np.int64).T + b32.astype(np.int64)
    want = npref.wrap(acc, 32).astype(np.int64).astype(np.int32)
    np.testing.assert_array_equal(oracle.linear_out_32(x, w, b32), want)
    np.testing.assert_array_equal(oracle.linear_out_32(x, w, None),
                                  (x.astype(np.int64) @ w.astype(np.int64).T).astype(np.int32))


@pytest.mark.parametrize("case", [
    # H, W, C, kernel(kx,ky), strides(sx,sy), out_hw
    (63, 63, 16, (2, 2), (2, 2), (32, 32)),   # config 4: ceil mode through the window clamp
    (63, 63, 16, (2, 2), (2, 2), (31, 31)),   # floor mode
    (8, 8, 5, (2, 2), (2, 2), (4, 4)),
    (9, 7, 3, (3, 2), (2, 1), (8, 3)),
    (6, 6, 4, (3, 3), (3, 3), (2, 2)),
])
def test_maxpool_matches_windowed_max(case):
    H, W, C, kernel, strides, out_hw = case
    r = rng_for(600 + H)
    x = rand_u8(r, (2, H, W, C))
    keep = x.copy()
    got = oracle.maxpool(x, kernel, strides, out_hw=out_hw)
    np.testing.assert_array_equal(x, keep)            # clobber=False leaves the input alone
    for i in range(2):
        np.testing.assert_array_equal(got[i], npref.maxpool(x[i], kernel, strides, out_hw))


def test_maxpool_clobbers_input_like_the_reference():
    """The first pass pools along x in place: after the call, column i_x of every
    input row holds the x-pooled value (pulp_nn_maxpool.c:58-94)."""
    r = rng_for(7)
    x = rand_u8(r, (6, 8, 3))
    orig = x.copy()
    oracle.maxpool(x, (2, 2), (2, 2), out_hw=(3, 4), clobber=True)
    want_cols = np.maximum(orig[:, 0::2], orig[:, 1::2])
    np.testing.assert_array_equal(x[:, :4], want_cols)
    np.testing.assert_array_equal(x[:, 4:], orig[:, 4:])


@pytest.mark.parametrize("bn_bits", [32, 64])
def test_avgpool_global_and_windowed(bn_bits):
    r = rng_for(8)
    x = rand_u8(r, (3, 4, 4, 512))
    got = oracle.avgpool(x, (4, 4), (4, 4), bn_bits=bn_bits)
    want = (x.astype(np.int64).sum(axis=(1, 2)) // 16).astype(np.uint8).reshape(3, 1, 1, 512)
    np.testing.assert_array_equal(got, want)
    x2 = rand_u8(r, (8, 6, 5))
    got = oracle.avgpool(x2, (2, 2), (2, 2), bn_bits=bn_bits)
    s = x2.astype(np.int64).reshape(4, 2, 3, 2, 5).sum(axis=(1, 3))
    np.testing.assert_array_equal(got, (s // 4).astype(np.uint8))


def test_avgpool_requant_32_is_unsigned_and_64_is_signed():
    x = np.full((2, 2, 1), 100, np.uint8)       # sum = 400, ksize = 4
    # positive parameters: both trees agree: (400*3/4 + 20) >> 2 = 80
    assert oracle.avgpool(x, (2, 2), (2, 2), lam=3, out_shift=2, out_add=20, flag_requant=1, bn_bits=32)[0, 0, 0] == 80
    assert oracle.avgpool(x, (2, 2), (2, 2), lam=3, out_shift=2, out_add=20, flag_requant=1, bn_bits=64)[0, 0, 0] == 80
    # negative lambda: 32bit tree works in uint32: (2^32-400)/4 = 1073741724; +500 -> >>22 = 256 -> 255
    assert oracle.avgpool(x, (2, 2), (2, 2), lam=-1, out_shift=22, out_add=500, flag_requant=1, bn_bits=32)[0, 0, 0] == 255
    # 64bit tree is signed: (-400/4 + 500) >> 2 = 100
    assert oracle.avgpool(x, (2, 2), (2, 2), lam=-1, out_shift=2, out_add=500, flag_requant=1, bn_bits=64)[0, 0, 0] == 100
    # 64bit signed division truncates toward zero: -401/4 = -100 (not -101): (-100+101)>>0 = 1
    x[0, 0, 0] = 101
    assert oracle.avgpool(x, (2, 2), (2, 2), lam=-1, out_shift=0, out_add=101, flag_requant=1, bn_bits=64)[0, 0, 0] == 1


def test_avgpool_padding_arguments_as_written():
    """Window rows start at i_y*sy - padding_b and columns end at i_x*sx - padding_r + kx
    (pulp_nn_avgpool.c:82-86); the divisor stays kx*ky."""
    r = rng_for(9)
    x = rand_u8(r, (6, 6, 2))
    got = oracle.avgpool(x, (3, 3), (1, 1), pads=(1, 1, 1, 1), out_hw=(6, 6))
    xi = x.astype(np.int64)
    for oy in range(6):
        for ox in range(6):
            ys, ye = max(0, oy - 1), min(oy - 1 + 3, 6)
            xs, xe = max(0, ox - 1), min(ox - 1 + 3, 6)
            want = xi[ys:ye, xs:xe].sum(axis=(0, 1)) // 9
            np.testing.assert_array_equal(got[oy, ox], want.astype(np.uint8))


def test_avgpool_asymmetric_padding_known_answer():
    """Hand-derived: 3x3 image, one channel, 2x2 window, stride 1, pads (t,b,l,r) = (0,1,0,1).
    pulp_nn_avgpool.c:82-86: rows [max(0, iy - padding_b), min(iy - padding_t + 2, 3)),
    columns [max(0, ix - padding_l), min(ix - padding_r + 2, 3)); divisor 4.
      in = [[ 4,  8, 12],
            [16, 20, 24],
            [28, 32, 36]]
    output (1,1): rows [0,3), columns [1,2) -> (8+20+32)/4 = 15.  Reading padding_t as the row
    start and padding_l as the column end would give rows [1,3), columns [1,3) -> 112/4 = 28.
    output (0,0): rows [0,2), columns [0,1) -> (4+16)/4 = 5   (the other reading: (4+8+16+20)/4 = 12)
    output (0,1): rows [0,2), columns [1,2) -> (8+20)/4 = 7   (other: 64/4 = 16)
    output (1,0): rows [0,3), columns [0,1) -> (4+16+28)/4 = 12 (other: 96/4 = 24)"""
    x = np.array([[4, 8, 12], [16, 20, 24], [28, 32, 36]], np.uint8).reshape(3, 3, 1)
    got = oracle.avgpool(x, (2, 2), (1, 1), pads=(0, 1, 0, 1), out_hw=(2, 2))
    np.testing.assert_array_equal(got[:, :, 0], np.array([[5, 7], [12, 15]], np.uint8))
    # the mirrored pads (1,0,1,0): rows [max(0, iy), min(iy - 1 + 2, 3)), columns [max(0, ix - 1), min(ix + 2, 3))
    # (0,0): row 0, columns [0,2) -> 12/4 = 3; (0,1): row 0, columns [0,3) -> 24/4 = 6
    # (1,0): row 1, columns [0,2) -> 36/4 = 9; (1,1): row 1, columns [0,3) -> 60/4 = 15
    got = oracle.avgpool(x, (2, 2), (1, 1), pads=(1, 0, 1, 0), out_hw=(2, 2))
    np.testing.assert_array_equal(got[:, :, 0], np.array([[3, 6], [9, 15]], np.uint8))


def test_maxpool_padded_known_answers():
    """Hand-derived from pulp_nn_maxpool.c:58-144.
    (a) 3x3 window, stride 2, padding 1 on a 5x5 one-channel image: column windows
        [0,2) (start -1 < 0 -> the target column 0), [1,4), [3,5) (end clamped to 5), rows alike.
          in = [[ 1,  2,  3,  4,  5],
                [10,  9,  8,  7,  6],
                [11, 12, 13, 14, 15],
                [20, 19, 18, 17, 16],
                [21, 22, 23, 24, 25]]
        x pass (per row): [2,4,5] [10,9,7] [12,14,15] [20,19,17] [22,24,25]
        y pass rows [0,2) [1,4) [3,5): [[10,9,7],[20,19,17],[22,24,25]]
    (b) the left clamp is the output column itself, not column 0 (:65-68): 1x4 image [9,1,5,3],
        3-wide window, stride 1, padding_l 2, three outputs.  ix=0: start -2 -> column 0, end 1 -> 9;
        ix=1: start -1 -> column 1 (a clamp to 0 would include the 9), end 2 -> 1;
        ix=2: columns [0,3) of the row as the in-place pass has left it: [9,1,5] -> 9."""
    x = np.array([[1, 2, 3, 4, 5], [10, 9, 8, 7, 6], [11, 12, 13, 14, 15], [20, 19, 18, 17, 16],
                  [21, 22, 23, 24, 25]], np.uint8).reshape(5, 5, 1)
    got = oracle.maxpool(x, (3, 3), (2, 2), pads=(1, 1, 1, 1), out_hw=(3, 3))
    np.testing.assert_array_equal(got[:, :, 0], np.array([[10, 9, 7], [20, 19, 17], [22, 24, 25]], np.uint8))
    # and against the windowed maximum with the padding excluded, on random data
    r = rng_for(11)
    xr = rand_u8(r, (9, 11, 3))
    got = oracle.maxpool(xr, (3, 3), (2, 2), pads=(1, 1, 1, 1), out_hw=(5, 6))
    for oy in range(5):
        for ox in range(6):
            ys, ye = max(0, 2 * oy - 1), min(2 * oy + 2, 9)
            xs, xe = max(0, 2 * ox - 1), min(2 * ox + 2, 11)
            np.testing.assert_array_equal(got[oy, ox], xr[ys:ye, xs:xe].max(axis=(0, 1)))
    y = np.array([9, 1, 5, 3], np.uint8).reshape(1, 4, 1)
    got = oracle.maxpool(y, (3, 1), (1, 1), pads=(0, 0, 2, 0), out_hw=(1, 3))
    np.testing.assert_array_equal(got[0, :, 0], np.array([9, 1, 9], np.uint8))


def test_add_matches_exact_integers():
    r = rng_for(10)
    a, b = rand_u8(r, (3, 5, 7, 4)), rand_u8(r, (3, 5, 7, 4))
    for m1, m2, d in [(3, 5, 2), (120, 130, 8), (65535, 2, 0), (32767, 32767, 9)]:
        v = (a.astype(np.int64) * npref.as_i16(m1) + b.astype(np.int64) * npref.as_i16(m2)) % (1 << 32)
        want = np.minimum((v >> d) & 0xFFFF, 255).astype(np.uint8)
        np.testing.assert_array_equal(oracle.add(a, b, m1, m2, d), want)
