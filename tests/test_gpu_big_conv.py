"""GPU parity of the large-tile convolution path (persistent workgroups on 256 x 256 tiles fed by LDS-direct loads).

That path is taken by convolutions with input channels a multiple of 64, more than 128 output channels (a multiple
of 16), K of at least 256 bytes and at least two 256 x 256 tiles per compute unit; these geometries are sized to reach
it and to exercise its edges (channel tail, pixel tail, padding on every side, stride 2, several channel tiles, an
odd number of K sub-slices, the shortest K, every epilogue branch, both widths).  One geometry (136 channels) stays
on the tiled kernel of the same tile size.  3-wide stride-1 filters on images of 57 to 64 output columns take the
patch-tiled variant of the path (4 x 64 pixel patches, input rows staged once per filter row); five geometries reach it."""
import numpy as np
import pytest

import oracle
from gpu_helpers import conv, rand_s8, rand_u8, rng_for

pytestmark = pytest.mark.gpu

GEOMS = [
    # B, H, W, Ci, Co, ky, kx, pads (t, b, l, r), strides
    (84, 40, 40, 128, 256, 3, 3, (1, 1, 1, 1), (1, 1)),
    (140, 31, 33, 128, 192, 3, 3, (1, 0, 1, 0), (1, 1)),    # channel tail (192 of a 256 tile), odd sizes, asymmetric pads
    (150, 60, 62, 128, 136, 3, 3, (0, 1, 0, 1), (2, 2)),    # stride 2, pads bottom / right only
    (140, 32, 32, 256, 256, 1, 3, (0, 0, 1, 1), (1, 1)),    # 1 x 3 filter, K = 768
    (84, 40, 40, 64, 256, 3, 3, (1, 1, 1, 1), (1, 1)),      # 64 input channels: one K sub-slice per tap, nine in all (odd)
    (70, 48, 48, 192, 512, 3, 3, (1, 1, 1, 1), (1, 1)),     # two channel tiles per pixel tile, three sub-slices per tap
    (262, 23, 23, 320, 256, 1, 1, (0, 0, 0, 0), (1, 1)),    # K = 320: five sub-slices, one more than the ring has stages
    # 3-wide stride-1 filters on 57 to 64 output columns: patches of 4 rows x 64 columns, input rows staged once per
    # filter row (igemm_patch_kernel)
    (36, 62, 60, 64, 256, 3, 3, (1, 1, 1, 1), (1, 1)),      # 60 columns, 62 rows (two dead rows in the last patch), one group per filter row
    (34, 64, 64, 128, 512, 3, 3, (1, 0, 1, 0), (1, 1)),     # config 4 shape (63 x 63 out), two channel tiles
    (40, 60, 64, 128, 192, 1, 3, (0, 0, 1, 1), (1, 1)),     # 1 x 3 filter: two groups in all; channel tail
    (34, 64, 64, 64, 256, 5, 3, (2, 2, 0, 1), (1, 1)),      # 5 x 3 filter, no left padding, 63 columns
    (38, 58, 62, 192, 256, 3, 3, (0, 1, 1, 0), (1, 1)),     # no top padding, three groups per filter row, 57 x 61 out
]
FLAGS = [(1, 1), (1, 0), (0, 0), (0, 1)]


@pytest.mark.parametrize("bn_bits", [32, 64])
@pytest.mark.parametrize("flags", FLAGS)
@pytest.mark.parametrize("geom", GEOMS, ids=lambda g: "x".join(map(str, g[:7])))
def test_big_conv(geom, flags, bn_bits):
    B, H, W, Ci, Co, ky, kx, pads, strides = geom
    relu, bn = flags
    r = rng_for(4242 + 3 * relu + bn + bn_bits)
    x, w, b = rand_u8(r, (B, H, W, Ci)), rand_s8(r, (Co, ky, kx, Ci)), rand_s8(r, (Co,))
    K = ky * kx * Ci
    if bn_bits == 64:
        k, lam, bshift = r.integers(2 ** 20, 2 ** 24, Co), r.integers(-2 ** 36, 2 ** 36, Co), 38 - 3
    else:
        k, lam, bshift = r.integers(256, 1025, Co), r.integers(-2 ** 16, 2 ** 16, Co), 20
    mult = int(r.integers(256, 1025))
    lg = int(np.log2(K ** 0.5 * 128 * 74))
    shift = bshift if (relu and bn) else ((lg + 10 - 7) if relu == 1 else max(lg - 7, 0))
    # the oracle on a sample of the images (whole images: first, last and two in between)
    sample = sorted({0, B // 3, 2 * B // 3, B - 1})
    got = conv(x, w, b, k, lam, mult, shift, pads, strides, relu, bn, bn_bits)
    want = oracle.conv(x[sample], w, b, k, lam, mult, shift, pads, strides, relu, bn, bn_bits)
    assert got.shape[1:] == want.shape[1:]
    assert np.array_equal(got[sample], want), "big conv mismatch"
    assert want.max() > 0 and (want < 255).any(), "degenerate case"
    # images are independent: every image with the same input as a checked one must equal it
    x2 = x.copy()
    x2[1] = x[0]
    got2 = conv(x2, w, b, k, lam, mult, shift, pads, strides, relu, bn, bn_bits)
    assert np.array_equal(got2[1], want[0])


# ---- stride-2 depthwise on whole 64-channel groups (bands staged by LDS-direct loads), at config-2 scale ----
# That staging needs whole 64-channel groups, W % 4 == 0 and Wo % 4 == 0.
DW_GEOMS = [
    # B, CH, H, W, pads (t, b, l, r)
    (130, 128, 56, 56, (1, 1, 1, 1)),    # config 2 geometry: four bands, the top one with a row above the image
    (520, 64, 30, 32, (1, 0, 1, 0)),     # one band per image, 15 output rows
    (260, 128, 17, 24, (0, 0, 0, 1)),    # no top / left padding (the other window alignment), 8 x 12 outputs
    (70, 192, 63, 40, (1, 1, 1, 1)),     # three channel groups, bands of unequal height (32 output rows in 5 bands)
]


@pytest.mark.parametrize("bn_bits", [32, 64])
@pytest.mark.parametrize("flags", [(1, 1), (1, 0), (0, 0)])
@pytest.mark.parametrize("geom", DW_GEOMS, ids=lambda g: "x".join(map(str, g[:4])))
def test_big_depthwise_stride2(geom, flags, bn_bits):
    from gpu_helpers import depthwise_generic
    B, CH, H, W, pads = geom
    relu, bn = flags
    r = rng_for(977 + relu + 2 * bn + bn_bits)
    x, wt = rand_u8(r, (B, CH, H, W)), rand_s8(r, (CH, 3, 3))
    b = rand_s8(r, (CH,)) if (relu + bn) % 2 == 0 else None
    if bn_bits == 64:
        k, lam, shift = r.integers(2 ** 20, 2 ** 24, CH), r.integers(-2 ** 36, 2 ** 36, CH), 34
        if bn and relu and CH == 64:
            k = r.integers(2 ** 33, 2 ** 34, CH)     # k does not fit 32 bits: the general 64-bit path
            shift = 44
    else:
        k, lam, shift = r.integers(2 ** 12, 2 ** 14, CH), r.integers(-2 ** 16, 2 ** 16, CH), 16
    mult = int(r.integers(256, 1025))
    if not (relu and bn):
        shift = 19 if relu == 1 else 9
    sample = sorted({0, 1, B // 2, B - 1})
    got = depthwise_generic(x, wt, b, k, lam, mult, shift, pads, (2, 2), relu, bn, bn_bits)
    want = oracle.depthwise_generic(x[sample], wt, b, k, lam, mult, shift, pads, (2, 2), relu, bn, bn_bits)
    assert got.shape[1:] == want.shape[1:]
    assert np.array_equal(got[sample], want), "depthwise mismatch"
    assert want.max() > 0 and (want < 255).any(), "degenerate case"
    # a digest over all images against the same layer computed image by image in small batches (other kernel)
    step = 4
    parts = [depthwise_generic(x[i:i + step], wt, b, k, lam, mult, shift, pads, (2, 2), relu, bn, bn_bits)
             for i in range(0, min(B, 24), step)]
    assert np.array_equal(np.concatenate(parts), got[:min(B, 24)])


# ---- stride-1 depthwise on whole 64-channel groups: bands staged by LDS-direct loads in the band kernel ----
DW1_GEOMS = [
    # B, CH, H, W, pads (t, b, l, r)
    (6, 128, 56, 56, (1, 1, 1, 1)),      # config 2 geometry: seven bands of eight output rows
    (5, 64, 20, 20, (1, 1, 1, 1)),       # rows of 5 dwords: the 16-byte pieces straddle the image's first and last row
    (4, 192, 45, 24, (0, 1, 0, 2)),      # no top / left padding, two bands, three channel groups
    (3, 64, 9, 112, (1, 1, 1, 1)),       # wide rows: the 64 KiB band limit applies instead of the 40 KiB one
    (2, 64, 6, 8, (1, 1, 1, 1)),         # a band shorter than one load instruction covers
    # batches of several hundred images (more workgroups than the GPU holds at once)
    (260, 128, 20, 20, (1, 1, 1, 1)),
    (600, 64, 13, 56, (1, 1, 1, 1)),     # 14 column groups on 8 waves
    (514, 64, 31, 40, (1, 0, 1, 1)),     # no bottom padding: 30 output rows
]


@pytest.mark.parametrize("bn_bits", [32, 64])
@pytest.mark.parametrize("flags", [(1, 1), (1, 0), (0, 0)])
@pytest.mark.parametrize("geom", DW1_GEOMS, ids=lambda g: "x".join(map(str, g[:4])))
def test_depthwise_stride1_whole_groups(geom, flags, bn_bits):
    from gpu_helpers import depthwise_generic
    B, CH, H, W, pads = geom
    relu, bn = flags
    r = rng_for(1977 + relu + 2 * bn + bn_bits)
    x, wt = rand_u8(r, (B, CH, H, W)), rand_s8(r, (CH, 3, 3))
    b = rand_s8(r, (CH,)) if (relu + bn) % 2 == 0 else None
    if bn_bits == 64:
        k, lam, shift = r.integers(2 ** 20, 2 ** 24, CH), r.integers(-2 ** 36, 2 ** 36, CH), 34
    else:
        k, lam, shift = r.integers(2 ** 12, 2 ** 14, CH), r.integers(-2 ** 16, 2 ** 16, CH), 16
    mult = int(r.integers(256, 1025))
    if not (relu and bn):
        shift = 19 if relu == 1 else 9
    got = depthwise_generic(x, wt, b, k, lam, mult, shift, pads, (1, 1), relu, bn, bn_bits)
    sample = list(range(B)) if B <= 8 else sorted({0, 1, B // 2, B - 1})
    want = oracle.depthwise_generic(x[sample], wt, b, k, lam, mult, shift, pads, (1, 1), relu, bn, bn_bits)
    assert got.shape[1:] == want.shape[1:]
    assert np.array_equal(got[sample], want), "depthwise mismatch"
    assert want.max() > 0 and (want < 255).any(), "degenerate case"
    if B > 8:
        # a digest over many images against the same layer computed in small batches
        step = 4
        parts = [depthwise_generic(x[i:i + step], wt, b, k, lam, mult, shift, pads, (1, 1), relu, bn, bn_bits)
                 for i in range(0, 24, step)]
        assert np.array_equal(np.concatenate(parts), got[:24])
