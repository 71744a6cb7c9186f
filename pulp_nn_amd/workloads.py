"""Seeded synthetic tensors for the five benchmark configurations.

numpy only.  All tensors come from numpy's PCG64 generator with one fixed seed per
configuration: activations uniform in [0, 255], weights uniform in [-128, 127].

Choices where the configuration text cannot be passed through the reference ABI
as written:
  * bias is int8 in the reference ABI (one byte per output channel) for every
    conv / pointwise / depthwise / linear; it is drawn uniform in [-128, 127].
    Only linear_out_32 takes a 32-bit bias, drawn uniform in [-2^12, 2^12].
  * out_mult is one uint16 scalar per call, so "uniform [256, 1024]" is one draw.
  * the batch-norm branch is only taken when flag_relu is set as well, so the
    64-bit batch-norm stress case is run with flag_relu = 1 (and once literally,
    with flag_relu = 0, which ignores k / lambda).
"""
import numpy as np

SEEDS = {0: 20240, 1: 20241, 2: 20242, 3: 20243, 4: 20244}


def _rng(cfg):
    return np.random.Generator(np.random.PCG64(SEEDS[cfg]))


def _u8(r, shape):
    return r.integers(0, 256, size=shape, dtype=np.uint8)


def _s8(r, shape):
    return r.integers(-128, 128, size=shape, dtype=np.int8)


def config0(batch=1):
    """3x3 conv 16x16x32 -> 16x16x64, pad 1, stride 1, 32-bit batch-norm + relu."""
    r = _rng(0)
    return dict(
        name="cfg0_conv3x3_16x16x32_64", bn_bits=32, batch=batch,
        w=_s8(r, (64, 3, 3, 32)), bias=_s8(r, (64,)),
        k=r.integers(256, 1025, 64).astype(np.int32), lam=r.integers(-2 ** 16, 2 ** 16 + 1, 64).astype(np.int32),
        out_mult=0, out_shift=20, pads=(1, 1, 1, 1), strides=(1, 1), relu=1, bn=1,
        x=_u8(r, (batch, 16, 16, 32)), out_hw=(16, 16),
        ops=2 * batch * 16 * 16 * 64 * 288,
        bytes=batch * (16 * 16 * 32 + 16 * 16 * 64) + 64 * 288 + 64 * 9)


def config1(batch=256):
    """Pointwise 28x28x128 -> 256, scalar-multiplier requantisation + relu."""
    r = _rng(1)
    return dict(
        name="cfg1_pointwise_28x28x128_256", bn_bits=32, batch=batch,
        w=_s8(r, (256, 1, 1, 128)), bias=_s8(r, (256,)), k=None, lam=None,
        out_mult=int(r.integers(256, 1025)), out_shift=18, relu=1, bn=0,
        x=_u8(r, (batch, 28, 28, 128)), out_hw=(28, 28),
        ops=2 * batch * 28 * 28 * 256 * 128,
        bytes=batch * (28 * 28 * 128 + 28 * 28 * 256) + 256 * 128 + 256)


def config2(batch=256, stride=1):
    """Depthwise 3x3 on 56x56x128 (CHW in, HWC out), pad 1, 32-bit batch-norm + relu."""
    r = _rng(2)
    ho = 56 if stride == 1 else 28
    return dict(
        name="cfg2_depthwise3x3_s%d_56x56x128" % stride, bn_bits=32, batch=batch, stride=stride,
        w=_s8(r, (128, 3, 3)), bias=_s8(r, (128,)),
        k=r.integers(2 ** 12, 2 ** 14 + 1, 128).astype(np.int32),
        lam=r.integers(-2 ** 16, 2 ** 16 + 1, 128).astype(np.int32),
        out_mult=0, out_shift=16, relu=1, bn=1,
        x=_u8(r, (batch, 128, 56, 56)), out_hw=(ho, ho),
        ops=2 * batch * ho * ho * 128 * 9,
        bytes=batch * (56 * 56 * 128 + ho * ho * 128) + 128 * 9 + 128 * 9)


def config4(batch=64, relu=1):
    """64-bit batch-norm 3x3 conv 64x64x256 -> 63x63x256, padding (top 1, bottom 0, left 1, right 0)."""
    r = _rng(4)
    return dict(
        name="cfg4_conv3x3_64x64x256_256_bn64", bn_bits=64, batch=batch,
        w=_s8(r, (256, 3, 3, 256)), bias=_s8(r, (256,)),
        k=r.integers(2 ** 20, 2 ** 24 + 1, 256).astype(np.int64),
        lam=r.integers(-2 ** 36, 2 ** 36 + 1, 256).astype(np.int64),
        out_mult=0, out_shift=38, pads=(1, 0, 1, 0), strides=(1, 1), relu=relu, bn=1,
        x=_u8(r, (batch, 64, 64, 256)), out_hw=(63, 63),
        lin_w=_s8(r, (4096, 1024)), lin_bias=_s8(r, (4096,)),
        lin_k=r.integers(2 ** 20, 2 ** 24 + 1, 4096).astype(np.int64),
        lin_lam=r.integers(-2 ** 36, 2 ** 36 + 1, 4096).astype(np.int64), lin_shift=30,
        ops=2 * batch * 63 * 63 * 256 * 2304,
        bytes=batch * (64 * 64 * 256 + 63 * 63 * 256) + 256 * 2304 + 256 * 17)
