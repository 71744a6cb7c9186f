"""Independent numpy closed forms used to pin the C oracle.

Nothing here shares code with oracle/pulpnn_oracle.c: contractions are done by
numpy on explicitly zero-padded arrays (sliding windows + einsum in int64) and
the epilogue by exact Python integers followed by an explicit wrap to the
reference's C type, so an index, sign, transposition or width mistake in the
C restatement shows up as a mismatch.
"""
import numpy as np
from numpy.lib.stride_tricks import sliding_window_view


def wrap(v, bits):
    """Two's-complement wrap of exact integers (object or int64 arrays) to `bits`."""
    v = np.asarray(v, dtype=object)
    m = 1 << bits
    return ((v + (m >> 1)) % m) - (m >> 1)


def clipu8(x):
    x = np.asarray(x, dtype=object)
    return np.clip(x, 0, 255).astype(np.uint8)


def as_i8(v):
    return ((int(v) + 128) & 0xFF) - 128


def as_i16(v):
    return ((int(v) + 32768) & 0xFFFF) - 32768


def epilogue(acc, k, lam, out_mult, out_shift, flag_relu, flag_bn, bn_bits=32, relu_eq1=True):
    """acc: int array [..., C]; k, lam: [C] (only read in the batch-norm branch)."""
    acc = np.asarray(acc).astype(object)
    if flag_bn and flag_relu:
        d = as_i8(out_shift)
        kk = np.asarray(k).astype(object)
        ll = np.asarray(lam).astype(object)
        v = wrap(kk * acc + ll, bn_bits)
        x = v >> d
        if bn_bits == 64:
            x = wrap(x, 32)
        return clipu8(x)
    if (flag_relu == 1) if relu_eq1 else bool(flag_relu):
        d = as_i8(out_shift)
        prod = wrap(as_i16(out_mult) * acc, 32)
        return clipu8(wrap(prod >> d, 16))
    return clipu8(acc >> int(out_shift))


def conv_acc(x, w, bias, pads, strides):
    """x: H,W,Ci u8; w: Co,ky,kx,Ci s8 -> int64 Ho,Wo,Co (zero-padded cross-correlation)."""
    pt, pb, pl, pr = pads
    sx, sy = strides
    Co, ky, kx, Ci = w.shape
    xp = np.pad(x.astype(np.int64), ((pt, pb), (pl, pr), (0, 0)))
    win = sliding_window_view(xp, (ky, kx), axis=(0, 1))[::sy, ::sx]  # Ho,Wo,Ci,ky,kx
    acc = np.einsum("hwcyx,oyxc->hwo", win, w.astype(np.int64))
    if bias is not None:
        acc = acc + np.asarray(bias).astype(np.int64)
    return acc


def depthwise_acc(x_chw, wt, bias, pads, strides):
    """x: CH,H,W u8; wt: CH,ky,kx s8 -> int64 Ho,Wo,CH."""
    pt, pb, pl, pr = pads
    sx, sy = strides
    CH, ky, kx = wt.shape
    xp = np.pad(x_chw.astype(np.int64), ((0, 0), (pt, pb), (pl, pr)))
    win = sliding_window_view(xp, (ky, kx), axis=(1, 2))[:, ::sy, ::sx]  # CH,Ho,Wo,ky,kx
    acc = np.einsum("chwyx,cyx->hwc", win, wt.astype(np.int64))
    if bias is not None:
        acc = acc + np.asarray(bias).astype(np.int64)
    return acc


def maxpool(x, kernel, strides, out_hw):
    """Clamped-window max without padding; ceil-mode sizes allowed."""
    H, W, C = x.shape
    kx, ky = kernel
    sx, sy = strides
    Ho, Wo = out_hw
    out = np.empty((Ho, Wo, C), np.uint8)
    for oy in range(Ho):
        for ox in range(Wo):
            out[oy, ox] = x[oy * sy:min(oy * sy + ky, H), ox * sx:min(ox * sx + kx, W)].max(axis=(0, 1))
    return out
