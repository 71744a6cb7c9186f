"""Helpers for the GPU parity tests: numpy in, C-ABI call on device tensors, numpy out.

Every helper calls the HIP library through its C ABI with the reference's own
argument lists; the oracle is only ever used by the tests to check the result."""
import numpy as np
import torch

from pulp_nn_amd import PulpNN

_libs = {}


def nn(bn_bits):
    if bn_bits not in _libs:
        _libs[bn_bits] = PulpNN(bn_bits)
    return _libs[bn_bits]


def dev(a, dtype=None):
    if a is None:
        return None
    a = np.ascontiguousarray(a, dtype=dtype)
    if a.dtype == np.uint16:
        a = a.view(np.int16)
    return torch.from_numpy(a).cuda()


def bn_dev(a, bn_bits):
    return dev(a, np.int64 if bn_bits == 64 else np.int32)


def rng_for(seed):
    return np.random.Generator(np.random.PCG64(seed))


def rand_u8(r, shape):
    return r.integers(0, 256, size=shape, dtype=np.uint8)


def rand_s8(r, shape):
    return r.integers(-128, 128, size=shape, dtype=np.int8)


def conv(x, w, bias, k, lam, mult, shift, pads, strides, relu, bn, bn_bits=32, out_hw=None,
         fn="pulp_nn_conv_Ho_parallel"):
    """x: B,H,W,Ci u8 -> B,Ho,Wo,Co u8 via the named conv / pointwise entry point."""
    B, H, W, Ci = x.shape
    Co, ky, kx = w.shape[0], w.shape[1], w.shape[2]
    pt, pb, pl, pr = pads
    sx, sy = strides
    if out_hw is None:
        out_hw = ((H + pt + pb - ky) // sy + 1, (W + pl + pr - kx) // sx + 1)
    Ho, Wo = out_hw
    L = nn(bn_bits)
    out = torch.full((B, Ho, Wo, Co), 0xA5, dtype=torch.uint8, device="cuda")
    L.set_batch(B)
    getattr(L, fn)(dev(x), None, dev(bias), out, dev(w), bn_dev(k, bn_bits), bn_dev(lam, bn_bits), mult, shift,
                   W, H, Ci, Wo, Ho, Co, kx, ky, pt, pb, pl, pr, sx, sy, relu, bn)
    L.sync()
    L.set_batch(1)
    return out.cpu().numpy()


def depthwise_generic(x, wt, bias, k, lam, mult, shift, pads, strides, relu, bn, bn_bits=32, out_hw=None,
                      fn="pulp_nn_depthwise_generic"):
    B, CH, H, W = x.shape
    ky, kx = wt.shape[1], wt.shape[2]
    pt, pb, pl, pr = pads
    sx, sy = strides
    if out_hw is None:
        out_hw = ((H + pt + pb - ky) // sy + 1, (W + pl + pr - kx) // sx + 1)
    Ho, Wo = out_hw
    L = nn(bn_bits)
    out = torch.full((B, Ho, Wo, CH), 0xA5, dtype=torch.uint8, device="cuda")
    L.set_batch(B)
    getattr(L, fn)(dev(x), None, dev(bias), out, dev(wt), None, bn_dev(k, bn_bits), bn_dev(lam, bn_bits), mult, shift,
                   W, H, CH, Wo, Ho, CH, kx, ky, pt, pb, pl, pr, sx, sy, relu, bn)
    L.sync()
    L.set_batch(1)
    return out.cpu().numpy()


def depthwise_hwc(x_hwc, wt, bias, k, lam, mult, shift, stride, relu, bn, bn_bits=32):
    """3x3, padding 1, HWC in and out (pulp_nn_hip_depthwise_hwc)."""
    B, H, W, CH = x_hwc.shape
    Ho, Wo = (H - 1) // stride + 1, (W - 1) // stride + 1
    L = nn(bn_bits)
    out = torch.full((B, Ho, Wo, CH), 0xA5, dtype=torch.uint8, device="cuda")
    L.set_batch(B)
    try:
        L.depthwise_hwc(dev(x_hwc), dev(bias), out, dev(wt), bn_dev(k, bn_bits), bn_dev(lam, bn_bits), mult, shift,
                        W, H, CH, Wo, Ho, stride, relu, bn)
        L.sync()
    finally:
        L.set_batch(1)
    return out.cpu().numpy()


def depthwise_3x3_s1(xpad, kern, k, lam, mult, shift, relu, bn, bn_bits=32, p_l=1, p_r=1):
    B, CH, R, Cw = xpad.shape
    L = nn(bn_bits)
    out = torch.full((B, R - 2, Cw, CH), 0xA5, dtype=torch.uint8, device="cuda")
    L.set_batch(B)
    L.pulp_nn_depthwise_3x3_s1(dev(xpad), out, R, Cw, CH, p_l, p_r, dev(kern), shift, mult, bn_dev(k, bn_bits),
                               bn_dev(lam, bn_bits), relu, bn, None)
    L.sync()
    L.set_batch(1)
    return out.cpu().numpy()


def linear(x, w, bias, k, lam, mult, shift, relu, bn, bn_bits=32):
    B, K = x.shape
    N = w.shape[0]
    L = nn(bn_bits)
    out = torch.full((B, N), 0xA5, dtype=torch.uint8, device="cuda")
    L.set_batch(B)
    L.pulp_nn_linear(dev(x), dev(bias), out, dev(w), bn_dev(k, bn_bits), bn_dev(lam, bn_bits), mult, shift, K, N,
                     relu, bn)
    L.sync()
    L.set_batch(1)
    return out.cpu().numpy()


def linear_out_32(x, w, bias32, bn_bits=32):
    B, K = x.shape
    N = w.shape[0]
    L = nn(bn_bits)
    out = torch.full((B, N), -7, dtype=torch.int32, device="cuda")
    L.set_batch(B)
    L.pulp_nn_linear_out_32(dev(x), dev(bias32, np.int32), out, dev(w), K, N)
    L.sync()
    L.set_batch(1)
    return out.cpu().numpy()


def maxpool(x, kernel, strides, out_hw, pads=(0, 0, 0, 0), bn_bits=32):
    B, H, W, Cc = x.shape
    Ho, Wo = out_hw
    L = nn(bn_bits)
    xin = dev(x)
    out = torch.full((B, Ho, Wo, Cc), 0xA5, dtype=torch.uint8, device="cuda")
    L.set_batch(B)
    L.pulp_nn_maxpool(xin, out, W, H, Cc, Wo, Ho, kernel[0], kernel[1], pads[0], pads[1], pads[2], pads[3],
                      strides[0], strides[1])
    L.sync()
    L.set_batch(1)
    return out.cpu().numpy(), xin.cpu().numpy()


def avgpool(x, kernel, strides, out_hw, pads=(0, 0, 0, 0), lam=0, shift=0, add=0, requant=0, bn_bits=32):
    B, H, W, Cc = x.shape
    Ho, Wo = out_hw
    L = nn(bn_bits)
    out = torch.full((B, Ho, Wo, Cc), 0xA5, dtype=torch.uint8, device="cuda")
    L.set_batch(B)
    L.pulp_nn_avgpool(dev(x), out, lam, shift, add, W, H, Cc, Wo, Ho, kernel[0], kernel[1], pads[0], pads[1],
                      pads[2], pads[3], strides[0], strides[1], requant)
    L.sync()
    L.set_batch(1)
    return out.cpu().numpy()


def add(a, b, m1, m2, shift, bn_bits=32):
    B, H, W, Cc = a.shape
    L = nn(bn_bits)
    out = torch.full(a.shape, 0xA5, dtype=torch.uint8, device="cuda")
    L.set_batch(B)
    L.pulp_nn_add(dev(a), dev(b), out, m1, m2, shift, H, W, Cc)
    L.sync()
    L.set_batch(1)
    return out.cpu().numpy()


def assert_same(got, want, what=""):
    got, want = np.asarray(got), np.asarray(want)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    bad = np.argwhere(got != want)
    if len(bad):
        i = tuple(bad[0])
        raise AssertionError("%s: %d of %d elements differ; first at %s: got %d want %d"
                             % (what, len(bad), got.size, i, int(got[i]), int(want[i])))
