"""CPU oracle for the PULP-NN int8 kernels: numpy front end of libpulpnn_oracle.so.

TEST INFRASTRUCTURE ONLY.  Imported by tests/, by __graft_entry__.smoke() and by
bench.py's cpu_baseline leg, always as the checker or the timed baseline and
never by the shipped HIP path (pulp_nn_amd/).

Every wrapper takes and returns numpy arrays; ``bn_bits`` selects the 32-bit or
64-bit batch-norm parameter variant (the reference's 32bit/ and 64bit/ trees);
a leading batch dimension on the activations means that many images stored
back to back.  The restated reference file and lines are cited per function
in pulpnn_oracle.c.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_DIR = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_DIR, "libpulpnn_oracle.so")
_lib = None


def build(force=False):
    """Compile the oracle with gcc (a few seconds)."""
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-s", "-B", "-C", _DIR, "libpulpnn_oracle.so"])
    return _SO


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_SO)
        _lib.oracle_bn_quant_u8.restype = C.c_uint8
        _lib.oracle_bn_quant_u8.argtypes = [C.c_int32, C.c_int64, C.c_int64, C.c_int8, C.c_int]
        _lib.oracle_quant_u8.restype = C.c_uint8
        _lib.oracle_quant_u8.argtypes = [C.c_int32, C.c_int16, C.c_int8]
        _lib.oracle_add_quant_u8.restype = C.c_uint8
        _lib.oracle_add_quant_u8.argtypes = [C.c_uint8, C.c_uint8, C.c_int16, C.c_int16, C.c_int8]
        _lib.oracle_epilogue.restype = C.c_uint8
        _lib.oracle_epilogue.argtypes = [C.c_int32, C.c_int64, C.c_int64, C.c_uint16, C.c_int,
                                         C.c_int, C.c_int, C.c_int, C.c_int]
    return _lib


def default_threads():
    return max(1, min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "64"))))


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _bn(a, bn_bits):
    if a is None:
        return None
    return np.ascontiguousarray(a, dtype=np.int64 if bn_bits == 64 else np.int32)


def _u8(a):
    return np.ascontiguousarray(a, dtype=np.uint8)


def _s8(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.int8)


def _batched(x, nd):
    """Return (array with a leading batch dim, had_batch)."""
    x = _u8(x)
    if x.ndim == nd:
        return x[None], False
    assert x.ndim == nd + 1, x.shape
    return x, True


def _u16(v):
    return C.c_uint16(int(v) & 0xFFFF)


# -- scalar epilogue helpers ------------------------------------------------

def bn_quant_u8(phi, k, lam, d, bn_bits=32):
    return int(lib().oracle_bn_quant_u8(int(phi), int(k), int(lam), int(d), bn_bits))


def quant_u8(phi, m, d):
    m = int(m) & 0xFFFF
    m = m - 0x10000 if m >= 0x8000 else m
    return int(lib().oracle_quant_u8(int(phi), m, int(d)))


def add_quant_u8(p1, p2, m1, m2, d):
    f = lambda m: (int(m) & 0xFFFF) - (0x10000 if (int(m) & 0x8000) else 0)
    return int(lib().oracle_add_quant_u8(int(p1), int(p2), f(m1), f(m2), int(d)))


def epilogue(acc, k, lam, out_mult, out_shift, flag_relu, flag_bn, bn_bits=32, relu_eq1=True):
    return int(lib().oracle_epilogue(int(acc), int(k), int(lam), int(out_mult) & 0xFFFF, int(out_shift),
                                     int(flag_relu), int(flag_bn), bn_bits, 1 if relu_eq1 else 0))


# -- layers -----------------------------------------------------------------

def conv(x, w, bias, k, lam, out_mult, out_shift, pads, strides, flag_relu, flag_bn,
         bn_bits=32, out_hw=None, nthreads=None):
    """x: [B,]H,W,Ci u8; w: Co,ky,kx,Ci s8; pads=(top,bottom,left,right); strides=(sx,sy)."""
    xb, had = _batched(x, 3)
    w = _s8(w)
    B, H, W, Ci = xb.shape
    Co, ky, kx, _ = w.shape
    pt, pb, pl, pr = pads
    sx, sy = strides
    if out_hw is None:
        out_hw = ((H + pt + pb - ky) // sy + 1, (W + pl + pr - kx) // sx + 1)
    Ho, Wo = out_hw
    out = np.empty((B, Ho, Wo, Co), np.uint8)
    k, lam, bias = _bn(k, bn_bits), _bn(lam, bn_bits), _s8(bias)
    lib().oracle_conv(_p(xb), _p(bias), _p(out), _p(w), _p(k), _p(lam), _u16(out_mult), _u16(out_shift),
                      _u16(W), _u16(H), _u16(Ci), _u16(Wo), _u16(Ho), _u16(Co), _u16(kx), _u16(ky),
                      _u16(pt), _u16(pb), _u16(pl), _u16(pr), _u16(sx), _u16(sy),
                      C.c_int(flag_relu), C.c_int(flag_bn), C.c_int(bn_bits), C.c_int(B),
                      C.c_int(nthreads or default_threads()))
    return out if had else out[0]


def conv_acc(x, w, bias, pads, strides, out_hw=None, nthreads=None):
    xb, had = _batched(x, 3)
    w = _s8(w)
    B, H, W, Ci = xb.shape
    Co, ky, kx, _ = w.shape
    pt, pb, pl, pr = pads
    sx, sy = strides
    if out_hw is None:
        out_hw = ((H + pt + pb - ky) // sy + 1, (W + pl + pr - kx) // sx + 1)
    Ho, Wo = out_hw
    out = np.empty((B, Ho, Wo, Co), np.int32)
    bias = _s8(bias)
    lib().oracle_conv_acc(_p(xb), _p(bias), _p(out), _p(w), _u16(W), _u16(H), _u16(Ci), _u16(Wo), _u16(Ho),
                          _u16(Co), _u16(kx), _u16(ky), _u16(pt), _u16(pb), _u16(pl), _u16(pr),
                          _u16(sx), _u16(sy), C.c_int(B), C.c_int(nthreads or default_threads()))
    return out if had else out[0]


def pointwise(x, w, bias, k, lam, out_mult, out_shift, flag_relu, flag_bn, bn_bits=32,
              out_hw=None, nthreads=None):
    """x: [B,]H,W,Ci u8; w: Co,Ci (or Co,1,1,Ci) s8."""
    xb, had = _batched(x, 3)
    w = _s8(w).reshape(w.shape[0], -1)
    B, H, W, Ci = xb.shape
    Co = w.shape[0]
    Ho, Wo = out_hw or (H, W)
    out = np.empty((B, Ho, Wo, Co), np.uint8)
    k, lam, bias = _bn(k, bn_bits), _bn(lam, bn_bits), _s8(bias)
    lib().oracle_pointwise(_p(xb), _p(bias), _p(out), _p(w), _p(k), _p(lam), _u16(out_mult), _u16(out_shift),
                           _u16(W), _u16(H), _u16(Ci), _u16(Wo), _u16(Ho), _u16(Co),
                           C.c_int(flag_relu), C.c_int(flag_bn), C.c_int(bn_bits), C.c_int(B),
                           C.c_int(nthreads or default_threads()))
    return out if had else out[0]


def matmul(w, in2, bias, k, lam, out_mult, out_shift, flag_relu, flag_bn, bn_bits=32):
    """w: Co,K s8; in2: 2,K u8 -> (out0[Co], out1[Co])."""
    w, in2 = _s8(w), _u8(in2)
    Co, K = w.shape
    o0, o1 = np.empty(Co, np.uint8), np.empty(Co, np.uint8)
    k, lam, bias = _bn(k, bn_bits), _bn(lam, bn_bits), _s8(bias)
    lib().oracle_matmul(_p(w), _p(in2), _u16(Co), _u16(K), _u16(out_shift), _u16(out_mult), _p(k), _p(lam),
                        _p(bias), _p(o0), _p(o1), C.c_int(flag_relu), C.c_int(flag_bn), C.c_int(bn_bits))
    return o0, o1


def depthwise_3x3_s1(x, kernel, k, lam, out_mult, out_shift, p_l, p_r, flag_relu, flag_bn,
                     bn_bits=32, nthreads=None):
    """x: [B,]CH,R,C u8 (CHW, rows already padded); kernel: CH,3,3 s8 -> [B,]R-2,C,CH."""
    xb, had = _batched(x, 3)
    kernel = _s8(kernel)
    B, CH, R, Cw = xb.shape
    out = np.zeros((B, R - 2, Cw, CH), np.uint8)
    k, lam = _bn(k, bn_bits), _bn(lam, bn_bits)
    lib().oracle_depthwise_3x3_s1(_p(xb), _p(out), C.c_int(R), C.c_int(Cw), C.c_int(CH), C.c_int(p_l),
                                  C.c_int(p_r), _p(kernel), C.c_int8(out_shift), _u16(out_mult), _p(k), _p(lam),
                                  C.c_int(flag_relu), C.c_int(flag_bn), C.c_int(bn_bits), C.c_int(B),
                                  C.c_int(nthreads or default_threads()))
    return out if had else out[0]


def depthwise_generic(x, wt, bias, k, lam, out_mult, out_shift, pads, strides, flag_relu, flag_bn,
                      bn_bits=32, out_hw=None, nthreads=None):
    """x: [B,]CH,H,W u8 (CHW); wt: CH,ky,kx s8 -> [B,]Ho,Wo,CH (HWC)."""
    xb, had = _batched(x, 3)
    wt = _s8(wt)
    B, CH, H, W = xb.shape
    _, ky, kx = wt.shape
    pt, pb, pl, pr = pads
    sx, sy = strides
    if out_hw is None:
        out_hw = ((H + pt + pb - ky) // sy + 1, (W + pl + pr - kx) // sx + 1)
    Ho, Wo = out_hw
    out = np.empty((B, Ho, Wo, CH), np.uint8)
    k, lam, bias = _bn(k, bn_bits), _bn(lam, bn_bits), _s8(bias)
    f8 = lambda v: C.c_int8(((int(v) + 128) & 0xFF) - 128)
    lib().oracle_depthwise_generic(_p(xb), _p(bias), _p(out), _p(wt), _p(k), _p(lam), _u16(out_mult),
                                   _u16(out_shift), _u16(W), _u16(H), _u16(Wo), _u16(Ho), _u16(CH),
                                   _u16(kx), _u16(ky), _u16(pt), _u16(pb), _u16(pl), _u16(pr),
                                   _u16(sx), _u16(sy), f8(flag_relu), f8(flag_bn), C.c_int(bn_bits),
                                   C.c_int(B), C.c_int(nthreads or default_threads()))
    return out if had else out[0]


def linear(x, w, bias, k, lam, out_mult, out_shift, flag_relu, flag_bn, bn_bits=32, nthreads=None):
    """x: [B,]K u8; w: N,K s8 -> [B,]N u8."""
    xb, had = _batched(x, 1)
    w = _s8(w)
    B, K = xb.shape
    N = w.shape[0]
    out = np.empty((B, N), np.uint8)
    k, lam, bias = _bn(k, bn_bits), _bn(lam, bn_bits), _s8(bias)
    lib().oracle_linear(_p(xb), _p(bias), _p(out), _p(w), _p(k), _p(lam), _u16(out_mult), C.c_int8(out_shift),
                        _u16(K), _u16(N), C.c_int(flag_relu), C.c_int(flag_bn), C.c_int(bn_bits), C.c_int(B),
                        C.c_int(nthreads or default_threads()))
    return out if had else out[0]


def linear_out_32(x, w, bias32, nthreads=None):
    """x: [B,]K u8; w: N,K s8; bias32: N int32 or None -> [B,]N int32."""
    xb, had = _batched(x, 1)
    w = _s8(w)
    B, K = xb.shape
    N = w.shape[0]
    out = np.empty((B, N), np.int32)
    b = None if bias32 is None else np.ascontiguousarray(bias32, dtype=np.int32)
    lib().oracle_linear_out_32(_p(xb), _p(b), _p(out), _p(w), _u16(K), _u16(N), C.c_int(B),
                               C.c_int(nthreads or default_threads()))
    return out if had else out[0]


def maxpool(x, kernel, strides, pads=(0, 0, 0, 0), out_hw=None, clobber=False, nthreads=None):
    """x: [B,]H,W,C u8; kernel=(kx,ky); strides=(sx,sy); pads=(t,b,l,r).
    With clobber=True x itself is modified like the reference's Im_in."""
    xb, had = _batched(x, 3)
    if not clobber:
        xb = xb.copy()
    B, H, W, Cc = xb.shape
    kx, ky = kernel
    sx, sy = strides
    pt, pb, pl, pr = pads
    if out_hw is None:
        out_hw = (-(-(H + pt + pb - ky) // sy) + 1, -(-(W + pl + pr - kx) // sx) + 1)
    Ho, Wo = out_hw
    out = np.empty((B, Ho, Wo, Cc), np.uint8)
    lib().oracle_maxpool(_p(xb), _p(out), _u16(W), _u16(H), _u16(Cc), _u16(Wo), _u16(Ho), _u16(kx), _u16(ky),
                         _u16(pt), _u16(pb), _u16(pl), _u16(pr), _u16(sx), _u16(sy), C.c_int(1), C.c_int(B),
                         C.c_int(nthreads or default_threads()))
    return out if had else out[0]


def avgpool(x, kernel, strides, pads=(0, 0, 0, 0), out_hw=None, lam=0, out_shift=0, out_add=0,
            flag_requant=0, bn_bits=32, nthreads=None):
    xb, had = _batched(x, 3)
    B, H, W, Cc = xb.shape
    kx, ky = kernel
    sx, sy = strides
    pt, pb, pl, pr = pads
    if out_hw is None:
        out_hw = ((H + pt + pb - ky) // sy + 1, (W + pl + pr - kx) // sx + 1)
    Ho, Wo = out_hw
    out = np.empty((B, Ho, Wo, Cc), np.uint8)
    lib().oracle_avgpool(_p(xb), _p(out), C.c_int64(lam), _u16(out_shift), C.c_int64(out_add), _u16(W), _u16(H),
                         _u16(Cc), _u16(Wo), _u16(Ho), _u16(kx), _u16(ky), _u16(pt), _u16(pb), _u16(pl),
                         _u16(pr), _u16(sx), _u16(sy), C.c_int(flag_requant), C.c_int(bn_bits), C.c_int(B),
                         C.c_int(nthreads or default_threads()))
    return out if had else out[0]


def add(a, b, m1, m2, out_shift, nthreads=None):
    a, b = _u8(a), _u8(b)
    assert a.shape == b.shape
    shp = a.shape
    out = np.empty(shp, np.uint8)
    n = a.size
    # flat call: H*W*C*batch elements, expressed as batch x (1,1,chunk) within uint16 limits
    chunk = 1
    for c in (32768, 16384, 4096, 1024, 256, 64, 16, 4, 2, 1):
        if n % c == 0:
            chunk = c
            break
    lib().oracle_add(_p(a), _p(b), _p(out), _u16(m1), _u16(m2), _u16(out_shift), _u16(1), _u16(1), _u16(chunk),
                     C.c_int(n // chunk), C.c_int(nthreads or default_threads()))
    return out
