"""ctypes binding of libpulpnn_hip{32,64}.so (the C ABI declared in include/)."""
import ctypes as C
import os

from .build import lib_path

_U16, _I8, _INT, _PTR = C.c_uint16, C.c_int8, C.c_int, C.c_void_p

_CONV_ARGS = [_PTR] * 7 + [_U16] * 16 + [_INT, _INT]


class HipBlock(C.Structure):
    """pulp_nn_hip_block of include/pulp_nn_hip.h: the parameters of one depthwise + pointwise block."""
    _fields_ = [("dw_wt", _PTR), ("dw_bias", _PTR), ("dw_k", _PTR), ("dw_lambda", _PTR),
                ("dw_out_mult", _U16), ("dw_out_shift", _U16), ("dw_flag_relu", _I8), ("dw_flag_batch_norm", _I8),
                ("pw_weight", _PTR), ("pw_bias", _PTR), ("pw_k", _PTR), ("pw_lambda", _PTR),
                ("pw_out_mult", _U16), ("pw_out_shift", _U16), ("pw_flag_relu", _I8), ("pw_flag_batch_norm", _I8)]

_DW_ARGS = [_PTR] * 8 + [_U16] * 16 + [_I8, _I8]

CONV_NAMES = ("pulp_nn_conv_Ho_parallel", "pulp_nn_conv_Co_parallel", "pulp_nn_conv_HoWo_parallel",
              "pulp_nn_pointwise_HoWo_parallel", "pulp_nn_pointwise_Ho_parallel", "pulp_nn_pointwise_Co_parallel")
DW_NAMES = ("pulp_nn_depthwise_generic", "pulp_nn_depthwise_generic_less_4_weights")

ERRORS = {0: "ok", 1: "argument", 2: "unsupported", 3: "runtime"}


class PulpNNError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("%s (%s)" % (msg, ERRORS.get(code, code)))
        self.code = code


def _ptr(x):
    """torch tensor / int / None -> device address."""
    if x is None:
        return None
    if isinstance(x, int):
        return x
    if not x.is_cuda:
        raise ValueError("PULP-NN HIP kernels take device tensors")
    if not x.is_contiguous():
        raise ValueError("tensor must be contiguous")
    return x.data_ptr()


class PulpNN:
    """One loaded library (32- or 64-bit batch-norm parameters).

    With check=True (default) every layer call raises PulpNNError if the library
    rejected it; the C functions themselves return void like the reference's."""

    def __init__(self, bn_bits=32, check=True):
        if bn_bits not in (32, 64):
            raise ValueError("bn_bits must be 32 or 64")
        path = lib_path(bn_bits)
        if not os.path.exists(path):
            raise ImportError("%s is missing: build it with `python -m pulp_nn_amd.build` "
                              "(there is no CPU fallback)" % path)
        self.bn_bits = bn_bits
        self.check = check
        self.path = path
        L = self._lib = C.CDLL(path)
        bn_scalar = C.c_int64 if bn_bits == 64 else C.c_int32
        for n in CONV_NAMES:
            getattr(L, n).argtypes, getattr(L, n).restype = _CONV_ARGS, None
        for n in DW_NAMES:
            getattr(L, n).argtypes, getattr(L, n).restype = _DW_ARGS, None
        L.pulp_nn_linear.argtypes = [_PTR] * 6 + [_U16, _I8, _U16, _U16, _INT, _INT]
        L.pulp_nn_linear.restype = None
        L.pulp_nn_linear_out_32.argtypes = [_PTR] * 4 + [_U16, _U16]
        L.pulp_nn_linear_out_32.restype = None
        L.pulp_nn_matmul.argtypes = [_PTR, _PTR, _U16, _U16, _U16, _U16, _PTR, _PTR, _PTR, _PTR, _PTR, _INT, _INT]
        L.pulp_nn_matmul.restype = _PTR
        L.pulp_nn_maxpool.argtypes = [_PTR, _PTR] + [_U16] * 13
        L.pulp_nn_maxpool.restype = None
        L.pulp_nn_avgpool.argtypes = [_PTR, _PTR, bn_scalar, _U16, bn_scalar] + [_U16] * 13 + [_INT]
        L.pulp_nn_avgpool.restype = None
        L.pulp_nn_add.argtypes = [_PTR] * 3 + [_U16] * 6
        L.pulp_nn_add.restype = None
        L.pulp_nn_depthwise_3x3_s1.argtypes = [_PTR, _PTR, _INT, _INT, _INT, _INT, _INT, _PTR, _I8, _U16, _PTR, _PTR,
                                               _INT, _INT, _PTR]
        L.pulp_nn_depthwise_3x3_s1.restype = None
        L.pulp_nn_hip_set_batch.argtypes = [C.c_uint]
        L.pulp_nn_hip_get_batch.restype = C.c_uint
        L.pulp_nn_hip_set_stream.argtypes = [_PTR]
        L.pulp_nn_hip_get_stream.restype = _PTR
        L.pulp_nn_hip_sync.restype = _INT
        L.pulp_nn_hip_clock_probe.argtypes = [_PTR]
        L.pulp_nn_hip_clock_probe.restype = None
        L.pulp_nn_hip_last_error.restype = _INT
        L.pulp_nn_hip_last_error_string.restype = C.c_char_p
        L.pulp_nn_hip_bn_bits.restype = _INT
        L.pulp_nn_hip_hwc_to_chw.argtypes = [_PTR, _PTR] + [C.c_uint] * 5
        L.pulp_nn_hip_hwc_to_chw.restype = None
        L.pulp_nn_hip_depthwise_hwc.argtypes = [_PTR] * 6 + [_U16] * 8 + [_I8, _I8]
        L.pulp_nn_hip_depthwise_hwc.restype = None
        L.pulp_nn_hip_dw_pw_hwc.argtypes = ([_PTR] * 2 + [_U16] * 7 + [_PTR] * 4 + [_U16] * 2 + [_I8] * 2 + [_PTR] * 4 +
                                            [_U16] * 2 + [_I8] * 2)
        L.pulp_nn_hip_dw_pw_hwc.restype = None
        L.pulp_nn_hip_dw_pw_chain_hwc.argtypes = [_PTR] * 2 + [_U16] * 3 + [C.c_uint, C.POINTER(HipBlock)]
        L.pulp_nn_hip_dw_pw_chain_hwc.restype = None
        _U64 = C.c_uint64
        L.pulp_nn_hip_calib_workspace_bytes.argtypes, L.pulp_nn_hip_calib_workspace_bytes.restype = [_U64], _U64
        L.pulp_nn_hip_calib_conv.argtypes = [_PTR] * 4 + [_U16] * 12 + [_PTR, _U64, _PTR]
        L.pulp_nn_hip_calib_conv.restype = None
        L.pulp_nn_hip_calib_depthwise.argtypes = [_PTR] * 4 + [_U16] * 11 + [_INT, _PTR, _U64, _PTR]
        L.pulp_nn_hip_calib_depthwise.restype = None
        L.pulp_nn_hip_calib_conv_static.argtypes = [_PTR] * 4 + [_U16] * 12 + [_PTR]
        L.pulp_nn_hip_calib_conv_static.restype = None
        assert L.pulp_nn_hip_bn_bits() == bn_bits

    # -- added entry points ------------------------------------------------
    def set_batch(self, n):
        self._lib.pulp_nn_hip_set_batch(int(n))

    def get_batch(self):
        return int(self._lib.pulp_nn_hip_get_batch())

    def set_stream(self, stream):
        """stream: a torch.cuda.Stream, a raw hipStream_t address, or None (default stream)."""
        h = getattr(stream, "cuda_stream", stream)
        self._lib.pulp_nn_hip_set_stream(h if h else None)

    def use_torch_stream(self):
        import torch
        self.set_stream(torch.cuda.current_stream())

    def sync(self):
        rc = self._lib.pulp_nn_hip_sync()
        if rc:
            self._raise()

    def clock_probe(self, out):
        """Queues the 20 us clock probe; out: device tensor of two int64 (wall-clock ticks at 100 MHz, shader cycles)."""
        self._call("pulp_nn_hip_clock_probe", _ptr(out))

    def last_error(self):
        return int(self._lib.pulp_nn_hip_last_error())

    def last_error_string(self):
        return self._lib.pulp_nn_hip_last_error_string().decode()

    def clear_error(self):
        self._lib.pulp_nn_hip_clear_error()

    def _raise(self):
        code, msg = self.last_error(), self.last_error_string()
        self.clear_error()
        raise PulpNNError(code, msg)

    def _call(self, name, *args):
        res = getattr(self._lib, name)(*args)
        if self.check and self._lib.pulp_nn_hip_last_error():
            self._raise()
        return res

    def hwc_to_chw(self, x, out, dim_x, dim_y, ch, pad_top=0, pad_bottom=0):
        self._call("pulp_nn_hip_hwc_to_chw", _ptr(x), _ptr(out), dim_x, dim_y, ch, pad_top, pad_bottom)

    def depthwise_hwc(self, x, bias, out, wt, k, lam, out_mult, out_shift, dim_in_x, dim_in_y, ch, dim_out_x,
                      dim_out_y, stride, flag_relu, flag_batch_norm):
        """3x3 depthwise, padding 1, HWC in and out (the layout change fused in).  Raises
        PulpNNError (unsupported) for geometries without a fused kernel."""
        self._call("pulp_nn_hip_depthwise_hwc", _ptr(x), _ptr(bias), _ptr(out), _ptr(wt), _ptr(k), _ptr(lam), out_mult,
                   out_shift, dim_in_x, dim_in_y, ch, dim_out_x, dim_out_y, stride, flag_relu, flag_batch_norm)

    def dw_pw_hwc(self, x, out, dim_in_x, dim_in_y, ch, dim_out_x, dim_out_y, ch_out, stride, dw_wt, dw_bias, dw_k, dw_lam,
                  dw_mult, dw_shift, dw_relu, dw_bn, pw_w, pw_bias, pw_k, pw_lam, pw_mult, pw_shift, pw_relu, pw_bn):
        """3x3 depthwise (padding 1, HWC in) and the pointwise layer behind it in one launch.  Raises
        PulpNNError (unsupported) for geometries without a fused kernel."""
        self._call("pulp_nn_hip_dw_pw_hwc", _ptr(x), _ptr(out), dim_in_x, dim_in_y, ch, dim_out_x, dim_out_y, ch_out, stride,
                   _ptr(dw_wt), _ptr(dw_bias), _ptr(dw_k), _ptr(dw_lam), dw_mult, dw_shift, dw_relu, dw_bn,
                   _ptr(pw_w), _ptr(pw_bias), _ptr(pw_k), _ptr(pw_lam), pw_mult, pw_shift, pw_relu, pw_bn)

    def dw_pw_chain_hwc(self, x, out, dim_x, dim_y, ch, blocks):
        """Several depthwise + pointwise blocks of one shape (stride 1, ch channels throughout) in one launch.
        blocks: a list of tuples (dw_wt, dw_bias, dw_k, dw_lam, dw_mult, dw_shift, dw_relu, dw_bn, pw_w, pw_bias,
        pw_k, pw_lam, pw_mult, pw_shift, pw_relu, pw_bn), the arguments dw_pw_hwc takes per block.  Raises PulpNNError
        (unsupported) where the blocks cannot be chained."""
        arr = (HipBlock * len(blocks))()
        for dst, b in zip(arr, blocks):
            (dst.dw_wt, dst.dw_bias, dst.dw_k, dst.dw_lambda) = [_ptr(v) for v in b[0:4]]
            (dst.dw_out_mult, dst.dw_out_shift, dst.dw_flag_relu, dst.dw_flag_batch_norm) = b[4:8]
            (dst.pw_weight, dst.pw_bias, dst.pw_k, dst.pw_lambda) = [_ptr(v) for v in b[8:12]]
            (dst.pw_out_mult, dst.pw_out_shift, dst.pw_flag_relu, dst.pw_flag_batch_norm) = b[12:16]
        self._call("pulp_nn_hip_dw_pw_chain_hwc", _ptr(x), _ptr(out), dim_x, dim_y, ch, len(blocks), arr)

    # -- calibration ---------------------------------------------------------
    def calib_workspace_bytes(self, n_outputs):
        return int(self._lib.pulp_nn_hip_calib_workspace_bytes(int(n_outputs)))

    def calib_conv(self, x, bias, w, k, dim_in_x, dim_in_y, ch_in, dim_out_x, dim_out_y, ch_out, kx, ky, pad_top,
                   pad_left, stride_x, stride_y, workspace, workspace_bytes, result):
        """result (device, 2 x uint64) <- max |acc * k|, and the out_shift floor(log2(max)) - 7 derived from it."""
        self._call("pulp_nn_hip_calib_conv", _ptr(x), _ptr(bias), _ptr(w), _ptr(k), dim_in_x, dim_in_y, ch_in,
                   dim_out_x, dim_out_y, ch_out, kx, ky, pad_top, pad_left, stride_x, stride_y, _ptr(workspace),
                   int(workspace_bytes), _ptr(result))

    def calib_depthwise(self, x, bias, wt, k, dim_in_x, dim_in_y, ch, dim_out_x, dim_out_y, kx, ky, pad_top, pad_left,
                        stride_x, stride_y, input_is_hwc, workspace, workspace_bytes, result):
        self._call("pulp_nn_hip_calib_depthwise", _ptr(x), _ptr(bias), _ptr(wt), _ptr(k), dim_in_x, dim_in_y, ch,
                   dim_out_x, dim_out_y, kx, ky, pad_top, pad_left, stride_x, stride_y, int(input_is_hwc),
                   _ptr(workspace), int(workspace_bytes), _ptr(result))

    def calib_conv_static(self, x, bias, w, k, dim_in_x, dim_in_y, ch_in, dim_out_x, dim_out_y, ch_out, kx, ky,
                          pad_top, pad_left, stride_x, stride_y, result):
        """calib_conv without a workspace argument: the library's fixed scratch array holds the partial maxima."""
        self._call("pulp_nn_hip_calib_conv_static", _ptr(x), _ptr(bias), _ptr(w), _ptr(k), dim_in_x, dim_in_y, ch_in,
                   dim_out_x, dim_out_y, ch_out, kx, ky, pad_top, pad_left, stride_x, stride_y, _ptr(result))

    # -- the reference API ---------------------------------------------------
    def _conv(self, name, pIn, pIm2Col, bias, pOut, pWeight, k, lam, *scalars):
        assert len(scalars) == 18, "expected out_mult .. flag_batch_norm"
        self._call(name, _ptr(pIn), _ptr(pIm2Col), _ptr(bias), _ptr(pOut), _ptr(pWeight), _ptr(k), _ptr(lam),
                   *[int(s) & 0xFFFF for s in scalars[:16]], int(scalars[16]), int(scalars[17]))

    def _dw(self, name, Im_in, bufferC, bias, Im_out, wt, bufferB, k, lam, *scalars):
        assert len(scalars) == 18, "expected out_mult .. FLAG_BATCH_NORM"
        f8 = lambda v: ((int(v) + 128) & 0xFF) - 128
        self._call(name, _ptr(Im_in), _ptr(bufferC), _ptr(bias), _ptr(Im_out), _ptr(wt), _ptr(bufferB), _ptr(k),
                   _ptr(lam), *[int(s) & 0xFFFF for s in scalars[:16]], f8(scalars[16]), f8(scalars[17]))

    def pulp_nn_linear(self, pIn, bias, pOut, pWeights, k, lam, out_mult, out_shift, dim_vec, num_o_neurons,
                       flag_relu, flag_batch_norm):
        self._call("pulp_nn_linear", _ptr(pIn), _ptr(bias), _ptr(pOut), _ptr(pWeights), _ptr(k), _ptr(lam),
                   int(out_mult) & 0xFFFF, int(out_shift), int(dim_vec), int(num_o_neurons), int(flag_relu),
                   int(flag_batch_norm))

    def pulp_nn_linear_out_32(self, pIn, bias, pOut, pWeights, dim_vec, num_o_neurons):
        self._call("pulp_nn_linear_out_32", _ptr(pIn), _ptr(bias), _ptr(pOut), _ptr(pWeights), int(dim_vec),
                   int(num_o_neurons))

    def pulp_nn_matmul(self, pWeight, pIn, ch_out, num_col_im2col, out_shift, out_mult, k, lam, bias, pOut, pOut2,
                       flag_relu, flag_batch_norm):
        return self._call("pulp_nn_matmul", _ptr(pWeight), _ptr(pIn), int(ch_out), int(num_col_im2col),
                          int(out_shift) & 0xFFFF, int(out_mult) & 0xFFFF, _ptr(k), _ptr(lam), _ptr(bias), _ptr(pOut),
                          _ptr(pOut2), int(flag_relu), int(flag_batch_norm))

    def pulp_nn_maxpool(self, Im_in, Im_out, *scalars):
        assert len(scalars) == 13
        self._call("pulp_nn_maxpool", _ptr(Im_in), _ptr(Im_out), *[int(s) & 0xFFFF for s in scalars])

    def pulp_nn_avgpool(self, Im_in, Im_out, lam, out_shift, out_add, *scalars):
        assert len(scalars) == 14
        self._call("pulp_nn_avgpool", _ptr(Im_in), _ptr(Im_out), int(lam), int(out_shift) & 0xFFFF, int(out_add),
                   *[int(s) & 0xFFFF for s in scalars[:13]], int(scalars[13]))

    def pulp_nn_add(self, in1, in2, out, out_mult1, out_mult2, out_shift, dim_h, dim_w, ch):
        self._call("pulp_nn_add", _ptr(in1), _ptr(in2), _ptr(out), int(out_mult1) & 0xFFFF, int(out_mult2) & 0xFFFF,
                   int(out_shift) & 0xFFFF, int(dim_h), int(dim_w), int(ch))

    def pulp_nn_depthwise_3x3_s1(self, In_Img, Out_Img, R, C_, CH, p_l, p_r, Kernel, out_shift, out_mult, kappa, lam,
                                 flag_relu, flag_batch_norm, memory_chan=None):
        self._call("pulp_nn_depthwise_3x3_s1", _ptr(In_Img), _ptr(Out_Img), int(R), int(C_), int(CH), int(p_l),
                   int(p_r), _ptr(Kernel), int(out_shift), int(out_mult) & 0xFFFF, _ptr(kappa), _ptr(lam),
                   int(flag_relu), int(flag_batch_norm), _ptr(memory_chan))


def _make_forwarders():
    for n in CONV_NAMES:
        def f(self, *a, _n=n):
            return self._conv(_n, *a)
        f.__name__ = n
        setattr(PulpNN, n, f)
    for n in DW_NAMES:
        def f(self, *a, _n=n):
            return self._dw(_n, *a)
        f.__name__ = n
        setattr(PulpNN, n, f)


_make_forwarders()
