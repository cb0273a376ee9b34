"""MI355X (gfx950) implementation of Euler's int8 convolution path -- Python binding of the C-ABI.

The compute lives in ``libeuler_hip.so`` (hand-written HIP kernels behind ``include/euler_hip.h``);
this module only loads it with ctypes and mirrors the descriptor of ``eld_conv_t`` so that tests and
benchmarks read like the reference's harness: fill a descriptor, ``setup()``, then ``execute()``.
Device memory and streams come from the caller (torch tensors or raw device pointers).

There is no CPU fallback: if the library is missing or fails to load, importing this package
raises.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("EULER_HIP_LIB") or os.path.join(_HERE, "libeuler_hip.so")

# ---- enum values of include/euler_hip.h (== the reference's include/euler.hpp) -----------------
EHIP_OK, EHIP_UNIMPLEMENTED, EHIP_GENERAL_ERROR, EHIP_HIP_ERROR = 0, 1, 2, 3
F32, F16, U8, S8, S32 = 1, 2, 3, 4, 5
CONV_AUTO, CONV_DIRECT_1X1, CONV_DIRECT, CONV_WINOGRAD = 0, 1, 2, 4
NCHW, NHWC, NCHW16C, OIHW, OIHW16I16O, GOIHW = 1, 2, 3, 5, 7, 9
FINE, COARSE, CALIBRATED = 0, 1, 2
Q_WEIGHTS_S8, Q_SCALE, Q_SHIFT, Q_WSUM, Q_TINPUT_U8, Q_TOUTPUT_F32 = 1, 2, 3, 4, 5, 6
EL_NO_CALI = float(np.finfo(np.float32).max)
FLT_MAX = EL_NO_CALI

NP_DTYPE = {F32: np.float32, U8: np.uint8, S8: np.int8, S32: np.int32}


class ConvDesc(ctypes.Structure):
    """ehip_conv_desc_t"""
    _fields_ = [(k, ctypes.c_int32) for k in (
        "n", "g", "ic", "oc", "ih", "iw", "oh", "ow", "kh", "kw",
        "pad_l", "pad_r", "pad_t", "pad_b",
        "stride_h", "stride_w", "dilation_h", "dilation_w",
        "input_type", "weights_type", "output_type", "bias_type",
        "input_fmt", "weights_fmt", "output_fmt",
        "algorithm", "tile_size", "execution_mode",
        "with_relu", "with_bias", "with_ip_sum",
        "flatting_o", "flatting_t", "sampling_kind")] + [(k, ctypes.c_float) for k in (
        "input_scale", "input_z", "tinput_scale", "tinput_z", "output_scale", "output_z",
        "sum_scale", "sum_z", "relu_lower", "relu_upper")]


class EulerHipError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("euler_hip error %d: %s" % (code, msg))
        self.code = code


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "libeuler_hip.so is not built (%s); run `python -c 'import __graft_entry__ as g; g.build()'`" % LIB_PATH)
    # PyTorch-ROCm ships its own copy of the HIP runtime under the same SONAME as /opt/rocm's.  A
    # process must hold exactly one of them: importing torch first makes this library's dependency
    # resolve to the copy torch already loaded (the other order leaves torch without a GPU).
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    lib = ctypes.CDLL(LIB_PATH)
    vp, ci, sz, fl = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t, ctypes.c_float
    lib.ehip_last_error.restype = ctypes.c_char_p
    lib.ehip_conv_kernel_name.restype = ctypes.c_char_p
    lib.ehip_conv_kernel_name.argtypes = [vp]
    lib.ehip_init.argtypes = [ci]
    lib.ehip_conv_create.argtypes = [ctypes.POINTER(ConvDesc), ctypes.POINTER(vp)]
    lib.ehip_conv_destroy.argtypes = [vp]
    lib.ehip_conv_prepare.argtypes = [vp, vp, vp, vp]
    lib.ehip_conv_execute.argtypes = [vp, vp, vp, vp, vp, vp]
    lib.ehip_conv_execute_repeat.argtypes = [vp, vp, vp, vp, ci, vp]
    lib.ehip_conv_execute_stages.argtypes = [vp, vp, vp, vp, ci, ci, vp]
    lib.ehip_conv_query.argtypes = [vp, ci, vp, ctypes.POINTER(sz)]
    lib.ehip_quantize_input_u8.argtypes = [vp, vp, sz, fl, fl, vp]
    lib.ehip_wino_tinput_range.argtypes = [ctypes.POINTER(ConvDesc), vp, ctypes.POINTER(fl), ctypes.POINTER(fl)]
    lib.ehip_wino_tinput_range_noalloc.argtypes = [ctypes.POINTER(ConvDesc), vp, vp, vp]
    lib.ehip_ref_conv_f32_range.argtypes = [ctypes.POINTER(ConvDesc), vp, vp, vp, vp, ctypes.POINTER(fl), ctypes.POINTER(fl)]
    lib.ehip_calibrate_output_quant.argtypes = [ctypes.POINTER(ConvDesc), fl, fl, fl, fl] + [ctypes.POINTER(fl)] * 3
    lib.ehip_reorder_nchw_to_blocked.argtypes = [vp, vp, ci, ci, ci, ci, ci, vp]
    lib.ehip_reorder_blocked_to_nchw.argtypes = [vp, vp, ci, ci, ci, ci, ci, vp]
    lib.ehip_reorder_oihw_to_blocked.argtypes = [vp, vp, ci, ci, ci, ci, vp]
    return lib


lib = _load()

EXPORTED_SYMBOLS = (
    "ehip_init", "ehip_last_error", "ehip_conv_create", "ehip_conv_destroy", "ehip_conv_prepare",
    "ehip_conv_execute", "ehip_conv_execute_repeat", "ehip_conv_execute_stages", "ehip_conv_query", "ehip_conv_kernel_name", "ehip_quantize_input_u8",
    "ehip_wino_tinput_range", "ehip_wino_tinput_range_noalloc", "ehip_reorder_nchw_to_blocked", "ehip_reorder_blocked_to_nchw",
    "ehip_reorder_oihw_to_blocked", "ehip_ref_conv_f32_range", "ehip_calibrate_output_quant",
)


def _check(rc):
    if rc != EHIP_OK:
        raise EulerHipError(rc, lib.ehip_last_error().decode(errors="replace"))


def _ptr(x):
    """device pointer of a torch tensor / int / None"""
    if x is None:
        return ctypes.c_void_p(0)
    if isinstance(x, int):
        return ctypes.c_void_p(x)
    return ctypes.c_void_p(x.data_ptr())


def up16(x):
    return (x + 15) // 16 * 16


def make_desc(n, ic, oc, ih, iw, kh=1, kw=1, pad=0, stride=1, g=1, algorithm=CONV_DIRECT,
              input_type=U8, output_type=U8, with_bias=True, with_relu=True, with_ip_sum=False,
              input_quant=(1.0 / 255.0, 0.0), output_quant=(1.0, 0.0), sum_quant=(0.0, 0.0),
              wino_tinput_quant=(EL_NO_CALI, EL_NO_CALI), relu_bound=(0.0, FLT_MAX), flatting_t=0,
              tile_size=0, execution_mode=0, weights_fmt=None, sampling_kind=CALIBRATED):
    """A descriptor for the common case (square kernel/pad/stride), filled the way the reference's
    harness fills eld_conv_t."""
    d = ConvDesc()
    d.n, d.g, d.ic, d.oc, d.ih, d.iw, d.kh, d.kw = n, g, ic, oc, ih, iw, kh, kw
    d.oh = (ih + 2 * pad - kh) // stride + 1
    d.ow = (iw + 2 * pad - kw) // stride + 1
    d.pad_l = d.pad_r = d.pad_t = d.pad_b = pad
    d.stride_h = d.stride_w = stride
    d.dilation_h = d.dilation_w = 1
    d.input_type, d.weights_type, d.output_type, d.bias_type = input_type, F32, output_type, F32
    d.input_fmt = d.output_fmt = NCHW16C
    d.weights_fmt = weights_fmt if weights_fmt is not None else (GOIHW if (g > 1 and g == ic == oc) else OIHW16I16O)
    d.algorithm, d.tile_size, d.execution_mode = algorithm, tile_size, execution_mode
    d.with_relu, d.with_bias, d.with_ip_sum = int(with_relu), int(with_bias), int(with_ip_sum)
    d.flatting_o, d.flatting_t = 0, flatting_t
    d.sampling_kind = sampling_kind
    d.input_scale, d.input_z = input_quant
    d.tinput_scale, d.tinput_z = wino_tinput_quant
    d.output_scale, d.output_z = output_quant
    d.sum_scale, d.sum_z = sum_quant
    d.relu_lower, d.relu_upper = relu_bound
    return d


class Conv:
    """One convolution layer on the GPU: setup (ehip_conv_create), first-run weight preparation
    (ehip_conv_prepare) and execute (ehip_conv_execute), all through the C-ABI."""

    def __init__(self, desc):
        self.desc = desc
        h = ctypes.c_void_p()
        _check(lib.ehip_conv_create(ctypes.byref(desc), ctypes.byref(h)))
        self._h = h

    def close(self):
        if getattr(self, "_h", None) and lib is not None:
            lib.ehip_conv_destroy(self._h)
            self._h = None

    __del__ = close

    @property
    def kernel_name(self):
        return lib.ehip_conv_kernel_name(self._h).decode()

    def prepare(self, weights, bias=None, stream=0):
        _check(lib.ehip_conv_prepare(self._h, _ptr(weights), _ptr(bias), ctypes.c_void_p(stream)))

    def execute(self, output, input, weights=None, bias=None, stream=0):
        _check(lib.ehip_conv_execute(self._h, _ptr(output), _ptr(input), _ptr(weights), _ptr(bias),
                                     ctypes.c_void_p(stream)))

    def execute_repeat(self, output, input, count, bias=None, stream=0):
        _check(lib.ehip_conv_execute_repeat(self._h, _ptr(output), _ptr(input), _ptr(bias), count,
                                            ctypes.c_void_p(stream)))

    def execute_stages(self, output, input, stages, count=1, bias=None, stream=0):
        """stages of a Winograd layer on their own: mask of 1 (input transform), 2 (GEMMs, fused: + output
        transform), 4 (stand-alone output transform)"""
        _check(lib.ehip_conv_execute_stages(self._h, _ptr(output), _ptr(input), _ptr(bias), stages, count,
                                            ctypes.c_void_p(stream)))

    def query(self, what):
        d = self.desc
        n = ctypes.c_size_t()
        _check(lib.ehip_conv_query(self._h, what, None, ctypes.byref(n)))
        dtype = {Q_WEIGHTS_S8: np.int8, Q_SCALE: np.float32, Q_SHIFT: np.float32, Q_WSUM: np.int32,
                 Q_TINPUT_U8: np.uint8, Q_TOUTPUT_F32: np.float32}[what]
        buf = np.zeros(n.value // np.dtype(dtype).itemsize, dtype)
        _check(lib.ehip_conv_query(self._h, what, ctypes.c_void_p(buf.ctypes.data), ctypes.byref(n)))
        return buf


def quantize_input_u8(dst, src, count, scale, z, stream=0):
    _check(lib.ehip_quantize_input_u8(_ptr(dst), _ptr(src), count, scale, z, ctypes.c_void_p(stream)))


def wino_tinput_range(desc, input):
    mn, mx = ctypes.c_float(), ctypes.c_float()
    _check(lib.ehip_wino_tinput_range(ctypes.byref(desc), _ptr(input), ctypes.byref(mn), ctypes.byref(mx)))
    return mn.value, mx.value


def wino_tinput_range_noalloc(desc, input, minmax_out, stream=0):
    """min / max into two floats of device memory (minmax_out), asynchronous, no device allocation"""
    _check(lib.ehip_wino_tinput_range_noalloc(ctypes.byref(desc), _ptr(input), _ptr(minmax_out), ctypes.c_void_p(stream)))


def ref_conv_f32_range(desc, input_f32, weights, bias, output_f32=None):
    """The harness's fp32 reference convolution on the device: (min, max) of its result; output_f32 (optional,
    required with with_ip_sum: it holds the sum operand) receives the result itself."""
    mn, mx = ctypes.c_float(), ctypes.c_float()
    _check(lib.ehip_ref_conv_f32_range(ctypes.byref(desc), _ptr(output_f32), _ptr(input_f32), _ptr(weights), _ptr(bias),
                                       ctypes.byref(mn), ctypes.byref(mx)))
    return mn.value, mx.value


def calibrate_output_quant(desc, out_min, out_max, sum_absmax=0.0, representation=127.0):
    """(output scale, output z, sum scale) from the range of the fp32 reference output, by the harness's rule"""
    s, z, ss = ctypes.c_float(), ctypes.c_float(), ctypes.c_float()
    _check(lib.ehip_calibrate_output_quant(ctypes.byref(desc), out_min, out_max, sum_absmax, representation,
                                           ctypes.byref(s), ctypes.byref(z), ctypes.byref(ss)))
    return s.value, z.value, ss.value


def reorder_nchw_to_blocked(dst, src, elem_size, n, c, h, w, stream=0):
    _check(lib.ehip_reorder_nchw_to_blocked(_ptr(dst), _ptr(src), elem_size, n, c, h, w, ctypes.c_void_p(stream)))


def reorder_blocked_to_nchw(dst, src, elem_size, n, c, h, w, stream=0):
    _check(lib.ehip_reorder_blocked_to_nchw(_ptr(dst), _ptr(src), elem_size, n, c, h, w, ctypes.c_void_p(stream)))


def reorder_oihw_to_blocked(dst, src, o, i, h, w, stream=0):
    _check(lib.ehip_reorder_oihw_to_blocked(_ptr(dst), _ptr(src), o, i, h, w, ctypes.c_void_p(stream)))
