"""ctypes bindings for the CPU oracle (oracle/libeuler_oracle.so) and, where it was built, the
reference's own compiled micro-kernels (oracle/_ref/libeuler_ref_kernels.so).

Test infrastructure only: nothing in the product package imports this module.
"""
import ctypes
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
ORACLE_SO = os.path.join(ORACLE_DIR, "libeuler_oracle.so")
REF_SO = os.path.join(ORACLE_DIR, "_ref", "libeuler_ref_kernels.so")
REF_GLUE_SO = os.path.join(ORACLE_DIR, "_ref", "libeuler_ref_wino_glue.so")
REF_HARNESS_SO = os.path.join(ORACLE_DIR, "_ref", "libeuler_ref_harness.so")

F32, U8, S8, S32 = 1, 3, 4, 5
NP_OF = {F32: np.float32, U8: np.uint8, S8: np.int8, S32: np.int32}


class ConvParams(ctypes.Structure):
    _fields_ = [(k, ctypes.c_int32) for k in (
        "n", "g", "ic", "oc", "ih", "iw", "oh", "ow", "kh", "kw",
        "pad_t", "pad_l", "stride_h", "stride_w", "out_type",
        "with_bias", "with_relu", "with_sum", "T")] + [(k, ctypes.c_float) for k in (
        "in_scale", "in_z", "out_scale", "out_z", "sum_scale", "sum_z",
        "tin_scale", "tin_z", "relu_lo", "relu_hi")] + [("wino_tile", ctypes.c_int32)]


FLT_MAX = float(np.finfo(np.float32).max)


def make_params(n, ic, oc, ih, iw, kh=1, kw=1, pad=0, stride=1, g=1, out_type=U8, with_bias=True,
                with_relu=True, with_sum=False, T=0, in_scale=1.0 / 255.0, in_z=0.0, out_scale=1.0,
                out_z=0.0, sum_scale=0.0, sum_z=0.0, tin_scale=1.0, tin_z=0.0, relu_lo=0.0,
                relu_hi=FLT_MAX, pad_tl=None, out_hw=None, wino_tile=0):
    """pad: on every side; pad_tl / out_hw: top-left pad and output size given separately (the right and
    bottom pads are then whatever the output size implies, src/elx_conv.cpp:36-37)"""
    oh = (ih + 2 * pad - kh) // stride + 1
    ow = (iw + 2 * pad - kw) // stride + 1
    if out_hw is not None:
        oh, ow = out_hw
    p = ConvParams()
    p.n, p.g, p.ic, p.oc, p.ih, p.iw, p.oh, p.ow, p.kh, p.kw = n, g, ic, oc, ih, iw, oh, ow, kh, kw
    p.pad_t = p.pad_l = pad if pad_tl is None else pad_tl
    p.stride_h = p.stride_w = stride
    p.out_type, p.with_bias, p.with_relu, p.with_sum, p.T = out_type, int(with_bias), int(with_relu), int(with_sum), T
    p.in_scale, p.in_z, p.out_scale, p.out_z = in_scale, in_z, out_scale, out_z
    p.sum_scale, p.sum_z, p.tin_scale, p.tin_z = sum_scale, sum_z, tin_scale, tin_z
    p.relu_lo, p.relu_hi = relu_lo, relu_hi
    p.wino_tile = wino_tile   # Winograd tile size A (0 / 6, 4 or 5)
    return p


def aligned(shape, dtype, fill=None):
    """numpy array whose data pointer is 64-byte aligned (the reference kernels use aligned moves)."""
    dtype = np.dtype(dtype)
    n = int(np.prod(shape)) if np.ndim(shape) else int(shape)
    raw = np.zeros(n * dtype.itemsize + 64, np.uint8)
    off = (-raw.ctypes.data) % 64
    a = raw[off:off + n * dtype.itemsize].view(dtype).reshape(shape)
    if fill is not None:
        a[...] = fill
    return a


def ptr(a):
    return ctypes.c_void_p(a.ctypes.data) if a is not None else ctypes.c_void_p(0)


_oracle = None
_ref = None
_ref_glue = None


def oracle():
    global _oracle
    if _oracle is None:
        if not os.path.exists(ORACLE_SO):
            subprocess.check_call(["make", "-C", ORACLE_DIR, "oracle"])
        lib = ctypes.CDLL(ORACLE_SO)
        lib.orc_quantize_input_u8.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t,
                                              ctypes.c_float, ctypes.c_float]
        lib.orc_wino_tile_input_a.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
        lib.orc_wino_tile_weights_a.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
        lib.orc_wino_tile_output_a.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
        lib.orc_wino_output_value_a.argtypes = [ctypes.c_int, ctypes.c_float, ctypes.c_int, ctypes.c_float, ctypes.c_int,
                                                ctypes.c_float, ctypes.c_float, ctypes.c_int,
                                                ctypes.POINTER(ctypes.c_float)]
        lib.orc_wino_output_value_sum.argtypes = [ctypes.c_int, ctypes.c_float, ctypes.c_int, ctypes.c_float, ctypes.c_int,
                                                  ctypes.c_float, ctypes.c_float, ctypes.c_int, ctypes.c_int,
                                                  ctypes.c_float, ctypes.POINTER(ctypes.c_float)]
        lib.orc_epilogue.argtypes = [ctypes.c_int, ctypes.c_int32, ctypes.c_float, ctypes.c_float, ctypes.c_int,
                                     ctypes.c_int, ctypes.c_float, ctypes.c_int, ctypes.c_float, ctypes.c_float,
                                     ctypes.POINTER(ctypes.c_float)]
        lib.orc_calibrate_output_quant.argtypes = [ctypes.c_int] * 3 + [ctypes.c_float] * 4 + [ctypes.POINTER(ctypes.c_float)] * 3
        lib.orc_calibrate_output_quant.restype = None
        _oracle = lib
    return _oracle


def ref_kernels():
    """The reference's compiled kernel templates, or None where oracle/_ref was not built
    (it needs /root/reference and an AVX-512-VNNI host)."""
    global _ref
    if _ref is None:
        if not os.path.exists(REF_SO):
            return None
        try:
            flags = open("/proc/cpuinfo").read()
        except OSError:
            flags = ""
        if "avx512_vnni" not in flags or "avx512bw" not in flags:
            return None
        lib = ctypes.CDLL(REF_SO)
        fl = ctypes.c_float
        ci = ctypes.c_int
        vp = ctypes.c_void_p
        lib.ref_u8s8_gemm.argtypes = [ci, ci, ci, ci, ci, fl, fl, fl, vp, vp, vp, vp, vp, vp]
        lib.ref_u8s8_depthwise.argtypes = [ci] * 14 + [fl, fl, vp, vp, vp, vp, vp]
        lib.ref_u8s8_conv3x3.argtypes = [ci] * 11 + [fl, fl, vp, vp, vp, vp, vp, vp]
        if hasattr(lib, "ref_u8s8_convk"):
            lib.ref_u8s8_convk.argtypes = [ci] * 13 + [fl, fl, vp, vp, vp, vp, vp, vp]
        if hasattr(lib, "ref_u8s8_conv3x3_s2"):
            lib.ref_u8s8_conv3x3_s2.argtypes = [ci] * 13 + [fl, fl, vp, vp, vp, vp, vp, vp]
            lib.ref_u8s8_depthwise_s2.argtypes = [ci] * 14 + [fl, fl, vp, vp, vp, vp, vp]
        lib.ref_wino_trans_input.argtypes = [ci, ci, ci, vp, vp, ci, ci, ci, ci]
        lib.ref_wino_trans_weights.argtypes = [vp, vp]
        lib.ref_wino_trans_output.argtypes = [ci, ci, ci, ci, ci, vp, vp, vp, ci, ci]
        if hasattr(lib, "ref_wino_trans_output_q"):
            lib.ref_wino_trans_output_q.argtypes = [ci, ci, ci, ci, ci, ci, vp, vp, vp, ci, ci, fl, fl]
        if hasattr(lib, "ref_wino_trans_input_a"):
            lib.ref_wino_trans_input_a.argtypes = [ci, ci, ci, ci, vp, vp, ci, ci, ci, ci]
            lib.ref_wino_trans_weights_a.argtypes = [ci, vp, vp]
            lib.ref_wino_trans_output_a.argtypes = [ci, ci, ci, ci, ci, ci, ci, vp, vp, vp, ci, ci, fl, fl]
        if hasattr(lib, "ref_wino_trans_output_sum"):
            lib.ref_wino_trans_output_sum.argtypes = [ci, ci, ci, ci, ci, ci, ci, vp, vp, vp, ci, ci, fl, fl]
        _ref = lib
    return _ref


def ref_wino_glue():
    """The reference's Winograd input / weight transform classes with their quantization glue
    (src/elx_conv_wino_trans_input.cpp, src/elx_conv_wino_trans_weights.cpp compiled from the reference
    tree by oracle/Makefile), or None where oracle/_ref was not built or the host lacks AVX-512."""
    global _ref_glue
    if _ref_glue is None:
        if not os.path.exists(REF_GLUE_SO):
            return None
        try:
            flags = open("/proc/cpuinfo").read()
        except OSError:
            flags = ""
        if "avx512_vnni" not in flags or "avx512bw" not in flags:
            return None
        lib = ctypes.CDLL(REF_GLUE_SO)
        fl, ci, vp = ctypes.c_float, ctypes.c_int, ctypes.c_void_p
        lib.ref_wino_glue_trans_input.argtypes = [ci] * 11 + [fl, fl, fl, vp, vp]
        lib.ref_wino_glue_trans_input_f32.argtypes = [ci] * 10 + [vp, vp]
        lib.ref_wino_glue_trans_weights.argtypes = [ci, ci, ci, fl, fl, vp, vp, vp, vp]
        _ref_glue = lib
    return _ref_glue


def ref_harness():
    """The reference's test harness (tests/elt_conv_utils.cpp: fp32 reference convolution, scale calibration,
    input quantization) compiled from the reference tree by oracle/Makefile, or None where oracle/_ref was
    not built or the host lacks AVX-512."""
    global _ref_harness
    if _ref_harness is None:
        if not os.path.exists(REF_HARNESS_SO):
            return None
        try:
            flags = open("/proc/cpuinfo").read()
        except OSError:
            flags = ""
        if "avx512_vnni" not in flags or "avx512bw" not in flags:
            return None
        # The harness unit calls the executor library in one place (elx_conv, for Winograd calibration), which
        # is not built here and which nothing below reaches: bind lazily, so that the unresolved function
        # does not stop the load (ctypes itself always asks for immediate binding).
        dl = ctypes.CDLL(None)
        dl.dlopen.restype = ctypes.c_void_p
        dl.dlopen.argtypes = [ctypes.c_char_p, ctypes.c_int]
        handle = dl.dlopen(REF_HARNESS_SO.encode(), os.RTLD_LAZY | os.RTLD_LOCAL)
        if not handle:
            return None
        lib = ctypes.CDLL(REF_HARNESS_SO, handle=handle)
        ci, vp = ctypes.c_int, ctypes.c_void_p
        lib.ref_harness_conv2d.argtypes = [ci] * 17 + [vp] * 4
        lib.ref_harness_prepare.argtypes = [ci] * 18 + [vp] * 7
        _ref_harness = lib
    return _ref_harness


_ref_harness = None


# --------------------------------------------------------------------------------------------
# numpy-level wrappers
# --------------------------------------------------------------------------------------------
def ref_conv_f32(p, x_nchw, w_goihw, bias, out_init=None):
    """the harness's fp32 reference convolution on plain tensors (out_init: the sum operand)"""
    out = np.zeros((p.n, p.oc, p.oh, p.ow), np.float32)
    if out_init is not None:
        out[...] = out_init
    x_nchw, w_goihw, bias = (np.ascontiguousarray(a, np.float32) for a in (x_nchw, w_goihw, bias))
    assert oracle().orc_ref_conv_f32(ctypes.byref(p), ptr(out), ptr(x_nchw), ptr(w_goihw), ptr(bias)) == 0
    return out


def calibrate_output_quant(with_relu, out_type, with_sum, out_min, out_max, sum_absmax, representation):
    """(output scale, output z, sum scale) by the harness's rule"""
    s, z, ss = ctypes.c_float(), ctypes.c_float(), ctypes.c_float()
    oracle().orc_calibrate_output_quant(int(with_relu), int(out_type), int(with_sum), float(out_min), float(out_max),
                                        float(sum_absmax), float(representation), ctypes.byref(s), ctypes.byref(z),
                                        ctypes.byref(ss))
    return s.value, z.value, ss.value


def up16(x):
    return (x + 15) // 16 * 16


def to_blocked(x):
    """nchw -> nChw16c (zero-filled channel tail)"""
    n, c, h, w = x.shape
    C = up16(c)
    xp = np.zeros((n, C, h, w), x.dtype)
    xp[:, :c] = x
    return np.ascontiguousarray(xp.reshape(n, C // 16, 16, h, w).transpose(0, 1, 3, 4, 2))


def from_blocked(xb, c):
    n, c2, h, w, _ = xb.shape
    return np.ascontiguousarray(xb.transpose(0, 1, 4, 2, 3).reshape(n, c2 * 16, h, w)[:, :c])


def blocked_to_nhwc(xb, c):
    """nChw16c -> nhwc = [n][h][w][c] (the reference indexes it as [n*h*w][c],
    src/elx_int8_conv_direct_1x1.cpp:417-425)"""
    n, c2, h, w, _ = xb.shape
    return np.ascontiguousarray(xb.transpose(0, 2, 3, 1, 4).reshape(n, h, w, c2 * 16)[..., :c])


def weights_to_blocked(wt):
    """oihw -> OIhw16i16o"""
    o, i, kh, kw = wt.shape
    O, I = up16(o), up16(i)
    wp = np.zeros((O, I, kh, kw), wt.dtype)
    wp[:o, :i] = wt
    return np.ascontiguousarray(wp.reshape(O // 16, 16, I // 16, 16, kh, kw).transpose(0, 2, 4, 5, 3, 1))


def direct_prepare(p, w_blocked, bias):
    OCp, ICp = up16(p.oc), up16(p.ic)
    wq = np.zeros((OCp, ICp, p.kh, p.kw), np.int8)
    scale = np.zeros(OCp, np.float32)
    shift = np.zeros(OCp, np.float32)
    wsum = np.zeros(OCp, np.int32)
    rc = oracle().orc_direct_prepare(ctypes.byref(p), ptr(w_blocked), ptr(bias), ptr(wq), ptr(scale), ptr(shift),
                                     ptr(wsum))
    assert rc == 0
    return wq, scale, shift, wsum


def direct_execute(p, x_blocked, wq, scale, shift, out_init=None):
    OC2 = up16(p.oc) // 16
    out = np.zeros((p.n, OC2, p.oh, p.ow, 16), NP_OF[p.out_type])
    if out_init is not None:
        out[...] = out_init
    acc = np.zeros((p.n, OC2, p.oh, p.ow, 16), np.int32)
    rc = oracle().orc_direct_execute(ctypes.byref(p), ptr(x_blocked), ptr(wq), ptr(scale), ptr(shift), ptr(out),
                                     ptr(acc))
    assert rc == 0
    return out, acc


def direct_execute_border(p, x_blocked, w_blocked, bias, wq, scale):
    """non-zero input zero point with padding: per-pixel shift (sum of the weights of the valid taps)"""
    OCp = up16(p.oc)
    smap = np.zeros((p.oh, p.ow, OCp), np.float32)
    assert oracle().orc_direct_border_shifts(ctypes.byref(p), ptr(w_blocked), ptr(bias), ptr(smap)) == 0
    out = np.zeros((p.n, OCp // 16, p.oh, p.ow, 16), NP_OF[p.out_type])
    acc = np.zeros((p.n, OCp // 16, p.oh, p.ow, 16), np.int32)
    assert oracle().orc_direct_execute_border(ctypes.byref(p), ptr(x_blocked), ptr(wq), ptr(scale), ptr(smap), ptr(out),
                                              ptr(acc)) == 0
    return out, acc, smap


def depthwise_prepare(p, w_goihw, bias):
    G = up16(p.g)
    wq = np.zeros((G, 3, 3), np.int8)
    scale = np.zeros(G, np.float32)
    shift = np.zeros(G, np.float32)
    wsum = np.zeros(G, np.int32)
    rc = oracle().orc_depthwise_prepare(ctypes.byref(p), ptr(w_goihw), ptr(bias), ptr(wq), ptr(scale), ptr(shift),
                                        ptr(wsum))
    assert rc == 0
    return wq, scale, shift, wsum


def depthwise_execute(p, x_blocked, wq, scale, shift):
    G2 = up16(p.g) // 16
    out = np.zeros((p.n, G2, p.oh, p.ow, 16), NP_OF[p.out_type])
    acc = np.zeros((p.n, G2, p.oh, p.ow, 16), np.int32)
    rc = oracle().orc_depthwise_execute(ctypes.byref(p), ptr(x_blocked), ptr(wq), ptr(scale), ptr(shift), ptr(out),
                                        ptr(acc))
    assert rc == 0
    return out, acc


def wino_tiles(p):
    return oracle().orc_wino_tiles(ctypes.byref(p))


def wino_tinput_range(p, x_blocked):
    mn, mx = ctypes.c_float(), ctypes.c_float()
    oracle().orc_wino_tinput_range(ctypes.byref(p), ptr(x_blocked), ctypes.byref(mn), ctypes.byref(mx))
    return mn.value, mx.value


def wino_positions(p):
    """A x A positions of the Winograd tile size the parameters ask for"""
    a = p.wino_tile if p.wino_tile in (4, 5) else 6
    return a * a


def wino_prepare(p, w_blocked):
    OCp, ICp = up16(p.oc), up16(p.ic)
    twq = np.zeros((wino_positions(p), OCp, ICp), np.int8)
    tscale = np.zeros((wino_positions(p), OCp), np.float32)
    tshift = np.zeros((wino_positions(p), OCp), np.float32)
    assert oracle().orc_wino_prepare(ctypes.byref(p), ptr(w_blocked), ptr(twq), ptr(tscale), ptr(tshift)) == 0
    return twq, tscale, tshift


def wino_trans_input(p, x_blocked):
    t = wino_tiles(p)
    tin = np.zeros((wino_positions(p), up16(p.ic) // 16, t, 16), np.uint8)
    assert oracle().orc_wino_trans_input(ctypes.byref(p), ptr(x_blocked), ptr(tin)) == 0
    return tin


def wino_gemm(p, tin, twq, tscale, tshift):
    t = wino_tiles(p)
    OC2 = up16(p.oc) // 16
    tout = np.zeros((wino_positions(p), OC2, t, 16), np.float32)
    acc = np.zeros((wino_positions(p), OC2, t, 16), np.int32)
    assert oracle().orc_wino_gemm(ctypes.byref(p), ptr(tin), ptr(twq), ptr(tscale), ptr(tshift), ptr(tout),
                                  ptr(acc)) == 0
    return tout, acc


def wino_trans_output(p, tout, bias, out_init=None):
    """out_init: the output tensor on entry (the sum operand when p.with_sum)"""
    out = np.zeros((p.n, up16(p.oc) // 16, p.oh, p.ow, 16), NP_OF[p.out_type])
    if out_init is not None:
        out[...] = out_init
    assert oracle().orc_wino_trans_output(ctypes.byref(p), ptr(tout), ptr(bias), ptr(out)) == 0
    return out


def quantize_input_u8(x, scale, z):
    x = np.ascontiguousarray(x, np.float32)
    out = np.zeros(x.shape, np.uint8)
    oracle().orc_quantize_input_u8(ptr(out), ptr(x), x.size, scale, z)
    return out
