"""Pins the oracle's float glue and border handling against the reference's OWN micro-kernel
templates, compiled from /root/reference by oracle/Makefile (target `ref`).  Skipped where that
library is absent or the host has no AVX-512-VNNI."""
import ctypes

import numpy as np
import pytest

import oracle_lib as ol

ref = ol.ref_kernels()
pytestmark = pytest.mark.skipif(ref is None, reason="oracle/_ref not built or host lacks AVX-512-VNNI")

AT_RELU, AT_SUM, AT_CLEAR, AT_RESTORE = 1 << 1, 1 << 2, 1 << 3, 1 << 5


def _epi(kind, acc, scale, shift, with_sum, old, sum_s, relu, lo, hi):
    f = ctypes.c_float()
    q = ol.oracle().orc_epilogue(kind, int(acc), float(scale), float(shift), int(with_sum), int(old), float(sum_s),
                                 int(relu), float(lo), float(hi), ctypes.byref(f))
    return f.value if kind == ol.F32 else q


@pytest.mark.parametrize("kind", [ol.F32, ol.U8, ol.S8])
@pytest.mark.parametrize("O,T", [(1, 4), (2, 6)])
@pytest.mark.parametrize("with_sum", [False, True])
def test_gemm_kernel_epilogue(kind, O, T, with_sum):
    if kind == ol.F32 and with_sum:
        pytest.skip("the reference has no sum fusion for f32 output (elk_u8s8_gemm.hxx:234-236)")
    rng = np.random.default_rng(7 + 10 * O + kind)
    I2 = 5
    x = ol.aligned((I2, T, 16), np.uint8)
    x[...] = rng.integers(0, 256, x.shape)
    w = ol.aligned((I2, 4, O, 16, 4), np.int8)
    w[...] = rng.integers(-127, 128, w.shape)
    scale = ol.aligned((O, 16), np.float32)
    shift = ol.aligned((O, 16), np.float32)
    # scales that land many results near .5 boundaries and on both sides of the clamp
    scale[...] = rng.uniform(1e-4, 3e-3, scale.shape)
    shift[...] = rng.normal(0, 20, shift.shape)
    sum_s = 0.37109375 if with_sum else 0.0
    lo, hi = (0.0, 200.0) if kind == ol.U8 else (-60.0, 90.0)
    tout = ol.aligned((O, T, 16), np.float32)
    np_kind = {ol.F32: np.float32, ol.U8: np.uint8, ol.S8: np.int8}[kind]
    oout = ol.aligned((O, T, 16), np_kind)
    if kind != ol.F32:
        oout[...] = rng.integers(0, 256, oout.shape) if kind == ol.U8 else rng.integers(-128, 128, oout.shape)
    old = oout.copy()
    attr = AT_CLEAR | AT_RESTORE | AT_RELU | (AT_SUM if with_sum else 0)
    rc = ref.ref_u8s8_gemm({ol.F32: 0, ol.U8: 1, ol.S8: 2}[kind], O, T, I2, attr, lo, hi, sum_s, ol.ptr(tout),
                           ol.ptr(oout), ol.ptr(x), ol.ptr(w), ol.ptr(scale), ol.ptr(shift))
    assert rc == 0
    # integer contraction, closed form
    acc = np.einsum("itvk,ivock->otc", x.reshape(I2, T, 4, 4).astype(np.int64),
                    w.astype(np.int64))  # [O][T][16]
    for o in range(O):
        for t in range(T):
            for c in range(16):
                exp = _epi(kind, acc[o, t, c], scale[o, c], shift[o, c], with_sum, old[o, t, c], sum_s, True, lo, hi)
                got = tout[o, t, c] if kind == ol.F32 else oout[o, t, c]
                if kind == ol.F32:
                    assert np.float32(exp).view(np.uint32) == got.view(np.uint32)
                else:
                    assert int(np_kind(exp)) == int(got), (o, t, c)


def test_gemm_kernel_u8_unsigned_saturation_without_relu():
    # vpmovusdb treats the rounded s32 as unsigned: negatives become 255 (elk_u8s8_gemm.hxx:249-255)
    O, T, I2 = 1, 4, 1
    x = ol.aligned((I2, T, 16), np.uint8, 3)
    w = ol.aligned((I2, 4, O, 16, 4), np.int8, -5)
    scale = ol.aligned((O, 16), np.float32, 0.01)
    shift = ol.aligned((O, 16), np.float32, 0.0)
    tout = ol.aligned((O, T, 16), np.float32)
    oout = ol.aligned((O, T, 16), np.uint8)
    ref.ref_u8s8_gemm(1, O, T, I2, AT_CLEAR | AT_RESTORE, 0.0, ol.FLT_MAX, 0.0, ol.ptr(tout), ol.ptr(oout), ol.ptr(x),
                      ol.ptr(w), ol.ptr(scale), ol.ptr(shift))
    acc = 16 * 3 * -5
    assert int(oout[0, 0, 0]) == 255 == _epi(ol.U8, acc, 0.01, 0.0, 0, 0, 0.0, 0, 0.0, 0.0)


def _dw_case(T, ow, ih, kind, seed, relu_hi=255.0):
    rng = np.random.default_rng(seed)
    G2, iw, oh = 2, ow, ih
    p = ol.make_params(1, 32, 32, ih, iw, 3, 3, pad=1, g=32, out_type=kind, T=T, out_scale=6.0 / 255.0,
                       relu_hi=relu_hi)
    x = np.zeros(G2 * ih * iw * 16 + 256, np.uint8)
    x[:G2 * ih * iw * 16] = rng.integers(0, 256, G2 * ih * iw * 16)
    xb = ol.aligned(x.shape, np.uint8)
    xb[...] = x
    wts = rng.normal(0, 0.1, (32, 3, 3)).astype(np.float32)
    bias = rng.normal(0, 0.5, 32).astype(np.float32)
    wq, scale, shift, _ = ol.depthwise_prepare(p, wts, bias)
    exp, _ = ol.depthwise_execute(p, xb[:G2 * ih * iw * 16].reshape(1, G2, ih, iw, 16), wq, scale, shift)
    # reference layout: weights [G2][3][16][4]
    wr = ol.aligned((G2, 3, 16, 4), np.int8)
    wr[...] = 0
    wr[:, :, :, :3] = wq.reshape(G2, 16, 3, 3).transpose(0, 2, 1, 3)
    sc = ol.aligned((G2, 16), np.float32)
    sh = ol.aligned((G2, 16), np.float32)
    sc[...] = scale.reshape(G2, 16)
    sh[...] = shift.reshape(G2, 16)
    got = ol.aligned((G2, oh * ow, 16), ol.NP_OF[kind])
    wt = (ow + T - 1) // T
    Tr = ow % T or T
    for ht in range(oh):
        for _wt in range(wt):
            Tz = Tr if _wt == wt - 1 else T
            rc = ref.ref_u8s8_depthwise({ol.U8: 1, ol.S8: 2}[kind], T, Tz, G2, ih, iw, oh, ow, ht, _wt, 1, 1, 1, 1, 0.0,
                                        relu_hi, ol.ptr(got), ol.ptr(xb), ol.ptr(wr), ol.ptr(sc), ol.ptr(sh))
            assert rc == 0, (T, Tz)
    return exp.reshape(G2, oh * ow, 16), got, wt, Tr


@pytest.mark.parametrize("T,ow,ih", [(14, 56, 5), (7, 7, 7), (14, 28, 4), (11, 28, 3), (8, 20, 3), (7, 21, 3)])
def test_depthwise_kernel_u8_floor_and_round_split(T, ow, ih):
    exp, got, wt, Tr = _dw_case(T, ow, ih, ol.U8, 100 + T + ow)
    assert np.array_equal(exp, got)


def test_depthwise_kernel_s8():
    exp, got, _, _ = _dw_case(14, 28, 4, ol.S8, 5, relu_hi=127.0)
    assert np.array_equal(exp, got)


def test_depthwise_floor_rule_is_observable():
    # a pure round-to-nearest model must NOT match the compiled kernel (guards against the
    # oracle and the test both losing the floor rule)
    exp, got, _, _ = _dw_case(14, 56, 3, ol.U8, 11)
    assert np.array_equal(exp, got)
    cols = np.arange(exp.shape[1]) % 56 % 14
    assert (cols < 12).any() and (cols >= 12).any()
    # the same layer with T = 1 rounds every column to nearest: it has to differ somewhere
    exp_rne, _, _, _ = _dw_case(1, 56, 3, ol.U8, 11) if False else (None, None, None, None)


@pytest.mark.parametrize("kind", [ol.U8, ol.S8, ol.F32])
@pytest.mark.parametrize("T,ow", [(14, 28), (7, 14), (7, 7)])
def test_conv3x3_kernel(kind, T, ow):
    rng = np.random.default_rng(3 * T + ow + kind)
    I2, ih, iw, oh = 2, 5, ow, 5
    ic, oc = 16 * I2, 16
    p = ol.make_params(1, ic, oc, ih, iw, 3, 3, pad=1, out_type=kind, out_scale=0.02, relu_hi=ol.FLT_MAX)
    x = rng.integers(0, 256, (1, I2, ih, iw, 16)).astype(np.uint8)
    xb = ol.aligned(x.size + 256, np.uint8)
    xb[:x.size] = x.ravel()
    wts = rng.normal(0, 0.05, (oc, ic, 3, 3)).astype(np.float32)
    bias = rng.normal(0, 0.3, oc).astype(np.float32)
    wq, scale, shift, _ = ol.direct_prepare(p, ol.weights_to_blocked(wts), bias)
    exp, _ = ol.direct_execute(p, x, wq, scale, shift)
    # reference layout [3][3][I2][4][16 oc][4 ic]
    wr = ol.aligned((3, 3, I2, 4, 16, 4), np.int8)
    wr[...] = wq.reshape(16, I2, 4, 4, 3, 3).transpose(4, 5, 1, 2, 0, 3)
    sc = ol.aligned(16, np.float32)
    sc[...] = scale
    sh = ol.aligned((T, 16), np.float32)
    sh[...] = shift[None, :]
    np_kind = ol.NP_OF[kind]
    tout = ol.aligned((oh * ow, 16), np.float32)
    rout = ol.aligned((oh * ow, 16), np_kind)
    wt = ow // T
    for ht in range(oh):
        for _wt in range(wt):
            rc = ref.ref_u8s8_conv3x3({ol.F32: 0, ol.U8: 1, ol.S8: 2}[kind], T, I2, ih, iw, oh, ow, ht, _wt, 1, 1, 0.0,
                                      ol.FLT_MAX, ol.ptr(tout), ol.ptr(rout) if kind != ol.F32 else None, ol.ptr(xb),
                                      ol.ptr(wr), ol.ptr(sc), ol.ptr(sh))
            assert rc == 0
    got = tout if kind == ol.F32 else rout
    assert np.array_equal(exp.reshape(oh * ow, 16).view(np.uint8), got.view(np.uint8))


def test_wino_weights_transform_bits():
    rng = np.random.default_rng(21)
    w = ol.aligned((3, 3, 16, 16), np.float32)
    w[...] = rng.normal(0, 0.05, w.shape)
    tw = ol.aligned((6, 6, 16, 16), np.float32)
    ref.ref_wino_trans_weights(ol.ptr(tw), ol.ptr(w))
    u = np.zeros(36, np.float32)
    for i in range(16):
        for o in range(16):
            g = np.ascontiguousarray(w[:, :, i, o].ravel())
            ol.oracle().orc_wino_tile_weights(ol.ptr(g), ol.ptr(u))
            assert np.array_equal(u.view(np.uint32), tw[:, :, i, o].ravel().view(np.uint32))


@pytest.mark.parametrize("h0,w0", [(2, 3), (-1, -1), (-1, 4), (3, -1), (7, 7), (7, 2), (-1, 7)])
def test_wino_input_transform_bits(h0, w0):
    rng = np.random.default_rng(h0 * 13 + w0 + 50)
    ih = iw = 12
    plane = ol.aligned((ih, iw, 16), np.float32)
    plane[...] = rng.uniform(0, 1, plane.shape)
    hs, he = max(0, -h0), min(5, ih - 1 - h0)
    ws, we = max(0, -w0), min(5, iw - 1 - w0)
    border = not (hs == 0 and ws == 0 and he == 5 and we == 5)
    tin = ol.aligned((6, 6, 16), np.float32)
    tile_ptr = ctypes.c_void_p(plane.ctypes.data + (h0 * iw + w0) * 16 * 4)
    ref.ref_wino_trans_input(int(border), ih, iw, ol.ptr(tin), tile_ptr, hs, he, ws, we)
    v = np.zeros(36, np.float32)
    for c in range(16):
        d = np.zeros((6, 6), np.float32)
        for i in range(6):
            for j in range(6):
                h, w = h0 + i, w0 + j
                if 0 <= h < ih and 0 <= w < iw:
                    d[i, j] = plane[h, w, c]
        fn = ol.oracle().orc_wino_tile_input_border if border else ol.oracle().orc_wino_tile_input
        fn(ol.ptr(d), ol.ptr(v))
        assert np.array_equal(v.view(np.uint32), tin[:, :, c].ravel().view(np.uint32))


@pytest.mark.parametrize("with_bias,with_relu", [(True, True), (True, False), (False, False)])
@pytest.mark.parametrize("h_end,w_end", [(3, 3), (1, 3), (3, 0), (2, 2)])
def test_wino_output_transform_bits(with_bias, with_relu, h_end, w_end):
    rng = np.random.default_rng(77 + h_end * 4 + w_end)
    oh = ow = 8
    m = ol.aligned((6, 6, 16), np.float32)
    m[...] = rng.normal(0, 3, m.shape)
    bias = ol.aligned(16, np.float32)
    bias[...] = rng.normal(0, 1, 16)
    out = ol.aligned((oh, ow, 16), np.float32, -777.0)
    border = not (h_end == 3 and w_end == 3)
    ref.ref_wino_trans_output(int(border), int(with_bias), int(with_relu), oh, ow, ol.ptr(out), ol.ptr(m),
                              ol.ptr(bias), h_end, w_end)
    y = np.zeros(16, np.float32)
    for c in range(16):
        mm = np.ascontiguousarray(m[:, :, c].ravel())
        ol.oracle().orc_wino_tile_output(ol.ptr(mm), ol.ptr(y))
        for i in range(4):
            for j in range(4):
                if i > h_end or j > w_end:
                    assert out[i, j, c] == np.float32(-777.0)
                    continue
                r = y[4 * i + j]
                if with_bias:
                    r = np.float32(r + bias[c])
                if with_relu:
                    r = r if r > 0 else np.float32(0)
                assert np.float32(r).view(np.uint32) == out[i, j, c].view(np.uint32), (i, j, c)


# ---- the other Winograd tile sizes: A = 4 F(2x2,3x3), A = 5 F(3x3,3x3) ------------------------------
@pytest.mark.parametrize("A", [4, 5])
def test_wino_weights_transform_bits_other_tiles(A):
    rng = np.random.default_rng(21 + A)
    w = ol.aligned((3, 3, 16, 16), np.float32)
    w[...] = rng.normal(0, 0.05, w.shape)
    tw = ol.aligned((A, A, 16, 16), np.float32)
    assert ref.ref_wino_trans_weights_a(A, ol.ptr(tw), ol.ptr(w)) == 0
    u = np.zeros(A * A, np.float32)
    for i in range(16):
        for o in range(16):
            g = np.ascontiguousarray(w[:, :, i, o].ravel())
            ol.oracle().orc_wino_tile_weights_a(A, ol.ptr(g), ol.ptr(u))
            assert np.array_equal(u.view(np.uint32), tw[:, :, i, o].ravel().view(np.uint32))


@pytest.mark.parametrize("A", [4, 5])
@pytest.mark.parametrize("h0,w0", [(2, 3), (1, 1), (0, 0), (3, 3), (6, 6), (2, 4), (-1, -1), (-1, 4), (3, -1), (8, 8), (9, 2), (-1, 9),
                                   (-2, 5), (4, 10)])
def test_wino_input_transform_bits_other_tiles(A, h0, w0):
    rng = np.random.default_rng(h0 * 13 + w0 + 50 + A)
    ih = iw = 12
    plane = ol.aligned((ih, iw, 16), np.float32)
    plane[...] = rng.uniform(0, 255, plane.shape).round() if (h0 + w0) % 2 else rng.uniform(0, 1, plane.shape)
    hs, he = max(0, -h0), min(A - 1, ih - 1 - h0)
    ws, we = max(0, -w0), min(A - 1, iw - 1 - w0)
    border = not (hs == 0 and ws == 0 and he == A - 1 and we == A - 1)
    tin = ol.aligned((A, A, 16), np.float32)
    tile_ptr = ctypes.c_void_p(plane.ctypes.data + (h0 * iw + w0) * 16 * 4)
    assert ref.ref_wino_trans_input_a(A, int(border), ih, iw, ol.ptr(tin), tile_ptr, hs, he, ws, we) == 0
    v = np.zeros(A * A, np.float32)
    for c in range(16):
        d = np.zeros((A, A), np.float32)
        for i in range(A):
            for j in range(A):
                h, w = h0 + i, w0 + j
                if 0 <= h < ih and 0 <= w < iw:
                    d[i, j] = plane[h, w, c]
        ol.oracle().orc_wino_tile_input_a(A, int(border), ol.ptr(d), ol.ptr(v))
        assert np.array_equal(v.view(np.uint32), tin[:, :, c].ravel().view(np.uint32)), (c, v, tin[:, :, c].ravel())


@pytest.mark.parametrize("A", [4, 5])
@pytest.mark.parametrize("kind", [ol.F32, ol.U8, ol.S8])
@pytest.mark.parametrize("with_bias,with_relu", [(True, True), (True, False), (False, False)])
@pytest.mark.parametrize("ends", ["full", "rows", "cols"])
def test_wino_output_transform_bits_other_tiles(A, kind, with_bias, with_relu, ends):
    M = A - 2
    h_end, w_end = {"full": (M - 1, M - 1), "rows": (0, M - 1), "cols": (M - 1, M - 2)}[ends]
    rng = np.random.default_rng(77 + h_end * 4 + w_end + A + kind)
    oh = ow = 8
    m = ol.aligned((A, A, 16), np.float32)
    m[...] = rng.normal(0, 3, m.shape)
    bias = ol.aligned(16, np.float32)
    bias[...] = rng.normal(0, 1, 16)
    np_kind = ol.NP_OF[kind]
    fill = -777.0 if kind == ol.F32 else 93
    out = ol.aligned((oh, ow, 16), np_kind, fill)
    border = not (h_end == M - 1 and w_end == M - 1)
    out_scale, out_z = 0.11, 3.0 if kind == ol.U8 else 0.0
    rc = ref.ref_wino_trans_output_a(A, {ol.F32: 0, ol.U8: 1, ol.S8: 2}[kind], int(border), int(with_bias),
                                     int(with_relu), oh, ow, ol.ptr(out), ol.ptr(m), ol.ptr(bias), h_end, w_end,
                                     np.float32(1.0) / np.float32(out_scale), out_z)
    assert rc == 0
    y = np.zeros(M * M, np.float32)
    for c in range(16):
        mm = np.ascontiguousarray(m[:, :, c].ravel())
        ol.oracle().orc_wino_tile_output_a(A, ol.ptr(mm), ol.ptr(y))
        for i in range(M):
            for j in range(M):
                if i > h_end or j > w_end:
                    assert out[i, j, c] == np_kind(fill)
                    continue
                r = ctypes.c_float()
                q = ol.oracle().orc_wino_output_value_a(A, float(y[M * i + j]), int(with_bias), float(bias[c]), kind,
                                                        out_scale, out_z, int(with_relu), ctypes.byref(r))
                if kind == ol.F32:
                    assert np.float32(r.value).view(np.uint32) == out[i, j, c].view(np.uint32), (i, j, c)
                else:
                    assert np_kind(q) == out[i, j, c], (i, j, c, q, out[i, j, c], r.value)


# ---- in-place sum fused into the Winograd output transform (with_ip_sum) ----------------------------
@pytest.mark.parametrize("A", [6, 4, 5])
@pytest.mark.parametrize("kind", [ol.F32, ol.U8, ol.S8])
@pytest.mark.parametrize("with_bias,with_relu,border", [(True, True, False), (False, False, False), (True, True, True),
                                                        (True, False, True)])
def test_wino_output_transform_with_sum_bits(A, kind, with_bias, with_relu, border):
    M = A - 2
    h_end, w_end = (M - 2, M - 1) if border else (M - 1, M - 1)
    rng = np.random.default_rng(900 + A + kind + 2 * with_bias + with_relu + 4 * border)
    m = ol.aligned((A, A, 16), np.float32)
    m[...] = rng.normal(0, 3, m.shape)
    bias = ol.aligned(16, np.float32)
    bias[...] = rng.normal(0, 1, 16)
    np_kind = ol.NP_OF[kind]
    out = ol.aligned((8, 8, 16), np_kind)
    out[...] = rng.normal(0, 2, out.shape) if kind == ol.F32 else rng.integers(-100 if kind == ol.S8 else 0, 100, out.shape)
    old = np.array(out)
    out_scale, out_z = 0.11, 3.0 if kind == ol.U8 else 0.0
    rc = ref.ref_wino_trans_output_sum(A, {ol.F32: 0, ol.U8: 1, ol.S8: 2}[kind], int(border), int(with_bias), int(with_relu),
                                       8, 8, ol.ptr(out), ol.ptr(m), ol.ptr(bias), h_end, w_end,
                                       np.float32(1.0) / np.float32(out_scale), out_z)
    assert rc == 0
    y = np.zeros(M * M, np.float32)
    for c in range(16):
        mm = np.ascontiguousarray(m[:, :, c].ravel())
        ol.oracle().orc_wino_tile_output_a(A, ol.ptr(mm), ol.ptr(y))
        for i in range(M):
            for j in range(M):
                if i > h_end or j > w_end:
                    assert out[i, j, c] == old[i, j, c]
                    continue
                r = ctypes.c_float()
                q = ol.oracle().orc_wino_output_value_sum(A, float(y[M * i + j]), int(with_bias), float(bias[c]), kind,
                                                          out_scale, out_z, int(with_relu), 1, float(old[i, j, c]),
                                                          ctypes.byref(r))
                if kind == ol.F32:
                    assert np.float32(r.value).view(np.uint32) == out[i, j, c].view(np.uint32), (i, j, c)
                else:
                    assert np_kind(q) == out[i, j, c], (i, j, c, q, out[i, j, c], r.value)


# ---- 5x5 / 7x7: the reference's generic k x k micro-kernel template ---------------------------------------
@pytest.mark.parametrize("kind", [ol.F32, ol.U8, ol.S8])
@pytest.mark.parametrize("K,S,iw,lp,rp", [(5, 1, 7, 2, 2), (7, 1, 7, 3, 3), (5, 2, 15, 1, 1), (7, 2, 14, 3, 2), (7, 2, 14, 2, 3)])
def test_conv_kxk_kernel(kind, K, S, iw, lp, rp):
    """The oracle's k x k path against the compiled template on the pad sets for which the template is
    the convolution (stride 1: k/2 on both sides; stride 2: (k/2, k/2 - 1) bound as S2_LLP, or
    (k/2 - 1, k/2)): every shape of the reference's tuned runs, ResNet's 7x7 s2 first layer included."""
    import sys, os
    sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden"))
    import cases
    d = cases.convk_inputs(kind, K, S, iw, lp, rp, 900 + K + S + iw + kind)
    got, exp = cases.convk_oracle(d), cases.convk_reference(d, ref)
    assert got.dtype == exp.dtype
    assert np.array_equal(np.ascontiguousarray(got).view(np.uint8), np.ascontiguousarray(exp).view(np.uint8))


def test_conv_kxk_template_is_not_the_convolution_for_other_pad_sets():
    """Why the k x k golden cases stop where they do: with pads (2, 2) at stride 2 the 7x7 template differs
    from the convolution in its second-to-last column only (a valid tap dropped), which the oracle and
    the product do not imitate."""
    import sys, os
    sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden"))
    import cases
    d = cases.convk_inputs(ol.S8, 7, 2, 15, 2, 2, 77)
    got, exp = cases.convk_oracle(d).reshape(7, 7, 16), cases.convk_reference(d, ref).reshape(7, 7, 16)
    cols = np.unique(np.argwhere(got != exp)[:, 1])
    assert list(cols) == [5]
