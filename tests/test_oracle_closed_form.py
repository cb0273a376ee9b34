"""Pins the parts of the oracle that the mathematics fixes: integer contractions by brute force,
weight quantization and scale/shift folding by an independent numpy float32 evaluation, reorders by
numpy transposes, the harness rounding helper on exact ties, Winograd against a float64 convolution."""
import ctypes

import numpy as np
import pytest

import oracle_lib as ol

f32 = np.float32


def conv_int_bruteforce(x_nchw, wq_oihw, pad, stride):
    n, ic, ih, iw = x_nchw.shape
    oc, _, kh, kw = wq_oihw.shape
    oh = (ih + 2 * pad - kh) // stride + 1
    ow = (iw + 2 * pad - kw) // stride + 1
    xp = np.zeros((n, ic, ih + 2 * pad, iw + 2 * pad), np.int64)
    xp[:, :, pad:pad + ih, pad:pad + iw] = x_nchw
    out = np.zeros((n, oc, oh, ow), np.int64)
    for a in range(kh):
        for b in range(kw):
            patch = xp[:, :, a:a + stride * oh:stride, b:b + stride * ow:stride]
            out += np.einsum("nchw,oc->nohw", patch, wq_oihw[:, :, a, b].astype(np.int64))
    return out


def quant_weights_numpy(w_oihw):
    oc = w_oihw.shape[0]
    absmax = np.abs(w_oihw).reshape(oc, -1).max(axis=1).astype(f32)
    t = (w_oihw.astype(f32) * f32(127.0)).astype(f32)
    t = (t / absmax[:, None, None, None]).astype(f32)
    return np.rint(t).astype(np.int8), absmax


@pytest.mark.parametrize("kh,pad,stride,ic,oc,ihw", [(1, 0, 1, 64, 32, 9), (1, 0, 2, 32, 48, 10), (3, 1, 1, 32, 32, 7),
                                                     (3, 1, 1, 48, 16, 14)])
@pytest.mark.parametrize("out_type", [ol.U8, ol.S8, ol.F32])
def test_direct_closed_form(kh, pad, stride, ic, oc, ihw, out_type):
    rng = np.random.default_rng(kh * 100 + ic + oc + out_type)
    n = 2
    x = rng.integers(0, 256, (n, ic, ihw, ihw)).astype(np.uint8)
    w = rng.normal(0, 0.05, (oc, ic, kh, kh)).astype(f32)
    b = rng.normal(0, 0.01, oc).astype(f32)
    out_scale = f32(0.013)
    p = ol.make_params(n, ic, oc, ihw, ihw, kh, kh, pad, stride, out_type=out_type, out_scale=float(out_scale),
                       relu_hi=ol.FLT_MAX if out_type != ol.S8 else 100.0)
    wq, scale, shift, wsum = ol.direct_prepare(p, ol.weights_to_blocked(w), b)
    # weight quantization: abs-max, (w*127)/absmax, round-half-even, all float32
    wq_np, absmax = quant_weights_numpy(w)
    assert np.array_equal(wq, wq_np)
    assert np.array_equal(wsum, wq_np.reshape(oc, -1).sum(axis=1))
    in_S = f32(1.0 / 255.0)
    w_S = (absmax / f32(127.0)).astype(f32)
    if out_type == ol.F32:
        exp_scale = (in_S * w_S).astype(f32)
        exp_shift = b
    else:
        rep = f32(1.0) / out_scale
        exp_scale = ((in_S * w_S).astype(f32) * rep).astype(f32)
        # fused b*repS + z with z = 0 is the correctly rounded product
        exp_shift = (b.astype(np.float64) * np.float64(rep)).astype(f32)
    assert np.array_equal(scale.view(np.uint32), exp_scale.view(np.uint32))
    assert np.array_equal(shift.view(np.uint32), exp_shift.view(np.uint32))
    out, acc = ol.direct_execute(p, ol.to_blocked(x), wq, scale, shift)
    acc_bf = conv_int_bruteforce(x, wq_np, pad, stride)
    assert np.array_equal(ol.from_blocked(acc, oc), acc_bf)
    # epilogue in float64: fused multiply-add == correctly rounded exact value
    exact = acc_bf.astype(np.float64) * scale.astype(np.float64)[None, :, None, None] \
        + shift.astype(np.float64)[None, :, None, None]
    f = exact.astype(f32)
    f = np.minimum(np.maximum(f, f32(p.relu_lo)), f32(p.relu_hi))
    got = ol.from_blocked(out, oc)
    if out_type == ol.F32:
        assert np.array_equal(got.view(np.uint32), f.view(np.uint32))
    elif out_type == ol.U8:
        assert np.array_equal(got, np.clip(np.rint(f), 0, 255).astype(np.uint8))
    else:
        assert np.array_equal(got, np.clip(np.rint(f), -128, 127).astype(np.int8))


def test_direct_sum_fusion_closed_form():
    rng = np.random.default_rng(5)
    n, ic, oc, hw = 2, 64, 32, 6
    x = rng.integers(0, 256, (n, ic, hw, hw)).astype(np.uint8)
    w = rng.normal(0, 0.05, (oc, ic, 1, 1)).astype(f32)
    b = rng.normal(0, 0.01, oc).astype(f32)
    old = rng.integers(-128, 128, (n, oc, hw, hw)).astype(np.int8)
    p = ol.make_params(n, ic, oc, hw, hw, out_type=ol.S8, with_sum=True, out_scale=0.05, sum_scale=0.61,
                       relu_hi=127.0)
    wq, scale, shift, _ = ol.direct_prepare(p, ol.weights_to_blocked(w), b)
    out, acc = ol.direct_execute(p, ol.to_blocked(x), wq, scale, shift, out_init=ol.to_blocked(old))
    accn = ol.from_blocked(acc, oc).astype(np.float64)
    f = (accn * scale.astype(np.float64)[None, :, None, None] + shift.astype(np.float64)[None, :, None, None]).astype(f32)
    f = (old.astype(np.float64) * np.float64(f32(0.61)) + f.astype(np.float64)).astype(f32)
    f = np.minimum(np.maximum(f, f32(0)), f32(127))
    assert np.array_equal(ol.from_blocked(out, oc), np.clip(np.rint(f), -128, 127).astype(np.int8))


def test_depthwise_closed_form_integer_and_s8():
    rng = np.random.default_rng(9)
    n, g, hw = 2, 32, 9
    x = rng.integers(0, 256, (n, g, hw, hw)).astype(np.uint8)
    w = rng.normal(0, 0.1, (g, 3, 3)).astype(f32)
    b = rng.normal(0, 0.01, g).astype(f32)
    p = ol.make_params(n, g, g, hw, hw, 3, 3, 1, g=g, out_type=ol.S8, T=4, out_scale=0.02, relu_hi=127.0)
    wq, scale, shift, wsum = ol.depthwise_prepare(p, w, b)
    wq_np, absmax = quant_weights_numpy(w.reshape(g, 1, 3, 3))
    assert np.array_equal(wq, wq_np.reshape(g, 3, 3))
    out, acc = ol.depthwise_execute(p, ol.to_blocked(x), wq, scale, shift)
    xp = np.zeros((n, g, hw + 2, hw + 2), np.int64)
    xp[:, :, 1:-1, 1:-1] = x
    bf = np.zeros((n, g, hw, hw), np.int64)
    for a in range(3):
        for c in range(3):
            bf += xp[:, :, a:a + hw, c:c + hw] * wq[:, a, c].astype(np.int64)[None, :, None, None]
    assert np.array_equal(ol.from_blocked(acc, g), bf)
    f = (bf.astype(np.float64) * scale.astype(np.float64)[None, :, None, None]
         + shift.astype(np.float64)[None, :, None, None]).astype(f32)
    f = np.minimum(np.maximum(f, f32(0)), f32(127))
    assert np.array_equal(ol.from_blocked(out, g), np.clip(np.rint(f), -128, 127).astype(np.int8))


def test_depthwise_u8_floor_columns():
    # columns _T < 4*(Tz/4) of every width block floor, the rest round to nearest
    rng = np.random.default_rng(10)
    n, g, hw, T = 1, 16, 14, 7
    x = rng.integers(0, 256, (n, g, hw, hw)).astype(np.uint8)
    w = rng.normal(0, 0.1, (g, 3, 3)).astype(f32)
    b = rng.normal(0, 0.01, g).astype(f32)
    p = ol.make_params(n, g, g, hw, hw, 3, 3, 1, g=g, out_type=ol.U8, T=T, out_scale=6.0 / 255.0, relu_hi=255.0)
    wq, scale, shift, _ = ol.depthwise_prepare(p, w, b)
    out, acc = ol.depthwise_execute(p, ol.to_blocked(x), wq, scale, shift)
    a = ol.from_blocked(acc, g).astype(np.float64)
    f = (a * scale.astype(np.float64)[None, :, None, None] + shift.astype(np.float64)[None, :, None, None]).astype(f32)
    f = np.minimum(np.maximum(f, f32(0)), f32(255))
    col = np.arange(hw) % T
    exp = np.where(col[None, None, None, :] < 4, np.floor(f), np.rint(f)).astype(np.uint8)
    assert np.array_equal(ol.from_blocked(out, g), exp)
    assert (np.floor(f) != np.rint(f)).any()


def test_reorders():
    rng = np.random.default_rng(3)
    x = rng.normal(size=(2, 20, 3, 5)).astype(f32)
    xb = np.zeros((2, 2, 3, 5, 16), f32)
    ol.oracle().orc_reorder_nchw_to_blocked_f32(ol.ptr(xb), ol.ptr(x), 2, 20, 3, 5)
    assert np.array_equal(xb, ol.to_blocked(x))
    back = np.zeros_like(x)
    ol.oracle().orc_reorder_blocked_to_nchw_f32(ol.ptr(back), ol.ptr(xb), 2, 20, 3, 5)
    assert np.array_equal(back, x)
    w = rng.normal(size=(20, 35, 3, 3)).astype(f32)
    wb = np.zeros((2, 3, 3, 3, 16, 16), f32)
    ol.oracle().orc_reorder_oihw_to_blocked_f32(ol.ptr(wb), ol.ptr(w), 20, 35, 3, 3)
    assert np.array_equal(wb, ol.weights_to_blocked(w))
    wback = np.zeros_like(w)
    ol.oracle().orc_reorder_blocked_to_oihw_f32(ol.ptr(wback), ol.ptr(wb), 20, 35, 3, 3)
    assert np.array_equal(wback, w)
    u = rng.integers(0, 256, (1, 17, 2, 2)).astype(np.uint8)
    ub = np.zeros((1, 2, 2, 2, 16), np.uint8)
    ol.oracle().orc_reorder_nchw_to_blocked_u8(ol.ptr(ub), ol.ptr(u), 1, 17, 2, 2)
    assert np.array_equal(ub, ol.to_blocked(u))


def test_quantize_input_ties_go_to_odd():
    # the reference harness helper (tests/elt_conv_utils.cpp:354-370) is named round-to-nearest-even
    # but resolves exact .5 ties towards the odd neighbour; everything else rounds to nearest
    x = np.array([0.5, 1.5, 2.5, 3.5, 0.25, 0.75, 254.5, 255.49, 7.0, 2.4999998], f32)
    q = ol.quantize_input_u8(x, 1.0, 0.0)
    assert q.tolist() == [1, 1, 3, 3, 0, 1, 255, 255, 7, 2]
    rng = np.random.default_rng(0)
    y = rng.uniform(0, 1, 100000).astype(f32)
    v = (y / f32(1.0 / 255.0)).astype(f32)
    frac_is_half = (v - np.floor(v)) == 0.5
    exp = np.where(frac_is_half, np.floor(v) + (np.floor(v) % 2 == 0), np.rint(v)).astype(np.uint8)
    assert np.array_equal(ol.quantize_input_u8(y, 1.0 / 255.0, 0.0), exp)


def test_winograd_pipeline_matches_float_convolution():
    """With a fine tinput quantization step the int8 Winograd result must approach the float64 direct
    convolution; a wrong transform matrix, tile anchor or transposed operand fails this by far."""
    rng = np.random.default_rng(12)
    n, ic, oc, hw = 2, 32, 32, 10   # 10 -> 3x3 tiles with a ragged last tile
    x = rng.uniform(0, 1, (n, ic, hw, hw)).astype(f32)
    w = rng.normal(0, 0.02, (oc, ic, 3, 3)).astype(f32)
    b = rng.normal(0, 0.01, oc).astype(f32)
    p = ol.make_params(n, ic, oc, hw, hw, 3, 3, 1, out_type=ol.F32, in_scale=1.0)
    xb = ol.to_blocked(x)
    mn, mx = ol.wino_tinput_range(p, xb)
    p.tin_scale = (mx - mn + 1e-6) / 255.0
    p.tin_z = -mn * 255.0 / (mx - mn + 1e-6)
    twq, tscale, tshift = ol.wino_prepare(p, ol.weights_to_blocked(w))
    tin = ol.wino_trans_input(p, xb)
    tout, acc = ol.wino_gemm(p, tin, twq, tscale, tshift)
    out = ol.from_blocked(ol.wino_trans_output(p, tout, b), oc)
    xp = np.zeros((n, ic, hw + 2, hw + 2))
    xp[:, :, 1:-1, 1:-1] = x
    refo = np.zeros((n, oc, hw, hw))
    for a in range(3):
        for c in range(3):
            refo += np.einsum("nchw,oc->nohw", xp[:, :, a:a + hw, c:c + hw], w[:, :, a, c].astype(np.float64))
    refo = np.maximum(refo + b[None, :, None, None], 0)
    err = np.abs(out - refo).max() / np.abs(refo).max()
    assert err < 0.06, err
    # integer GEMM of the pipeline, brute force
    a_idx, o2, t = 7, 1, 5
    exp = (tin[a_idx, :, t, :].astype(np.int64).reshape(-1)[None, :] * twq[a_idx, 16:32, :].astype(np.int64)).sum(1)
    assert np.array_equal(acc[a_idx, o2, t], exp)
    # tinput zero point is ceil()-ed and the scale folding is (absmax/127)*tin_S
    u = np.zeros(36, f32)
    g = np.ascontiguousarray(w[3, 5].ravel())
    ol.oracle().orc_wino_tile_weights(ol.ptr(g), ol.ptr(u))
    G = np.array([[1.13777777777778, 0, 0], [-0.688403361344538, -0.430252100840336, -0.26890756302521],
                  [-0.688403361344538, 0.430252100840336, -0.26890756302521],
                  [0.119514472455649, 0.179271708683473, 0.26890756302521],
                  [0.119514472455649, -0.179271708683473, 0.26890756302521], [0, 0, 1]])
    assert np.allclose(u.reshape(6, 6), G @ w[3, 5].astype(np.float64) @ G.T, rtol=1e-5, atol=1e-7)


@pytest.mark.parametrize("k,pad,stride,hw,out_hw", [(3, 1, 1, 9, None), (3, 0, 2, 12, 6), (7, 3, 2, 15, None), (5, 2, 1, 8, None)])
@pytest.mark.parametrize("out_type", [ol.F32, ol.S8])
def test_zero_point_with_padding_matches_the_real_valued_convolution(k, pad, stride, hw, out_hw, out_type):
    """Input zero point with padding: the oracle's per-pixel shift must make the result equal to the
    real-valued convolution of the DEQUANTIZED input, (u8 - z) * S, with the dequantized weights --
    where padding contributes exactly zero.  A shift that folded all taps at the border (or none)
    misses this by far more than the tolerance."""
    rng = np.random.default_rng(k * 10 + stride + out_type)
    n, ic, oc = 2, 24, 16
    z, in_S = 113.0, 0.017
    x = rng.integers(0, 256, (n, ic, hw, hw)).astype(np.uint8)
    w = rng.normal(0, 0.05, (oc, ic, k, k)).astype(f32)
    b = np.zeros(16, f32)
    b[:oc] = rng.normal(0, 0.3, oc)
    out_scale = 0.05
    p = ol.make_params(n, ic, oc, hw, hw, k, k, stride=stride, out_type=out_type, in_scale=in_S, in_z=z,
                       out_scale=out_scale, with_relu=False, pad_tl=pad,
                       out_hw=None if out_hw is None else (out_hw, out_hw), pad=pad)
    wb = ol.weights_to_blocked(w)
    wq, scale, shift, wsum = ol.direct_prepare(p, wb, b)
    out, acc, smap = ol.direct_execute_border(p, ol.to_blocked(x), wb, b, wq, scale)
    # interior pixels use the plain shift
    ihs = [oh for oh in range(p.oh) if oh * stride - pad >= 0 and oh * stride - pad + k <= hw]
    assert ihs and np.array_equal(smap[ihs[0], ihs[0]], shift)
    assert not np.array_equal(smap[0, 0], shift) or pad == 0
    # float64 model
    wq_np, absmax = quant_weights_numpy(w)
    w_deq = wq_np.astype(np.float64) * (absmax.astype(np.float64) / 127.0)[:, None, None, None]
    xr = (x.astype(np.float64) - z) * in_S
    exp = np.zeros((n, oc, p.oh, p.ow))
    for oh in range(p.oh):
        for ow in range(p.ow):
            for kh in range(k):
                for kw in range(k):
                    ih, iw = oh * stride + kh - pad, ow * stride + kw - pad
                    if 0 <= ih < hw and 0 <= iw < hw:
                        exp[:, :, oh, ow] += np.einsum("nc,oc->no", xr[:, :, ih, iw], w_deq[:, :, kh, kw])
    exp += b[:oc].astype(np.float64)[None, :, None, None]
    got = ol.from_blocked(out, oc).astype(np.float64)
    if out_type == ol.S8:
        got = got * out_scale
        assert np.abs(got - np.clip(exp, -128 * out_scale, 127 * out_scale)).max() <= 0.5 * out_scale + 1e-4
    else:
        assert np.abs(got - exp).max() <= 2e-4 * max(1.0, np.abs(exp).max())


# ---- scale / shift folding with non-zero zero points -------------------------------------------------
# What the reference's translation units hold when compiled with its own flags (g++ -O2, default
# contraction; src/elx_int8_conv_direct_1x1.cpp:324-354, src/elx_int8_conv_direct.cpp:357-419,
# src/elx_int8_conv_direct_depthwise.cpp:261-291):
#   scale = (in_S * w_S) * out_repS                      vmulps, vmulps
#   t     = in_z * wsum                                  vmulps
#   shift = fma(bias, out_repS, out_z)                   vfmadd132ps
#   shift = fma(-t, scale, shift)                        vfnmadd132ps
#   shift = shift - (sum_z * sum_S)   (1x1 with sum)     vmulss, vbroadcastss, vsubps: NOT fused
# The executors themselves cannot be linked here (their kernel tables are generated by the reference's
# build), so these folds are evaluated independently in long doubles, where a product of two floats plus a
# float is exact, and rounded once -- and the inputs are checked to tell every other contraction apart.
L = np.longdouble


def _fma(a, b, c):
    return (np.asarray(a, f32).astype(L) * np.asarray(b, f32).astype(L) + np.asarray(c, f32).astype(L)).astype(f32)


def fold_variants(in_S, in_z, w_S, wsum, bias, rep, out_z, sum_S=None, sum_z=None):
    """{name: (scale, shift)}: "compiled" is the reference's compiled form, the others drop or add one fusion"""
    scale = ((f32(in_S) * w_S).astype(f32) * f32(rep)).astype(f32)
    t = (f32(in_z) * wsum.astype(f32)).astype(f32)
    fused_b = _fma(bias, f32(rep), f32(out_z))
    plain_b = ((bias * f32(rep)).astype(f32) + f32(out_z)).astype(f32)
    v = {"compiled": _fma(-t, scale, fused_b),
         "bias_unfused": _fma(-t, scale, plain_b),
         "zero_point_unfused": (fused_b - (t * scale).astype(f32)).astype(f32)}
    if sum_S is not None:
        prod = f32(f32(sum_z) * f32(sum_S))
        c = v["compiled"]
        v = {k: (s - prod).astype(f32) for k, s in v.items()}
        v["sum_fused"] = _fma(f32(-sum_z), f32(sum_S), c)
    return scale, v


@pytest.mark.parametrize("k,with_sum,out_type", [(1, True, ol.S8), (1, True, ol.U8), (1, False, ol.U8), (3, False, ol.S8),
                                                 (3, False, ol.U8)])
def test_direct_fold_with_zero_points_is_the_compiled_contraction(k, with_sum, out_type):
    rng = np.random.default_rng(70 + k + 2 * with_sum + out_type)
    ic, oc = 48, 256
    w = rng.normal(0, 0.05, (oc, ic, k, k)).astype(f32)
    b = rng.normal(0, 0.7, oc).astype(f32)
    in_S, in_z, out_S, out_z, sum_S, sum_z = 0.0173, 113.0, 0.0371, 3.0, 0.6113, -97.0
    p = ol.make_params(1, ic, oc, 8, 8, k, k, 0, out_type=out_type, with_sum=with_sum, in_scale=in_S, in_z=in_z,
                       out_scale=out_S, out_z=out_z, sum_scale=sum_S, sum_z=sum_z)
    wq, scale, shift, wsum = ol.direct_prepare(p, ol.weights_to_blocked(w), b)
    wq_np, absmax = quant_weights_numpy(w)
    assert np.array_equal(wq, wq_np)
    w_S = (absmax / f32(127.0)).astype(f32)
    rep = f32(1.0) / f32(out_S)
    exp_scale, v = fold_variants(in_S, in_z, w_S, wq_np.reshape(oc, -1).sum(axis=1), b, rep, out_z,
                                 sum_S if with_sum else None, sum_z if with_sum else None)
    assert np.array_equal(scale.view(np.uint32), exp_scale.view(np.uint32))
    assert np.array_equal(shift.view(np.uint32), v["compiled"].view(np.uint32))
    for name, alt in v.items():   # the data tells the compiled form from every neighbour
        assert name == "compiled" or (alt.view(np.uint32) != v["compiled"].view(np.uint32)).sum() >= 4, name


def test_depthwise_fold_with_zero_points_is_the_compiled_contraction():
    rng = np.random.default_rng(77)
    g = 256
    w = rng.normal(0, 0.1, (g, 3, 3)).astype(f32)
    b = rng.normal(0, 0.7, g).astype(f32)
    in_S, in_z, out_S, out_z = 0.0173, 113.0, 0.0371, 3.0
    p = ol.make_params(1, g, g, 8, 8, 3, 3, 1, g=g, out_type=ol.S8, T=4, in_scale=in_S, in_z=in_z, out_scale=out_S,
                       out_z=out_z, relu_hi=127.0)
    wq, scale, shift, wsum = ol.depthwise_prepare(p, w, b)
    wq_np, absmax = quant_weights_numpy(w.reshape(g, 1, 3, 3))
    exp_scale, v = fold_variants(in_S, in_z, (absmax / f32(127.0)).astype(f32), wq_np.reshape(g, -1).sum(axis=1), b,
                                 f32(1.0) / f32(out_S), out_z)
    assert np.array_equal(scale.view(np.uint32), exp_scale.view(np.uint32))
    assert np.array_equal(shift.view(np.uint32), v["compiled"].view(np.uint32))
    for name, alt in v.items():
        assert name == "compiled" or (alt.view(np.uint32) != v["compiled"].view(np.uint32)).sum() >= 4, name


@pytest.mark.parametrize("k,pad,stride,hw,out_hw", [(3, 1, 1, 9, None), (3, 0, 2, 12, 6), (7, 3, 2, 15, None), (5, 2, 1, 8, None),
                                                    (3, 1, 2, 11, None)])
@pytest.mark.parametrize("out_type", [ol.F32, ol.U8])
def test_border_shift_rows_fold_exactly_the_valid_taps(k, pad, stride, hw, out_hw, out_type):
    """Every row of the oracle's per-pixel shift map equals the fold above applied to the sum of the quantized
    weights of exactly the taps that fall inside the image for that pixel (taps found here by testing the
    input coordinate, not through the reference's range tables, src/elx_int8_conv_direct.cpp:227-309)."""
    rng = np.random.default_rng(k * 10 + stride + out_type)
    ic, oc = 24, 32
    in_S, in_z, out_S, out_z = 0.017, 113.0, 0.05, 2.0
    w = rng.normal(0, 0.05, (oc, ic, k, k)).astype(f32)
    b = rng.normal(0, 0.3, oc).astype(f32)
    p = ol.make_params(1, ic, oc, hw, hw, k, k, stride=stride, out_type=out_type, in_scale=in_S, in_z=in_z, out_scale=out_S,
                       out_z=out_z, with_relu=False, pad_tl=pad, out_hw=None if out_hw is None else (out_hw, out_hw),
                       pad=pad)
    wb = ol.weights_to_blocked(w)
    wq, scale, shift, _ = ol.direct_prepare(p, wb, b)
    smap = np.zeros((p.oh, p.ow, ol.up16(oc)), f32)
    assert ol.oracle().orc_direct_border_shifts(ctypes.byref(p), ol.ptr(wb), ol.ptr(b), ol.ptr(smap)) == 0
    wq_np, absmax = quant_weights_numpy(w)
    w_S = (absmax / f32(127.0)).astype(f32)
    seen = set()
    for oh in range(p.oh):
        for ow in range(p.ow):
            vh = [a for a in range(k) if 0 <= oh * stride + a - pad < hw]
            vw = [c for c in range(k) if 0 <= ow * stride + c - pad < hw]
            seen.add((tuple(vh), tuple(vw)))
            wsum = wq_np[:, :, vh][:, :, :, vw].reshape(oc, -1).astype(np.int64).sum(axis=1)
            if out_type == ol.F32:
                sc = (f32(in_S) * w_S).astype(f32)
                exp = _fma(-(f32(in_z) * wsum.astype(f32)).astype(f32), sc, b)
            else:
                sc, v = fold_variants(in_S, in_z, w_S, wsum, b, f32(1.0) / f32(out_S), out_z)
                exp = v["compiled"]
            assert np.array_equal(smap[oh, ow, :oc].view(np.uint32), exp.view(np.uint32)), (oh, ow)
    assert len(seen) >= (4 if pad else 1)
