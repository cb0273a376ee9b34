"""Golden cases for the CPU oracle: seeded inputs of the reference's micro-kernel templates and the
way the oracle evaluates the same case.  make_golden.py runs the COMPILED reference templates
(oracle/_ref, built from /root/reference by oracle/Makefile) on these inputs and stores inputs +
reference outputs as .npz; tests/test_golden.py replays the stored inputs through the oracle and
compares bit for bit -- without needing the reference tree or its build.
"""
import ctypes

import numpy as np

import oracle_lib as ol

AT_RELU, AT_SUM, AT_CLEAR, AT_RESTORE = 1 << 1, 1 << 2, 1 << 3, 1 << 5
KIND_ID = {ol.F32: 0, ol.U8: 1, ol.S8: 2}


def _al(a):
    b = ol.aligned(a.shape, a.dtype)
    b[...] = a
    return b


def _epi(kind, acc, scale, shift, with_sum, old, sum_s, relu, lo, hi):
    f = ctypes.c_float()
    q = ol.oracle().orc_epilogue(kind, int(acc), float(scale), float(shift), int(with_sum), int(old), float(sum_s),
                                 int(relu), float(lo), float(hi), ctypes.byref(f))
    return f.value if kind == ol.F32 else q


# ---- u8s8 GEMM micro-kernel + epilogue (src/kernel/elk_u8s8_gemm.hxx) ---------------------------
def gemm_inputs(kind, O, T, with_sum, seed):
    rng = np.random.default_rng(seed)
    I2 = 5
    np_kind = ol.NP_OF[kind]
    d = dict(kind=np.int32(kind), O=np.int32(O), T=np.int32(T), I2=np.int32(I2), with_sum=np.int32(with_sum),
             x=rng.integers(0, 256, (I2, T, 16)).astype(np.uint8),
             w=rng.integers(-127, 128, (I2, 4, O, 16, 4)).astype(np.int8),
             scale=rng.uniform(1e-4, 3e-3, (O, 16)).astype(np.float32),
             shift=rng.normal(0, 20, (O, 16)).astype(np.float32),
             sum_s=np.float32(0.37109375 if with_sum else 0.0),
             lo=np.float32(0.0 if kind == ol.U8 else -60.0), hi=np.float32(200.0 if kind == ol.U8 else 90.0))
    if kind == ol.F32:
        d["old"] = np.zeros((O, T, 16), np.float32)
    else:
        d["old"] = (rng.integers(0, 256, (O, T, 16)) if kind == ol.U8 else rng.integers(-128, 128, (O, T, 16))).astype(np_kind)
    return d


def gemm_reference(d, ref):
    kind, O, T, I2 = int(d["kind"]), int(d["O"]), int(d["T"]), int(d["I2"])
    tout = ol.aligned((O, T, 16), np.float32)
    oout = _al(d["old"])
    attr = AT_CLEAR | AT_RESTORE | AT_RELU | (AT_SUM if int(d["with_sum"]) else 0)
    x, w, sc, sh = _al(d["x"]), _al(d["w"]), _al(d["scale"]), _al(d["shift"])   # keep the buffers alive
    rc = ref.ref_u8s8_gemm(KIND_ID[kind], O, T, I2, attr, float(d["lo"]), float(d["hi"]), float(d["sum_s"]),
                           ol.ptr(tout), ol.ptr(oout), ol.ptr(x), ol.ptr(w), ol.ptr(sc), ol.ptr(sh))
    assert rc == 0
    return np.array(tout if kind == ol.F32 else oout)


def gemm_oracle(d):
    kind, O, T, I2 = int(d["kind"]), int(d["O"]), int(d["T"]), int(d["I2"])
    acc = np.einsum("itvk,ivock->otc", d["x"].reshape(I2, T, 4, 4).astype(np.int64), d["w"].astype(np.int64))
    out = np.zeros((O, T, 16), ol.NP_OF[kind])
    for o in range(O):
        for t in range(T):
            for c in range(16):
                out[o, t, c] = _epi(kind, acc[o, t, c], d["scale"][o, c], d["shift"][o, c], int(d["with_sum"]),
                                    d["old"][o, t, c] if kind != ol.F32 else 0, d["sum_s"], True, d["lo"], d["hi"])
    return out


# ---- depthwise micro-kernel (src/kernel/elk_u8s8_depthwise_conv.hxx) ------------------------------
def dw_inputs(T, ow, ih, kind, seed, relu_hi):
    rng = np.random.default_rng(seed)
    G2 = 2
    return dict(T=np.int32(T), ow=np.int32(ow), ih=np.int32(ih), kind=np.int32(kind), relu_hi=np.float32(relu_hi),
                x=rng.integers(0, 256, (1, G2, ih, ow, 16)).astype(np.uint8),
                w=rng.normal(0, 0.1, (32, 3, 3)).astype(np.float32),
                bias=rng.normal(0, 0.5, 32).astype(np.float32))


def _dw_params(d):
    return ol.make_params(1, 32, 32, int(d["ih"]), int(d["ow"]), 3, 3, pad=1, g=32, out_type=int(d["kind"]),
                          T=int(d["T"]), out_scale=6.0 / 255.0, relu_hi=float(d["relu_hi"]))


def dw_oracle(d):
    p = _dw_params(d)
    wq, scale, shift, _ = ol.depthwise_prepare(p, d["w"], d["bias"])
    out, _ = ol.depthwise_execute(p, d["x"], wq, scale, shift)
    return out.reshape(2, int(d["ih"]) * int(d["ow"]), 16)


def dw_reference(d, ref):
    """The reference micro-kernel gets the ORACLE's quantized weights / folded scale and shift (the
    weight side is pinned separately by closed forms): this pins contraction, borders and the
    floor-vs-round store rule."""
    p = _dw_params(d)
    G2, ih, iw, oh, ow, T, kind = 2, int(d["ih"]), int(d["ow"]), int(d["ih"]), int(d["ow"]), int(d["T"]), int(d["kind"])
    wq, scale, shift, _ = ol.depthwise_prepare(p, d["w"], d["bias"])
    xb = ol.aligned(d["x"].size + 256, np.uint8)
    xb[:d["x"].size] = d["x"].ravel()
    wr = ol.aligned((G2, 3, 16, 4), np.int8)
    wr[...] = 0
    wr[:, :, :, :3] = wq.reshape(G2, 16, 3, 3).transpose(0, 2, 1, 3)
    sc, sh = _al(scale.reshape(G2, 16)), _al(shift.reshape(G2, 16))
    got = ol.aligned((G2, oh * ow, 16), ol.NP_OF[kind])
    wt = (ow + T - 1) // T
    Tr = ow % T or T
    for ht in range(oh):
        for _wt in range(wt):
            Tz = Tr if _wt == wt - 1 else T
            rc = ref.ref_u8s8_depthwise(KIND_ID[kind], T, Tz, G2, ih, iw, oh, ow, ht, _wt, 1, 1, 1, 1, 0.0,
                                        float(d["relu_hi"]), ol.ptr(got), ol.ptr(xb), ol.ptr(wr), ol.ptr(sc), ol.ptr(sh))
            assert rc == 0
    return np.array(got)


# ---- 3x3 micro-kernel (src/kernel/elk_u8s8_conv.hxx) --------------------------------------------
def conv_inputs(kind, T, ow, seed):
    rng = np.random.default_rng(seed)
    I2, ih = 2, 5
    return dict(kind=np.int32(kind), T=np.int32(T), ow=np.int32(ow),
                x=rng.integers(0, 256, (1, I2, ih, ow, 16)).astype(np.uint8),
                w=rng.normal(0, 0.05, (16, 16 * I2, 3, 3)).astype(np.float32),
                bias=rng.normal(0, 0.3, 16).astype(np.float32))


def _conv_params(d):
    return ol.make_params(1, 32, 16, 5, int(d["ow"]), 3, 3, pad=1, out_type=int(d["kind"]), out_scale=0.02,
                          relu_hi=ol.FLT_MAX)


def conv_oracle(d):
    p = _conv_params(d)
    wq, scale, shift, _ = ol.direct_prepare(p, ol.weights_to_blocked(d["w"]), d["bias"])
    out, _ = ol.direct_execute(p, d["x"], wq, scale, shift)
    return out.reshape(5 * int(d["ow"]), 16)


def conv_reference(d, ref):
    p = _conv_params(d)
    kind, T, ow, I2, ih, oh = int(d["kind"]), int(d["T"]), int(d["ow"]), 2, 5, 5
    wq, scale, shift, _ = ol.direct_prepare(p, ol.weights_to_blocked(d["w"]), d["bias"])
    xb = ol.aligned(d["x"].size + 256, np.uint8)
    xb[:d["x"].size] = d["x"].ravel()
    wr = ol.aligned((3, 3, I2, 4, 16, 4), np.int8)
    wr[...] = wq.reshape(16, I2, 4, 4, 3, 3).transpose(4, 5, 1, 2, 0, 3)
    sc = _al(scale[:16])
    sh = ol.aligned((T, 16), np.float32)
    sh[...] = shift[None, :16]
    tout = ol.aligned((oh * ow, 16), np.float32)
    rout = ol.aligned((oh * ow, 16), ol.NP_OF[kind])
    for ht in range(oh):
        for _wt in range(ow // T):
            rc = ref.ref_u8s8_conv3x3(KIND_ID[kind], T, I2, ih, ow, oh, ow, ht, _wt, 1, 1, 0.0, ol.FLT_MAX, ol.ptr(tout),
                                      ol.ptr(rout) if kind != ol.F32 else None, ol.ptr(xb), ol.ptr(wr), ol.ptr(sc),
                                      ol.ptr(sh))
            assert rc == 0
    return np.array(tout if kind == ol.F32 else rout)


# ---- the same two micro-kernels at stride 2 (template parameter S = 2) ---------------------------
def _s2_geometry(d):
    """ih = iw, top/left pad lp, right pad rp -> output size"""
    iw, lp, rp = int(d["iw"]), int(d["lp"]), int(d["rp"])
    ow = (iw + lp + rp - 3) // 2 + 1
    return iw, lp, rp, ow


def conv_s2_inputs(kind, iw, lp, rp, seed):
    rng = np.random.default_rng(seed)
    I2 = 2
    return dict(kind=np.int32(kind), iw=np.int32(iw), lp=np.int32(lp), rp=np.int32(rp),
                x=rng.integers(0, 256, (1, I2, iw, iw, 16)).astype(np.uint8),
                w=rng.normal(0, 0.05, (16, 16 * I2, 3, 3)).astype(np.float32),
                bias=rng.normal(0, 0.3, 16).astype(np.float32))


def _conv_s2_params(d):
    iw, lp, rp, ow = _s2_geometry(d)
    return ol.make_params(1, 32, 16, iw, iw, 3, 3, stride=2, out_type=int(d["kind"]), out_scale=0.02,
                          relu_hi=ol.FLT_MAX, pad_tl=lp, out_hw=(ow, ow))


def conv_s2_oracle(d):
    p = _conv_s2_params(d)
    wq, scale, shift, _ = ol.direct_prepare(p, ol.weights_to_blocked(d["w"]), d["bias"])
    out, _ = ol.direct_execute(p, d["x"], wq, scale, shift)
    return out.reshape(p.oh * p.ow, 16)


def conv_s2_reference(d, ref):
    p = _conv_s2_params(d)
    iw, lp, rp, ow = _s2_geometry(d)
    kind, I2, T = int(d["kind"]), 2, 7
    assert ow == T
    wq, scale, shift, _ = ol.direct_prepare(p, ol.weights_to_blocked(d["w"]), d["bias"])
    xb = ol.aligned(d["x"].size + 512, np.uint8)
    xb[:d["x"].size] = d["x"].ravel()
    wr = ol.aligned((3, 3, I2, 4, 16, 4), np.int8)
    wr[...] = wq.reshape(16, I2, 4, 4, 3, 3).transpose(4, 5, 1, 2, 0, 3)
    sc = _al(scale[:16])
    sh = ol.aligned((T, 16), np.float32)
    sh[...] = shift[None, :16]
    tout = ol.aligned((ow * ow, 16), np.float32)
    rout = ol.aligned((ow * ow, 16), ol.NP_OF[kind])
    for ht in range(ow):
        rc = ref.ref_u8s8_conv3x3_s2(KIND_ID[kind], T, I2, iw, iw, ow, ow, ht, 0, lp, lp, rp, 1, 0.0, ol.FLT_MAX,
                                     ol.ptr(tout), ol.ptr(rout) if kind != ol.F32 else None, ol.ptr(xb), ol.ptr(wr),
                                     ol.ptr(sc), ol.ptr(sh))
        assert rc == 0
    return np.array(tout if kind == ol.F32 else rout)


# 5x5 and 7x7 kernels: the reference's generic micro-kernel template, stride 1 or 2, one width block of 7
def convk_inputs(kind, K, S, iw, lp, rp, seed):
    rng = np.random.default_rng(seed)
    I2 = 2
    return dict(kind=np.int32(kind), K=np.int32(K), S=np.int32(S), iw=np.int32(iw), lp=np.int32(lp), rp=np.int32(rp),
                x=rng.integers(0, 256, (1, I2, iw, iw, 16)).astype(np.uint8),
                w=rng.normal(0, 0.03, (16, 16 * I2, K, K)).astype(np.float32),
                bias=rng.normal(0, 0.3, 16).astype(np.float32))


def _convk_geometry(d):
    K, S, iw, lp, rp = (int(d[k]) for k in ("K", "S", "iw", "lp", "rp"))
    ow = (iw + lp + rp - K) // S + 1
    assert ow == 7 and (ow - 1) * S + K == iw + lp + rp
    return K, S, iw, lp, rp, ow


def _convk_params(d):
    K, S, iw, lp, rp, ow = _convk_geometry(d)
    return ol.make_params(1, 32, 16, iw, iw, K, K, stride=S, out_type=int(d["kind"]), out_scale=0.02,
                          relu_hi=ol.FLT_MAX, pad_tl=lp, out_hw=(ow, ow))


def convk_oracle(d):
    p = _convk_params(d)
    wq, scale, shift, _ = ol.direct_prepare(p, ol.weights_to_blocked(d["w"]), d["bias"])
    out, _ = ol.direct_execute(p, d["x"], wq, scale, shift)
    return out.reshape(p.oh * p.ow, 16)


def convk_reference(d, ref):
    p = _convk_params(d)
    K, S, iw, lp, rp, ow = _convk_geometry(d)
    kind, I2, T = int(d["kind"]), 2, 7
    wq, scale, shift, _ = ol.direct_prepare(p, ol.weights_to_blocked(d["w"]), d["bias"])
    xb = ol.aligned(d["x"].size + 1024, np.uint8)
    xb[:d["x"].size] = d["x"].ravel()
    wr = ol.aligned((K, K, I2, 4, 16, 4), np.int8)
    wr[...] = wq.reshape(16, I2, 4, 4, K, K).transpose(4, 5, 1, 2, 0, 3)
    sc = _al(scale[:16])
    sh = ol.aligned((T, 16), np.float32)
    sh[...] = shift[None, :16]
    tout = ol.aligned((ow * ow, 16), np.float32)
    rout = ol.aligned((ow * ow, 16), ol.NP_OF[kind])
    for ht in range(ow):
        rc = ref.ref_u8s8_convk(K, S, KIND_ID[kind], I2, iw, iw, ow, ow, ht, lp, lp, rp, 1, 0.0, ol.FLT_MAX,
                                ol.ptr(tout), ol.ptr(rout) if kind != ol.F32 else None, ol.ptr(xb), ol.ptr(wr),
                                ol.ptr(sc), ol.ptr(sh))
        assert rc == 0, rc
    return np.array(tout if kind == ol.F32 else rout)


def dw_s2_inputs(kind, iw, lp, rp, T, seed):
    rng = np.random.default_rng(seed)
    return dict(kind=np.int32(kind), iw=np.int32(iw), lp=np.int32(lp), rp=np.int32(rp), T=np.int32(T),
                x=rng.integers(0, 256, (1, 2, iw, iw, 16)).astype(np.uint8),
                w=rng.normal(0, 0.1, (32, 3, 3)).astype(np.float32),
                bias=rng.normal(0, 0.5, 32).astype(np.float32))


def _dw_s2_params(d):
    iw, lp, rp, ow = _s2_geometry(d)
    kind = int(d["kind"])
    return ol.make_params(1, 32, 32, iw, iw, 3, 3, stride=2, g=32, out_type=kind, T=int(d["T"]),
                          out_scale=6.0 / 255.0, relu_hi=255.0 if kind == ol.U8 else 127.0, pad_tl=lp, out_hw=(ow, ow))


def dw_s2_oracle(d):
    p = _dw_s2_params(d)
    wq, scale, shift, _ = ol.depthwise_prepare(p, d["w"], d["bias"])
    out, _ = ol.depthwise_execute(p, d["x"], wq, scale, shift)
    return out.reshape(2, p.oh * p.ow, 16)


def dw_s2_reference(d, ref):
    p = _dw_s2_params(d)
    iw, lp, rp, ow = _s2_geometry(d)
    G2, T, kind = 2, int(d["T"]), int(d["kind"])
    wq, scale, shift, _ = ol.depthwise_prepare(p, d["w"], d["bias"])
    xb = ol.aligned(d["x"].size + 512, np.uint8)
    xb[:d["x"].size] = d["x"].ravel()
    wr = ol.aligned((G2, 3, 16, 4), np.int8)
    wr[...] = 0
    wr[:, :, :, :3] = wq.reshape(G2, 16, 3, 3).transpose(0, 2, 1, 3)
    sc, sh = _al(scale.reshape(G2, 16)), _al(shift.reshape(G2, 16))
    got = ol.aligned((G2, ow * ow, 16), ol.NP_OF[kind])
    wt = (ow + T - 1) // T
    Tr = ow % T or T
    for ht in range(ow):
        for _wt in range(wt):
            Tz = Tr if _wt == wt - 1 else T
            rc = ref.ref_u8s8_depthwise_s2(KIND_ID[kind], T, Tz, G2, iw, iw, ow, ow, ht, _wt, lp, lp, rp, 1, 0.0,
                                           float(p.relu_hi), ol.ptr(got), ol.ptr(xb), ol.ptr(wr), ol.ptr(sc), ol.ptr(sh))
            assert rc == 0
    return np.array(got)


# ---- Winograd F(4x4,3x3) tile transforms (src/kernel/elk_conv_wino_4x4_3x3_*.hxx) ----------------
def wino_w_inputs(seed):
    return dict(w=np.random.default_rng(seed).normal(0, 0.05, (3, 3, 16, 16)).astype(np.float32))


def wino_w_reference(d, ref):
    tw = ol.aligned((6, 6, 16, 16), np.float32)
    w = _al(d["w"])
    ref.ref_wino_trans_weights(ol.ptr(tw), ol.ptr(w))
    return np.array(tw)


def wino_w_oracle(d):
    out = np.zeros((6, 6, 16, 16), np.float32)
    u = np.zeros(36, np.float32)
    for i in range(16):
        for o in range(16):
            g = np.ascontiguousarray(d["w"][:, :, i, o].ravel())
            ol.oracle().orc_wino_tile_weights(ol.ptr(g), ol.ptr(u))
            out[:, :, i, o] = u.reshape(6, 6)
    return out


def wino_in_inputs(h0, w0, seed):
    return dict(h0=np.int32(h0), w0=np.int32(w0),
                plane=np.random.default_rng(seed).uniform(0, 1, (12, 12, 16)).astype(np.float32))


def _wino_in_range(d):
    ih = iw = 12
    h0, w0 = int(d["h0"]), int(d["w0"])
    hs, he = max(0, -h0), min(5, ih - 1 - h0)
    ws, we = max(0, -w0), min(5, iw - 1 - w0)
    return h0, w0, hs, he, ws, we, not (hs == 0 and ws == 0 and he == 5 and we == 5)


def wino_in_reference(d, ref):
    h0, w0, hs, he, ws, we, border = _wino_in_range(d)
    plane = _al(d["plane"])
    tin = ol.aligned((6, 6, 16), np.float32)
    tile_ptr = ctypes.c_void_p(plane.ctypes.data + (h0 * 12 + w0) * 16 * 4)
    ref.ref_wino_trans_input(int(border), 12, 12, ol.ptr(tin), tile_ptr, hs, he, ws, we)
    return np.array(tin)


def wino_in_oracle(d):
    h0, w0, hs, he, ws, we, border = _wino_in_range(d)
    out = np.zeros((6, 6, 16), np.float32)
    v = np.zeros(36, np.float32)
    for c in range(16):
        t = np.zeros((6, 6), np.float32)
        for i in range(6):
            for j in range(6):
                h, w = h0 + i, w0 + j
                if 0 <= h < 12 and 0 <= w < 12:
                    t[i, j] = d["plane"][h, w, c]
        fn = ol.oracle().orc_wino_tile_input_border if border else ol.oracle().orc_wino_tile_input
        fn(ol.ptr(t), ol.ptr(v))
        out[:, :, c] = v.reshape(6, 6)
    return out


def wino_out_inputs(with_bias, with_relu, h_end, w_end, seed):
    rng = np.random.default_rng(seed)
    return dict(with_bias=np.int32(with_bias), with_relu=np.int32(with_relu), h_end=np.int32(h_end), w_end=np.int32(w_end),
                m=rng.normal(0, 3, (6, 6, 16)).astype(np.float32), bias=rng.normal(0, 1, 16).astype(np.float32))


def wino_out_reference(d, ref):
    out = ol.aligned((8, 8, 16), np.float32, -777.0)
    h_end, w_end = int(d["h_end"]), int(d["w_end"])
    border = not (h_end == 3 and w_end == 3)
    m, bias = _al(d["m"]), _al(d["bias"])
    ref.ref_wino_trans_output(int(border), int(d["with_bias"]), int(d["with_relu"]), 8, 8, ol.ptr(out), ol.ptr(m),
                              ol.ptr(bias), h_end, w_end)
    return np.array(out[:4, :4, :])


def wino_out_oracle(d):
    out = np.full((4, 4, 16), -777.0, np.float32)
    y = np.zeros(16, np.float32)
    for c in range(16):
        mm = np.ascontiguousarray(d["m"][:, :, c].ravel())
        ol.oracle().orc_wino_tile_output(ol.ptr(mm), ol.ptr(y))
        for i in range(4):
            for j in range(4):
                if i > int(d["h_end"]) or j > int(d["w_end"]):
                    continue
                r = y[4 * i + j]
                if int(d["with_bias"]):
                    r = np.float32(r + d["bias"][c])
                if int(d["with_relu"]):
                    r = r if r > 0 else np.float32(0)
                out[i, j, c] = r
    return out


# quantized store of the output transform (u8 / s8 user output)
def wino_outq_inputs(kind, with_bias, with_relu, h_end, w_end, seed):
    d = wino_out_inputs(with_bias, with_relu, h_end, w_end, seed)
    d["kind"] = np.int32(kind)
    d["out_scale"] = np.float32(0.0437)   # values of a few units land all over (and outside) the code range
    d["out_z"] = np.float32(0.0 if kind == ol.S8 else 3.0)
    return d


def wino_outq_reference(d, ref):
    kind = int(d["kind"])
    out = ol.aligned((8, 8, 16), ol.NP_OF[kind], 99)
    h_end, w_end = int(d["h_end"]), int(d["w_end"])
    border = not (h_end == 3 and w_end == 3)
    m, bias = _al(d["m"]), _al(d["bias"])
    rep = np.float32(1.0) / d["out_scale"]
    ref.ref_wino_trans_output_q(KIND_ID[kind], int(border), int(d["with_bias"]), int(d["with_relu"]), 8, 8, ol.ptr(out),
                                ol.ptr(m), ol.ptr(bias), h_end, w_end, float(rep), float(np.ceil(d["out_z"])))
    return np.array(out[:4, :4, :])


def wino_outq_oracle(d):
    kind = int(d["kind"])
    out = np.full((4, 4, 16), 99, ol.NP_OF[kind])
    y = np.zeros(16, np.float32)
    fn = ol.oracle().orc_wino_output_value
    fn.argtypes = [ctypes.c_float, ctypes.c_int, ctypes.c_float, ctypes.c_int, ctypes.c_float, ctypes.c_float, ctypes.c_int,
                   ctypes.c_void_p]
    for c in range(16):
        mm = np.ascontiguousarray(d["m"][:, :, c].ravel())
        ol.oracle().orc_wino_tile_output(ol.ptr(mm), ol.ptr(y))
        for i in range(4):
            for j in range(4):
                if i > int(d["h_end"]) or j > int(d["w_end"]):
                    continue
                q = fn(float(y[4 * i + j]), int(d["with_bias"]), float(d["bias"][c]), kind, float(d["out_scale"]),
                       float(d["out_z"]), int(d["with_relu"]), None)
                out[i, j, c] = np.array(q).astype(ol.NP_OF[kind])
    return out


# name -> (inputs, reference runner, oracle runner)
CASES = {}
for _k, _kn in ((ol.F32, "f32"), (ol.U8, "u8"), (ol.S8, "s8")):
    for _sum in (0, 1):
        if _k == ol.F32 and _sum:
            continue  # the reference has no sum fusion for f32 output (elk_u8s8_gemm.hxx:234-236)
        CASES["gemm_%s_sum%d" % (_kn, _sum)] = (lambda k=_k, s=_sum: gemm_inputs(k, 2, 6, s, 7 + k + 10 * s),
                                                gemm_reference, gemm_oracle)
for _T, _ow, _ih in ((14, 56, 5), (7, 7, 7), (11, 28, 3), (7, 21, 3)):
    CASES["depthwise_u8_T%d_w%d" % (_T, _ow)] = (lambda T=_T, ow=_ow, ih=_ih: dw_inputs(T, ow, ih, ol.U8, 100 + T + ow, 255.0),
                                                 dw_reference, dw_oracle)
CASES["depthwise_s8_T14_w28"] = (lambda: dw_inputs(14, 28, 4, ol.S8, 5, 127.0), dw_reference, dw_oracle)
for _k, _kn, _T, _ow in ((ol.U8, "u8", 14, 28), (ol.S8, "s8", 7, 14), (ol.F32, "f32", 7, 7)):
    CASES["conv3x3_%s_T%d_w%d" % (_kn, _T, _ow)] = (lambda k=_k, T=_T, ow=_ow: conv_inputs(k, T, ow, 3 * T + ow + k),
                                                    conv_reference, conv_oracle)
# stride 2: pre-padded input (no pads) and top / left pads.  No right pad for the direct kernel: the
# reference's 3x3-specialised template reads behind the row's end there (see oracle/ref_kernels.cpp),
# so its output is not a convolution for those shapes; the depthwise kernel masks the tap and is
# covered with right pads as well.
for _k, _kn, _iw, _lp, _rp in ((ol.U8, "u8", 15, 0, 0), (ol.S8, "s8", 14, 1, 0), (ol.F32, "f32", 15, 0, 0), (ol.U8, "u8", 14, 1, 0)):
    CASES["conv3x3_s2_%s_w%d_l%d_r%d" % (_kn, _iw, _lp, _rp)] = (
        lambda k=_k, iw=_iw, lp=_lp, rp=_rp: conv_s2_inputs(k, iw, lp, rp, 300 + iw + 2 * lp + rp + k), conv_s2_reference,
        conv_s2_oracle)
# 5x5 / 7x7.  The template takes its column bounds per tap from k/2 and the stride, not from the pads it
# is given (src/kernel/elk_u8s8_conv.hxx:312-470), so it is the convolution only for the pad sets it was
# written for: stride 1 with k/2 on both sides; stride 2 with (k/2, k/2 - 1) -- the "lean left padding"
# instantiation -- or (k/2 - 1, k/2), and 5x5 with (1, 1).  Elsewhere it reads a pixel of the neighbouring
# row or drops a valid tap (7x7 s2 pads (2, 2): column 5 differs; (3, 3): column 1; stride 1 pads (3, 2):
# columns 4-5), and the oracle and the product compute the convolution.  The cases below are the exact ones,
# which include every shape of the reference's tuned runs.
for _k, _kn, _K, _S, _iw, _lp, _rp in ((ol.U8, "u8", 5, 1, 7, 2, 2), (ol.S8, "s8", 5, 1, 7, 2, 2), (ol.F32, "f32", 5, 1, 7, 2, 2),
                                       (ol.U8, "u8", 7, 2, 14, 3, 2), (ol.S8, "s8", 7, 2, 14, 2, 3), (ol.F32, "f32", 7, 2, 14, 3, 2),
                                       (ol.U8, "u8", 5, 2, 15, 1, 1), (ol.S8, "s8", 7, 1, 7, 3, 3)):
    CASES["conv%dx%d_s%d_%s_w%d_l%d_r%d" % (_K, _K, _S, _kn, _iw, _lp, _rp)] = (
        lambda k=_k, K=_K, S=_S, iw=_iw, lp=_lp, rp=_rp: convk_inputs(k, K, S, iw, lp, rp, 500 + 10 * K + iw + 2 * lp + rp + k),
        convk_reference, convk_oracle)
for _k, _kn, _iw, _lp, _rp, _T in ((ol.U8, "u8", 15, 0, 0, 7), (ol.U8, "u8", 14, 0, 1, 7), (ol.S8, "s8", 13, 1, 1, 7),
                                   (ol.U8, "u8", 21, 1, 1, 7)):
    CASES["depthwise_s2_%s_w%d_l%d_r%d" % (_kn, _iw, _lp, _rp)] = (
        lambda k=_k, iw=_iw, lp=_lp, rp=_rp, T=_T: dw_s2_inputs(k, iw, lp, rp, T, 400 + iw + 2 * lp + rp + k), dw_s2_reference,
        dw_s2_oracle)
for _k, _kn, _b, _r, _he, _we in ((ol.U8, "u8", 1, 1, 3, 3), (ol.U8, "u8", 1, 0, 3, 3), (ol.U8, "u8", 1, 1, 2, 1),
                                  (ol.U8, "u8", 0, 0, 1, 3), (ol.S8, "s8", 1, 1, 3, 3), (ol.S8, "s8", 0, 0, 3, 3),
                                  (ol.S8, "s8", 1, 0, 3, 2), (ol.S8, "s8", 1, 1, 0, 0)):
    CASES["wino_output_%s_b%d_r%d_h%d_w%d" % (_kn, _b, _r, _he, _we)] = (
        lambda k=_k, b=_b, r=_r, he=_he, we=_we: wino_outq_inputs(k, b, r, he, we, 500 + 16 * k + 8 * b + 4 * r + he + we),
        wino_outq_reference, wino_outq_oracle)
CASES["wino_weights"] = (lambda: wino_w_inputs(21), wino_w_reference, wino_w_oracle)
for _h0, _w0 in ((2, 3), (-1, -1), (-1, 4), (3, -1), (7, 7), (7, 2), (-1, 7)):
    CASES["wino_input_h%d_w%d" % (_h0, _w0)] = (lambda h=_h0, w=_w0: wino_in_inputs(h, w, h * 13 + w + 50),
                                                wino_in_reference, wino_in_oracle)
for _b, _r, _he, _we in ((1, 1, 3, 3), (1, 0, 1, 3), (0, 0, 3, 0), (1, 1, 2, 2)):
    CASES["wino_output_b%d_r%d_h%d_w%d" % (_b, _r, _he, _we)] = (
        lambda b=_b, r=_r, he=_he, we=_we: wino_out_inputs(b, r, he, we, 77 + he * 4 + we), wino_out_reference,
        wino_out_oracle)


# ---- the other Winograd tile sizes: A = 4 F(2x2,3x3) (src/kernel/elk_conv_wino_2x2_3x3_*.hxx) and
# A = 5 F(3x3,3x3) (src/kernel/elk_conv_wino_3x3_3x3_*.hxx) -------------------------------------------
def winoa_w_inputs(A, seed):
    d = wino_w_inputs(seed)
    d["A"] = np.int32(A)
    return d


def winoa_w_reference(d, ref):
    A = int(d["A"])
    tw = ol.aligned((A, A, 16, 16), np.float32)
    w = _al(d["w"])
    assert ref.ref_wino_trans_weights_a(A, ol.ptr(tw), ol.ptr(w)) == 0
    return np.array(tw)


def winoa_w_oracle(d):
    A = int(d["A"])
    out = np.zeros((A, A, 16, 16), np.float32)
    u = np.zeros(A * A, np.float32)
    for i in range(16):
        for o in range(16):
            g = np.ascontiguousarray(d["w"][:, :, i, o].ravel())
            ol.oracle().orc_wino_tile_weights_a(A, ol.ptr(g), ol.ptr(u))
            out[:, :, i, o] = u.reshape(A, A)
    return out


def winoa_in_inputs(A, h0, w0, seed):
    d = wino_in_inputs(h0, w0, seed)
    d["A"] = np.int32(A)
    return d


def _winoa_in_range(d):
    A = int(d["A"])
    h0, w0 = int(d["h0"]), int(d["w0"])
    hs, he = max(0, -h0), min(A - 1, 11 - h0)
    ws, we = max(0, -w0), min(A - 1, 11 - w0)
    return A, h0, w0, hs, he, ws, we, not (hs == 0 and ws == 0 and he == A - 1 and we == A - 1)


def winoa_in_reference(d, ref):
    A, h0, w0, hs, he, ws, we, border = _winoa_in_range(d)
    plane = _al(d["plane"])
    tin = ol.aligned((A, A, 16), np.float32)
    tile_ptr = ctypes.c_void_p(plane.ctypes.data + (h0 * 12 + w0) * 16 * 4)
    assert ref.ref_wino_trans_input_a(A, int(border), 12, 12, ol.ptr(tin), tile_ptr, hs, he, ws, we) == 0
    return np.array(tin)


def winoa_in_oracle(d):
    A, h0, w0, hs, he, ws, we, border = _winoa_in_range(d)
    out = np.zeros((A, A, 16), np.float32)
    v = np.zeros(A * A, np.float32)
    for c in range(16):
        t = np.zeros((A, A), np.float32)
        for i in range(A):
            for j in range(A):
                h, w = h0 + i, w0 + j
                if 0 <= h < 12 and 0 <= w < 12:
                    t[i, j] = d["plane"][h, w, c]
        ol.oracle().orc_wino_tile_input_a(A, int(border), ol.ptr(t), ol.ptr(v))
        out[:, :, c] = v.reshape(A, A)
    return out


def winoa_out_inputs(A, kind, with_bias, with_relu, h_end, w_end, seed):
    rng = np.random.default_rng(seed)
    return dict(A=np.int32(A), kind=np.int32(kind), with_bias=np.int32(with_bias), with_relu=np.int32(with_relu),
                h_end=np.int32(h_end), w_end=np.int32(w_end), m=rng.normal(0, 3, (A, A, 16)).astype(np.float32),
                bias=rng.normal(0, 1, 16).astype(np.float32), out_scale=np.float32(0.0437),
                out_z=np.float32(3.0 if kind == ol.U8 else 0.0))


def winoa_out_reference(d, ref):
    A, kind = int(d["A"]), int(d["kind"])
    M = A - 2
    fill = -777.0 if kind == ol.F32 else 99
    out = ol.aligned((8, 8, 16), ol.NP_OF[kind], fill)
    h_end, w_end = int(d["h_end"]), int(d["w_end"])
    border = not (h_end == M - 1 and w_end == M - 1)
    m, bias = _al(d["m"]), _al(d["bias"])
    rep = np.float32(1.0) / d["out_scale"]
    assert ref.ref_wino_trans_output_a(A, KIND_ID[kind], int(border), int(d["with_bias"]), int(d["with_relu"]), 8, 8,
                                       ol.ptr(out), ol.ptr(m), ol.ptr(bias), h_end, w_end, float(rep),
                                       float(np.ceil(d["out_z"]))) == 0
    return np.array(out[:M, :M, :])


def winoa_out_oracle(d):
    A, kind = int(d["A"]), int(d["kind"])
    M = A - 2
    out = np.full((M, M, 16), -777.0 if kind == ol.F32 else 99, ol.NP_OF[kind])
    y = np.zeros(M * M, np.float32)
    for c in range(16):
        mm = np.ascontiguousarray(d["m"][:, :, c].ravel())
        ol.oracle().orc_wino_tile_output_a(A, ol.ptr(mm), ol.ptr(y))
        for i in range(M):
            for j in range(M):
                if i > int(d["h_end"]) or j > int(d["w_end"]):
                    continue
                r = ctypes.c_float()
                q = ol.oracle().orc_wino_output_value_a(A, float(y[M * i + j]), int(d["with_bias"]), float(d["bias"][c]), kind,
                                                        float(d["out_scale"]), float(d["out_z"]), int(d["with_relu"]),
                                                        ctypes.byref(r))
                out[i, j, c] = r.value if kind == ol.F32 else np.array(q).astype(ol.NP_OF[kind])
    return out


for _A in (4, 5):
    CASES["wino%d_weights" % _A] = (lambda A=_A: winoa_w_inputs(A, 21 + A), winoa_w_reference, winoa_w_oracle)
    for _h0, _w0 in ((2, 2), (1, 3), (-1, -1), (-1, 4), (3, -1), (9, 9), (8, 2), (-1, 9)):
        CASES["wino%d_input_h%d_w%d" % (_A, _h0, _w0)] = (
            lambda A=_A, h=_h0, w=_w0: winoa_in_inputs(A, h, w, h * 13 + w + 50 + A), winoa_in_reference, winoa_in_oracle)
    for _k, _kn in ((ol.F32, "f32"), (ol.U8, "u8"), (ol.S8, "s8")):
        for _b, _r, _he, _we in ((1, 1, _A - 3, _A - 3), (1, 0, 0, _A - 3), (0, 0, _A - 3, _A - 4)):
            CASES["wino%d_output_%s_b%d_r%d_h%d_w%d" % (_A, _kn, _b, _r, _he, _we)] = (
                lambda A=_A, k=_k, b=_b, r=_r, he=_he, we=_we: winoa_out_inputs(A, k, b, r, he, we, 700 + 16 * k + 8 * b + he + we + A),
                winoa_out_reference, winoa_out_oracle)


# ---- in-place sum fused into the Winograd output transform (with_ip_sum = true) -------------------
def winos_out_inputs(A, kind, with_bias, with_relu, border, seed):
    M = A - 2
    h_end, w_end = (M - 2, M - 1) if border else (M - 1, M - 1)
    d = winoa_out_inputs(A, kind, with_bias, with_relu, h_end, w_end, seed)
    rng = np.random.default_rng(seed + 1)
    if kind == ol.F32:
        d["old"] = rng.normal(0, 2, (8, 8, 16)).astype(np.float32)
    else:
        d["old"] = rng.integers(-100 if kind == ol.S8 else 0, 100, (8, 8, 16)).astype(ol.NP_OF[kind])
    return d


def winos_out_reference(d, ref):
    A, kind = int(d["A"]), int(d["kind"])
    M = A - 2
    out = ol.aligned((8, 8, 16), ol.NP_OF[kind])
    out[...] = d["old"]
    h_end, w_end = int(d["h_end"]), int(d["w_end"])
    border = not (h_end == M - 1 and w_end == M - 1)
    m, bias = _al(d["m"]), _al(d["bias"])
    rep = np.float32(1.0) / d["out_scale"]
    assert ref.ref_wino_trans_output_sum(A, KIND_ID[kind], int(border), int(d["with_bias"]), int(d["with_relu"]), 8, 8,
                                         ol.ptr(out), ol.ptr(m), ol.ptr(bias), h_end, w_end, float(rep),
                                         float(np.ceil(d["out_z"]))) == 0
    return np.array(out[:M, :M, :])


def winos_out_oracle(d):
    A, kind = int(d["A"]), int(d["kind"])
    M = A - 2
    out = np.array(d["old"][:M, :M, :])
    y = np.zeros(M * M, np.float32)
    for c in range(16):
        mm = np.ascontiguousarray(d["m"][:, :, c].ravel())
        ol.oracle().orc_wino_tile_output_a(A, ol.ptr(mm), ol.ptr(y))
        for i in range(M):
            for j in range(M):
                if i > int(d["h_end"]) or j > int(d["w_end"]):
                    continue
                r = ctypes.c_float()
                q = ol.oracle().orc_wino_output_value_sum(A, float(y[M * i + j]), int(d["with_bias"]), float(d["bias"][c]), kind,
                                                          float(d["out_scale"]), float(d["out_z"]), int(d["with_relu"]), 1,
                                                          float(d["old"][i, j, c]), ctypes.byref(r))
                out[i, j, c] = r.value if kind == ol.F32 else np.array(q).astype(ol.NP_OF[kind])
    return out


for _A in (6, 4, 5):
    for _k, _kn in ((ol.F32, "f32"), (ol.U8, "u8"), (ol.S8, "s8")):
        for _b, _r, _bd in ((1, 1, 0), (1, 0, 1)):
            CASES["wino%d_output_sum_%s_b%d_r%d_border%d" % (_A, _kn, _b, _r, _bd)] = (
                lambda A=_A, k=_k, b=_b, r=_r, bd=_bd: winos_out_inputs(A, k, b, r, bd, 800 + 16 * k + 8 * b + bd + A),
                winos_out_reference, winos_out_oracle)


# ---- Winograd quantization glue: whole small layers through the reference's transform CLASSES ------
# (src/elx_conv_wino_trans_input.cpp:599-654: tile gather, interior / border kernels, a * mrepS + mz ->
#  cvt_roundps_epu32 -> saturate; src/elx_conv_wino_trans_weights.cpp:175-195,437-535: U = G g Gt, per
#  (position, oc) abs-max quantization, scale = absmax / 127 * tin_S, shift = -sum * scale * ceil(tin_z)).
# The reference side is the pair of translation units compiled from the reference tree
# (oracle/ref_wino_glue.cpp); the `ref` argument of the other cases is not used here.
def glue_in_inputs(A, in_u8, n, ic, hw, pad, T, tin_scale, tin_z, seed, lo=-1.0, hi=2.0):
    rng = np.random.default_rng(seed)
    if in_u8:
        x = rng.integers(0, 256, (n, ic, hw, hw)).astype(np.float32)
    else:
        x = rng.uniform(lo, hi, (n, ic, hw, hw)).astype(np.float32)
    return dict(A=np.int32(A), in_u8=np.int32(in_u8), n=np.int32(n), ic=np.int32(ic), hw=np.int32(hw), pad=np.int32(pad),
                T=np.int32(T), in_scale=np.float32(1.0 / 255.0 if in_u8 else 1.0), tin_scale=np.float32(tin_scale),
                tin_z=np.float32(tin_z), x=ol.to_blocked(x))


def _glue_params(d):
    hw, pad = int(d["hw"]), int(d["pad"])
    return ol.make_params(int(d["n"]), int(d["ic"]), 16, hw, hw, 3, 3, pad, out_type=ol.F32, in_scale=float(d["in_scale"]),
                          tin_scale=float(d["tin_scale"]), tin_z=float(d["tin_z"]), wino_tile=int(d["A"]))


def glue_in_reference(d, ref):
    glue = ol.ref_wino_glue()
    assert glue is not None, "oracle/_ref/libeuler_ref_wino_glue.so is not built"
    p = _glue_params(d)
    A, t = int(d["A"]), ol.wino_tiles(p)
    out = np.zeros((A * A, ol.up16(p.ic) // 16, t, 16), np.uint8)
    x = _al(d["x"].astype(np.uint8) if int(d["in_u8"]) else d["x"])
    assert glue.ref_wino_glue_trans_input(A, int(d["in_u8"]), p.n, p.ic, p.ih, p.iw, p.oh, p.ow, p.pad_t, p.pad_l, int(d["T"]),
                                          float(d["in_scale"]), float(d["tin_scale"]), float(d["tin_z"]), ol.ptr(x),
                                          ol.ptr(out)) == 0
    return out


def glue_in_oracle(d):
    return ol.wino_trans_input(_glue_params(d), np.ascontiguousarray(d["x"], np.float32))


def glue_range_reference(d, ref):
    glue = ol.ref_wino_glue()
    assert glue is not None, "oracle/_ref/libeuler_ref_wino_glue.so is not built"
    p = _glue_params(d)
    A, t = int(d["A"]), ol.wino_tiles(p)
    tin = np.zeros((A * A, ol.up16(p.ic) // 16, t, 16), np.float32)
    x = _al(d["x"])
    assert glue.ref_wino_glue_trans_input_f32(A, p.n, p.ic, p.ih, p.iw, p.oh, p.ow, p.pad_t, p.pad_l, int(d["T"]), ol.ptr(x),
                                              ol.ptr(tin)) == 0
    # min / max over the transformed input as the harness takes it (tests/elt_conv_utils.cpp:222-262); the
    # zero-filled channel tail of the last 16-channel unit is not part of the tensor
    c = np.arange(tin.shape[1] * 16).reshape(tin.shape[1], 1, 16) < p.ic
    real = tin[np.broadcast_to(c[None], tin.shape)]
    return np.array([real.min(), real.max()], np.float32)


def glue_range_oracle(d):
    mn, mx = ol.wino_tinput_range(_glue_params(d), np.ascontiguousarray(d["x"], np.float32))
    return np.array([mn, mx], np.float32)


def glue_w_inputs(A, ic, oc, tin_scale, tin_z, seed):
    rng = np.random.default_rng(seed)
    w = rng.normal(0, 0.02, (oc, ic, 3, 3)).astype(np.float32)
    return dict(A=np.int32(A), ic=np.int32(ic), oc=np.int32(oc), tin_scale=np.float32(tin_scale), tin_z=np.float32(tin_z),
                w=ol.weights_to_blocked(w))


def _pack3(twq, tscale, tshift):
    return np.concatenate([np.ascontiguousarray(a).ravel().view(np.uint8) for a in (twq, tscale, tshift)])


def glue_w_reference(d, ref):
    glue = ol.ref_wino_glue()
    assert glue is not None, "oracle/_ref/libeuler_ref_wino_glue.so is not built"
    A, ic, oc = int(d["A"]), int(d["ic"]), int(d["oc"])
    twq = np.zeros((A * A, ol.up16(oc), ol.up16(ic)), np.int8)
    tscale = np.zeros((A * A, ol.up16(oc)), np.float32)
    tshift = np.zeros((A * A, ol.up16(oc)), np.float32)
    w = _al(d["w"])
    assert glue.ref_wino_glue_trans_weights(A, ic, oc, float(d["tin_scale"]), float(d["tin_z"]), ol.ptr(w), ol.ptr(twq),
                                            ol.ptr(tscale), ol.ptr(tshift)) == 0
    return _pack3(twq, tscale, tshift)


def glue_w_oracle(d):
    p = ol.make_params(1, int(d["ic"]), int(d["oc"]), 8, 8, 3, 3, 1, out_type=ol.F32, in_scale=1.0,
                       tin_scale=float(d["tin_scale"]), tin_z=float(d["tin_z"]), wino_tile=int(d["A"]))
    return _pack3(*ol.wino_prepare(p, np.ascontiguousarray(d["w"])))


def tie_values(m, z):
    """f32 values v for which fma(v, m, z) (one rounding) and (v * m) + z (two roundings) land on different
    sides of a rounding boundary of the final float -> integer conversion: one candidate search around every
    code k + 0.5.  Evaluated in 64-bit-mantissa long doubles, where v * m + z is exact."""
    L = np.longdouble
    m, z, out = np.float32(m), np.float32(z), []
    for k in range(0, 255):
        base = np.float32((np.float64(k) + 0.5 - np.float64(z)) / np.float64(m))
        bits = np.array([base], np.float32).view(np.int32)[0]
        cand = (bits + np.arange(-64, 65, dtype=np.int32)).view(np.float32)
        fused = (cand.astype(L) * L(m) + L(z)).astype(np.float32)
        unfused = (cand * m).astype(np.float32) + z
        hit = np.rint(fused) != np.rint(unfused)
        out.extend(cand[hit][:1].tolist())
    return np.array(out, np.float32)


def glue_ties_sites(A, hw):
    """pixels that are element (A-1, A-1) of an even-numbered tile and element (1, 1) of none that holds
    another such pixel (pad 1): rows / columns M * (2a + 1)"""
    M = A - 2
    r = np.arange(M, hw, 2 * M)
    return [(int(h), int(w)) for h in r for w in r]


def glue_ties_inputs(A, tin_scale, tin_z):
    """all-zero image except single pixels that carry tie_values: the transform hands such a value through
    unchanged to position (A-1, A-1) of its tile, so the quantization a * mrepS + mz sees exactly it"""
    M = A - 2
    hw = 8 * M
    v = tie_values(np.float32(1.0) * (np.float32(1.0) / np.float32(tin_scale)), np.ceil(np.float32(tin_z)))
    x = np.zeros((1, 16, hw, hw), np.float32)
    sites = glue_ties_sites(A, hw)
    for i, val in enumerate(v[:16 * len(sites)]):
        h, w = sites[i % len(sites)]
        x[0, i // len(sites), h, w] = val
    return dict(A=np.int32(A), in_u8=np.int32(0), n=np.int32(1), ic=np.int32(16), hw=np.int32(hw), pad=np.int32(1),
                T=np.int32(6), in_scale=np.float32(1.0), tin_scale=np.float32(tin_scale), tin_z=np.float32(tin_z),
                x=ol.to_blocked(x))


for _A in (6, 4, 5):
    # values chosen so that a dropped fusion in a * mrepS + mz changes the code
    CASES["wino_glue_input%d_ties" % _A] = (lambda A=_A: glue_ties_inputs(A, 0.0283, 40.37), glue_in_reference, glue_in_oracle)
    # f32 input with negative values, ragged last block of tiles (T = 5), every border kind (the image is not
    # a multiple of the output tile), a zero point with a fractional part (ceil) placed so that part of the
    # values round below zero (the float -> unsigned conversion's 255) and part saturate at 255
    CASES["wino_glue_input%d_f32" % _A] = (lambda A=_A: glue_in_inputs(A, 0, 2, 24, 10, 1, 5, 0.0283, 40.37, 900 + A),
                                           glue_in_reference, glue_in_oracle)
    # no padding: only right / bottom borders
    CASES["wino_glue_input%d_f32_nopad" % _A] = (lambda A=_A: glue_in_inputs(A, 0, 1, 16, 11, 0, 4, 0.05, 63.5, 910 + A),
                                                 glue_in_reference, glue_in_oracle)
    # u8 codes as input (U8F32*F32 user types): in_S / tin_S enters the factor
    CASES["wino_glue_input%d_u8" % _A] = (lambda A=_A: glue_in_inputs(A, 1, 2, 32, 9, 1, 7, 0.1171, 101.2, 920 + A),
                                          glue_in_reference, glue_in_oracle)
    CASES["wino_glue_range%d" % _A] = (lambda A=_A: glue_in_inputs(A, 0, 2, 24, 10, 1, 5, 1.0, 0.0, 930 + A, -3.0, 5.0),
                                       glue_range_reference, glue_range_oracle)
    CASES["wino_glue_weights%d" % _A] = (lambda A=_A: glue_w_inputs(A, 24, 32, 0.0283, 40.37, 940 + A),
                                         glue_w_reference, glue_w_oracle)
    CASES["wino_glue_weights%d_negz" % _A] = (lambda A=_A: glue_w_inputs(A, 48, 16, 0.4071, -12.6, 950 + A),
                                              glue_w_reference, glue_w_oracle)


# ---- the test harness: fp32 reference convolution, scale calibration, quantization of the input and of the
# sum operand (tests/elt_conv_utils.cpp:87-463, :666-750) -------------------------------------------------------
# The harness draws its own tensors (a default-seeded std::normal_distribution for input and weights, rand_r
# seeded from the clock for bias and sum operand), so the stored inputs of these cases are what the compiled
# harness produced, not something this file can regenerate: make_inputs() holds the layer only and the
# reference run adds the tensors before the fixture is written.
HARNESS_REPRESENTATION = 127.0   # PRECISION_REPRESENTATION_7B, used by the harness for every type


def harness_config(out_s8, zero_point, n, g, ic, oc, hw, k, pad, stride, with_relu, with_sum):
    oh = (hw + 2 * pad - k) // stride + 1
    return dict(out_s8=np.int32(out_s8), zero_point=np.int32(zero_point), n=np.int32(n), g=np.int32(g), ic=np.int32(ic),
                oc=np.int32(oc), hw=np.int32(hw), k=np.int32(k), pad=np.int32(pad), stride=np.int32(stride), oh=np.int32(oh),
                with_relu=np.int32(with_relu), with_sum=np.int32(with_sum))


def _harness_pack(quant, input_q, sum_q, conv_out):
    return np.concatenate([np.ascontiguousarray(quant, np.float32).view(np.uint8).ravel(), input_q.ravel(), sum_q.ravel(),
                           np.ascontiguousarray(conv_out, np.float32).view(np.uint8).ravel()])


def harness_reference(d, _ref):
    lib = ol.ref_harness()
    assert lib is not None, "oracle/_ref/libeuler_ref_harness.so is not built"
    n, g, ic, oc, hw, k, pad, stride, oh = (int(d[key]) for key in ("n", "g", "ic", "oc", "hw", "k", "pad", "stride", "oh"))
    x = np.zeros((n, ic, hw, hw), np.float32)
    w = np.zeros((oc, ic // g, k, k), np.float32)
    out = np.zeros((n, oc, oh, oh), np.float32)
    bias = np.zeros(oc, np.float32)
    xq = np.zeros(x.shape, np.uint8)
    sq = np.zeros(out.shape, np.uint8)
    quant = np.zeros(5, np.float32)
    lib.ref_harness_prepare(int(d["out_s8"]), int(d["zero_point"]), n, g, ic, oc, hw, hw, oh, oh, k, k, pad, pad, stride, stride,
                            int(d["with_relu"]), int(d["with_sum"]), ol.ptr(x), ol.ptr(w), ol.ptr(out), ol.ptr(bias),
                            ol.ptr(xq), ol.ptr(sq), ol.ptr(quant))
    if int(d["with_sum"]):
        sum_operand = out.copy()
    else:
        sum_operand = np.zeros_like(out)   # without a sum the harness leaves the convolution result there
    conv = sum_operand.copy()
    lib.ref_harness_conv2d(n, g, ic, oc, hw, hw, oh, oh, k, k, pad, pad, stride, stride, 1, int(d["with_relu"]),
                           int(d["with_sum"]), ol.ptr(conv), ol.ptr(x), ol.ptr(w), ol.ptr(bias))
    d.update(x=x, w=w, bias=bias, sum_operand=sum_operand)
    return _harness_pack(quant, xq, sq, conv)


def harness_oracle(d):
    f32 = np.float32
    n, g, ic, oc, hw, k, pad, stride, oh = (int(d[key]) for key in ("n", "g", "ic", "oc", "hw", "k", "pad", "stride", "oh"))
    with_relu, with_sum = int(d["with_relu"]), int(d["with_sum"])
    out_type = ol.S8 if int(d["out_s8"]) else ol.U8
    x, w, bias, sum_operand = d["x"], d["w"], d["bias"], d["sum_operand"]
    # input_quant: abs-max over 127, zero point 128 for the "...z" configurations (tests/elt_conv_utils.cpp:264-289)
    in_scale = f32(np.abs(x).max()) / f32(HARNESS_REPRESENTATION)
    in_z = f32(128.0 if int(d["zero_point"]) else 0.0)
    xq = ol.quantize_input_u8(x, float(in_scale), float(in_z))
    p = ol.make_params(n, ic, oc, hw, hw, k, k, pad, stride, g=g, with_relu=bool(with_relu), with_sum=bool(with_sum),
                       out_type=out_type)
    conv = ol.ref_conv_f32(p, x, w, bias, out_init=sum_operand if with_sum else None)
    sum_absmax = float(np.abs(sum_operand).max()) if with_sum else 0.0
    s_o, z_o, s_sum = ol.calibrate_output_quant(with_relu, out_type, with_sum, conv.min(), conv.max(), sum_absmax,
                                                HARNESS_REPRESENTATION)
    sq = np.zeros(conv.shape, np.uint8)
    if with_sum:
        # the sum operand is quantized with its own scale and the harness's rounding helper, then narrowed
        # to a byte (tests/elt_conv_utils.cpp:444-462)
        sq = ol.quantize_input_u8(sum_operand, float(f32(sum_absmax) / f32(HARNESS_REPRESENTATION)), 0.0)
    return _harness_pack(np.array([in_scale, in_z, s_o, z_o, s_sum if with_sum else 0.0], f32), xq, sq, conv)


CASES["harness_u8_relu_3x3"] = (lambda: harness_config(0, 0, 2, 1, 20, 24, 9, 3, 1, 1, 1, 0), harness_reference, harness_oracle)
CASES["harness_s8_relu_sum_1x1"] = (lambda: harness_config(1, 0, 2, 1, 32, 16, 7, 1, 0, 1, 1, 1), harness_reference, harness_oracle)
CASES["harness_u8_norelu_3x3_s2"] = (lambda: harness_config(0, 0, 1, 1, 16, 32, 11, 3, 1, 2, 0, 0), harness_reference, harness_oracle)
CASES["harness_s8_norelu_z128_1x1"] = (lambda: harness_config(1, 1, 2, 1, 48, 16, 6, 1, 0, 1, 0, 0), harness_reference, harness_oracle)
CASES["harness_u8_norelu_sum_1x1"] = (lambda: harness_config(0, 0, 1, 1, 16, 16, 8, 1, 0, 1, 0, 1), harness_reference, harness_oracle)
CASES["harness_u8_relu_depthwise"] = (lambda: harness_config(0, 0, 2, 16, 16, 16, 10, 3, 1, 1, 1, 0), harness_reference, harness_oracle)
