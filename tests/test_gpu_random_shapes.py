"""Seeded random shapes for every executor family through the C-ABI against the CPU oracle, bit for
bit: ragged channel counts, odd image sizes, one-sided pads, every output type, both layouts."""
import numpy as np
import pytest

import oracle_lib as ol
from gpu_common import Layer
from test_gpu_parity import run_and_compare

pytestmark = pytest.mark.gpu
OUT_TYPES = [ol.S32, ol.U8, ol.S8, ol.F32]


def _rng(seed):
    return np.random.default_rng(1000 + seed)


@pytest.mark.parametrize("seed", range(24))
def test_random_1x1(seed):
    r = _rng(seed)
    stride = int(r.choice([1, 1, 2]))
    nhwc_in, nhwc_out = bool(r.integers(0, 2)), bool(r.integers(0, 2))
    ic = int(r.integers(1, 20)) * (16 if nhwc_in else int(r.choice([3, 8, 16])))
    oc = int(r.integers(1, 20)) * (16 if nhwc_out else int(r.choice([5, 8, 16])))
    hw = int(r.integers(2, 19))
    if stride == 2:
        hw = max(3, hw | 1)   # (hw - 1) divisible by the stride: the reference has no tail there
    out_type = OUT_TYPES[int(r.integers(0, 4))]
    with_sum = bool(r.integers(0, 2)) and out_type in (ol.U8, ol.S8)
    run_and_compare(Layer(int(r.integers(1, 4)), ic, oc, hw, stride=stride, out_type=out_type, with_sum=with_sum,
                          seed=seed, in_nhwc=nhwc_in, out_nhwc=nhwc_out, with_bias=bool(r.integers(0, 2))))


@pytest.mark.parametrize("seed", range(24))
def test_random_kxk(seed):
    r = _rng(100 + seed)
    k = int(r.choice([3, 3, 3, 5, 7]))
    stride = int(r.choice([1, 2]))
    pad = int(r.choice([k // 2 - 1, k // 2]))
    hw = int(r.integers(k + 1, 26))
    ic = int(r.integers(1, 9)) * int(r.choice([4, 16, 24]))
    oc = int(r.integers(1, 9)) * int(r.choice([6, 16]))
    out_hw = None
    natural = (hw + 2 * pad - k) // stride + 1
    if stride == 2 and pad == k // 2 - 1 and (natural) * stride + k - hw - pad <= k // 2:
        # ask for one more output row / column: pads only at the right / bottom
        if r.integers(0, 2):
            out_hw = natural + 1
    # the right / bottom pad that the output size implies must be k/2 - 1 or k/2 as well: the reference's c160
    # shape set (src/elx_int8_conv_direct.cpp:66-77 with the pads of src/elx_conv.cpp:36-37); a drawn size whose
    # implied pad is another grows until it is one of them, so that no seed ends in a refused layer
    o = out_hw or natural
    while max(0, (o - 1) * stride + k - hw - pad) not in (k // 2 - 1, k // 2):
        hw += 1
        out_hw = None
        o = natural = (hw + 2 * pad - k) // stride + 1
    assert reference_c160_shape_ok(k, stride, pad, hw, o)
    out_type = OUT_TYPES[int(r.integers(0, 4))]
    nhwc_in = ic % 16 == 0 and bool(r.integers(0, 2))
    nhwc_out = oc % 16 == 0 and bool(r.integers(0, 2))
    run_and_compare(Layer(int(r.integers(1, 3)), ic, oc, hw, k=k, pad=pad, stride=stride, out_type=out_type, seed=seed,
                          out_hw=out_hw, in_nhwc=nhwc_in, out_nhwc=nhwc_out))


def reference_c160_shape_ok(k, stride, pad, hw, out_hw):
    """what the reference's direct int8 executor accepts for a square k x k layer (src/elx_int8_conv_direct.cpp:66-77):
    3 / 5 / 7 kernels, stride 1 or 2, left / top pad and the right / bottom pad it recomputes from the output size
    (rp = max(0, ws (ow - 1) + kw - iw - lp), src/elx_conv.cpp:36-37) all k/2 - 1 or k/2"""
    rp = max(0, stride * (out_hw - 1) + k - hw - pad)
    return k in (3, 5, 7) and stride in (1, 2) and pad in (k // 2 - 1, k // 2) and rp in (k // 2 - 1, k // 2)


def test_every_refused_kxk_shape_is_one_the_reference_refuses():
    """ehip_conv_create over seeded k x k shapes, pads and output sizes, fitting and not: wherever it answers
    "c160: shape not supported" the reference's own shape test fails too (the library may accept more: an output
    size that leaves input columns unused, which the reference's clamped pad turns away for 5x5 and 7x7)."""
    from gpu_common import pkg
    E = pkg()
    r = _rng(900)
    refused = accepted = 0
    for _ in range(600):
        k = int(r.choice([3, 5, 7]))
        stride = int(r.choice([1, 2, 3]))
        pad = int(r.integers(0, k // 2 + 2))
        hw = int(r.integers(k + 1, 30))
        natural = (hw + 2 * pad - k) // stride + 1
        out_hw = max(1, natural + int(r.integers(-1, 2)))
        d = E.make_desc(1, 32, 32, hw, hw, k, k, pad, stride, output_type=ol.U8)
        d.oh = d.ow = out_hw
        try:
            E.Conv(d).close()
            accepted += 1
        except E.EulerHipError as exc:
            if "c160: shape not supported" not in str(exc):
                continue
            refused += 1
            assert not reference_c160_shape_ok(k, stride, pad, hw, out_hw), (k, stride, pad, hw, out_hw)
    assert refused > 50 and accepted > 50


@pytest.mark.parametrize("seed", range(24))
def test_random_first_layer(seed):
    """k x k over 1..4 input channels: compact nhwc or blocked input, with and without a zero point"""
    r = _rng(400 + seed)
    k = int(r.choice([3, 5, 7]))
    stride = int(r.choice([1, 2]))
    pad = int(r.choice([k // 2 - 1, k // 2]))
    hw = int(r.integers(k + 1, 40))
    ic = int(r.integers(1, 5))
    oc = int(r.integers(1, 9)) * 16
    out_hw = None
    natural = (hw + 2 * pad - k) // stride + 1
    if stride == 2 and pad == k // 2 - 1 and natural * stride + k - hw - pad <= k // 2 and r.integers(0, 2):
        out_hw = natural + 1   # pads only at the right / bottom
    # the right / bottom pad that the output size implies must be k/2 - 1 or k/2 as well (c160 shapes)
    o = out_hw or natural
    while (o - 1) * stride + k - hw - pad not in (k // 2 - 1, k // 2) and (o - 1) * stride + k - hw - pad >= 0:
        hw += 1
        out_hw = None
        o = natural = (hw + 2 * pad - k) // stride + 1
    in_z = float(r.choice([0.0, 128.0, 3.0]))
    if in_z != 0.0 and (pad or out_hw) and min(natural, out_hw or natural) + (k // 2 - 1) < k:
        in_z = 0.0   # the reference refuses a zero point where one pad cannot be covered
    out_type = OUT_TYPES[int(r.integers(0, 4))]
    res = run_and_compare(Layer(int(r.integers(1, 4)), ic, oc, hw, k=k, pad=pad, stride=stride, out_type=out_type,
                                seed=seed, out_hw=out_hw, in_z=in_z, in_nhwc=bool(r.integers(0, 2)),
                                out_nhwc=bool(r.integers(0, 2)), with_relu=(out_type != ol.F32 or in_z == 0.0)))
    assert res["conv"].kernel_name.startswith("k_conv_fewch")


@pytest.mark.parametrize("seed", range(16))
def test_random_depthwise(seed):
    r = _rng(200 + seed)
    stride = int(r.choice([1, 2]))
    pad = int(r.integers(0, 2))
    hw = int(r.integers(4, 40))
    g = 16 * int(r.integers(1, 8))
    oh = (hw + 2 * pad - 3) // stride + 1
    divs = [t for t in range(1, oh + 1) if oh % t == 0]
    T = int(r.choice(divs + [0, oh]))
    out_type = [ol.U8, ol.S8, ol.S32][int(r.integers(0, 3))]
    in_z = float(r.choice([0.0, 0.0, 3.0, 128.0]))
    run_and_compare(Layer(int(r.integers(1, 4)), g, g, hw, k=3, pad=pad, stride=stride, out_type=out_type, depthwise=True,
                          seed=seed, w_sigma=0.1, T=T, in_z=in_z))


@pytest.mark.parametrize("seed", range(24))
def test_random_winograd(seed):
    import torch
    from gpu_common import bits, dev, host
    from test_gpu_wino import make_wino, make_wino_u8
    r = _rng(300 + seed)
    n, hw = int(r.integers(1, 4)), int(r.integers(4, 23))
    ic, oc = int(r.integers(1, 20)) * int(r.choice([8, 16])), int(r.integers(1, 12)) * int(r.choice([8, 16]))
    u8_in = bool(r.integers(0, 2))
    out_type = [ol.F32, ol.U8, ol.S8][int(r.integers(0, 3))] if u8_in else ol.F32
    bias_on, relu_on = bool(r.integers(0, 2)), bool(r.integers(0, 2))
    tile = int(r.choice([6, 4, 5]))   # F(4x4,3x3), F(2x2,3x3), F(3x3,3x3)
    with_sum = bool(r.integers(0, 3) == 0)
    in_nhwc = bool(r.integers(0, 3) == 0) and ic % 16 == 0
    out_nhwc = bool(r.integers(0, 3) == 0) and oc % 16 == 0
    if u8_in:
        E, p, d, x, wb, bias = make_wino_u8(n, ic, oc, hw, seed, out_type, with_bias=bias_on, with_relu=relu_on, tile=tile)
        xf = x.astype(np.float32)
    else:
        E, p, d, x, wb, bias = make_wino(n, ic, oc, hw, seed, with_bias=bias_on, with_relu=relu_on, tile=tile)
        xf = x
    p.tin_scale, p.tin_z = 22.0 / 255.0, 104.0
    d.tinput_scale, d.tinput_z = p.tin_scale, p.tin_z
    twq, tscale, tshift = ol.wino_prepare(p, wb)
    tout, _ = ol.wino_gemm(p, ol.wino_trans_input(p, xf), twq, tscale, tshift)
    old = None
    if with_sum:
        p.with_sum = d.with_ip_sum = 1
        shape = (n, ol.up16(oc) // 16, hw, hw, 16)
        old = (r.normal(0, 0.05, shape).astype(np.float32) if out_type == ol.F32 else
               r.integers(-30 if out_type == ol.S8 else 0, 60, shape).astype(ol.NP_OF[out_type]))
    exp = ol.wino_trans_output(p, tout, bias, out_init=old)
    if in_nhwc:
        d.input_fmt = E.NHWC
        x = ol.blocked_to_nhwc(x, ic)
    if out_nhwc:
        d.output_fmt = E.NHWC
        exp = ol.blocked_to_nhwc(exp, oc)
        old = ol.blocked_to_nhwc(old, oc) if with_sum else None
    conv = E.Conv(d)
    tdt = {ol.F32: torch.float32, ol.U8: torch.uint8, ol.S8: torch.int8}[out_type]
    d_out = dev(old) if with_sum else torch.full(exp.shape, 3, dtype=tdt, device="cuda")
    d_b = dev(bias) if bias_on else None
    conv.execute(d_out, dev(x), dev(wb), d_b)
    torch.cuda.synchronize()
    got = host(d_out)
    assert got.shape == exp.shape
    assert np.array_equal(bits(got), bits(exp)), "%d of %d values differ" % (int((got != exp).sum()), got.size)
