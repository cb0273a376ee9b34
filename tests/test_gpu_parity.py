"""GPU parity: the HIP path, called through the C-ABI, against the CPU oracle on the same seeded
inputs.  Bars: s32 accumulators, quantized weights and u8/s8 outputs bit-exact; f32 scale/shift and
f32 outputs bit-exact as well (the north-star tolerance is 1 ULP; the tests hold the tighter bar)."""
import numpy as np
import pytest

import oracle_lib as ol
from gpu_common import Layer, bits, dev, host, pkg

pytestmark = pytest.mark.gpu


def check_prepare(res, orc, E):
    conv = res["conv"]
    wq = conv.query(E.Q_WEIGHTS_S8)
    assert np.array_equal(wq, orc["wq"].ravel()), "quantized weights differ"
    assert np.array_equal(conv.query(E.Q_WSUM), orc["wsum"])
    assert np.array_equal(bits(conv.query(E.Q_SCALE)), bits(orc["scale"])), "scale differs"
    assert np.array_equal(bits(conv.query(E.Q_SHIFT)), bits(orc["shift"])), "shift differs"


def run_and_compare(layer, lazy=False):
    E = pkg()
    orc = layer.oracle()
    res = layer.run_gpu(lazy_prepare=lazy)
    check_prepare(res, orc, E)
    got, exp = res["out"], orc["out"]
    assert got.shape == exp.shape
    if not np.array_equal(bits(got), bits(exp)):
        bad = np.argwhere(got != exp)
        raise AssertionError("output differs at %d of %d positions, first %s: got %s expected %s (kernel %s)" % (
            len(bad), got.size, bad[0], got[tuple(bad[0])], exp[tuple(bad[0])], res["conv"].kernel_name))
    return res


# ---- 1x1 (CONV_DIRECT_1X1 a160; f32 output goes through CONV_DIRECT a160) ----------------------
@pytest.mark.parametrize("out_type", [ol.S32, ol.U8, ol.S8, ol.F32])
@pytest.mark.parametrize("n,ic,oc,hw", [(2, 64, 64, 9), (1, 80, 48, 7), (3, 128, 272, 5)])
def test_conv1x1_s1(out_type, n, ic, oc, hw):
    run_and_compare(Layer(n, ic, oc, hw, out_type=out_type, seed=11 + ic + out_type))


@pytest.mark.parametrize("out_type", [ol.U8, ol.S8])
def test_conv1x1_sum_relu(out_type):
    run_and_compare(Layer(2, 96, 64, 14, out_type=out_type, with_sum=True, seed=5))


@pytest.mark.parametrize("out_type", [ol.U8, ol.S8])
@pytest.mark.parametrize("with_sum", [False, True])
def test_conv1x1_every_zero_point(out_type, with_sum):
    """input, output and sum zero points all non-zero: the folded shift (compared bit for bit with the
    oracle's, whose contraction pattern is that of the reference's compiled fold) and the result"""
    run_and_compare(Layer(2, 96, 256, 9, out_type=out_type, with_sum=with_sum, seed=15 + out_type, in_z=113.0, out_z=3.0,
                          sum_z=-97.0))


def test_conv3x3_and_depthwise_output_zero_point():
    run_and_compare(Layer(2, 32, 64, 9, k=3, pad=0, out_type=ol.S8, seed=16, in_z=113.0, out_z=-2.0))
    run_and_compare(Layer(2, 64, 64, 9, k=3, pad=1, out_type=ol.U8, depthwise=True, T=3, w_sigma=0.1, seed=17, in_z=37.0,
                          out_z=2.0))


@pytest.mark.parametrize("out_type", [ol.S32, ol.S8])
def test_conv1x1_stride2(out_type):
    run_and_compare(Layer(2, 64, 96, 14, stride=2, out_type=out_type, with_sum=(out_type == ol.S8), seed=6))


@pytest.mark.parametrize("variant", [1, 2, 3, 4])
@pytest.mark.parametrize("n,ic,oc,hw,stride", [(2, 256, 256, 14, 1), (3, 144, 80, 9, 1), (1, 512, 272, 14, 2), (2, 1024, 128, 7, 1),
                                               (1, 272, 48, 5, 1)])
def test_conv1x1_resident_pixel_tile_kernel(variant, n, ic, oc, hw, stride, monkeypatch):
    """the 1x1 kernel for many input channels (pixel tile resident in LDS, weights streamed): every tile shape;
    K loop unrolled (8, 16, 32 k-steps) and as a loop; ragged channel and pixel counts; stride 2; with the sum"""
    monkeypatch.setenv("EHIP_GEMM1X1_RES", str(variant))
    for out_type, with_sum in ((ol.U8, False), (ol.S8, True), (ol.F32, False), (ol.S32, False)):
        res = run_and_compare(Layer(n, ic, oc, hw, stride=stride, out_type=out_type, with_sum=with_sum,
                                    seed=300 + variant + ic + out_type))
    monkeypatch.setenv("EHIP_GEMM1X1_UNROLL", "0")
    run_and_compare(Layer(n, ic, oc, hw, stride=stride, out_type=ol.U8, seed=301 + variant + ic, relu_hi=200.0))


@pytest.mark.parametrize("variant", ["", "1", "2", "3", "4"])
@pytest.mark.parametrize("n,ic,oc,hw,stride", [(2, 256, 272, 14, 1), (3, 144, 80, 9, 1), (1, 512, 176, 14, 2), (2, 1024, 256, 7, 1)])
def test_conv1x1_resident_pixel_tile_kernel_nhwc_output(variant, n, ic, oc, hw, stride, monkeypatch):
    """blocked input, nhwc output, u8 / s8 with ReLU (the lean epilogue's cases): a lane's 16 channels are 16
    contiguous bytes of its pixel's vector; with the sum the old output is read from the same place"""
    if variant:
        monkeypatch.setenv("EHIP_GEMM1X1_RES", variant)
    for out_type, with_sum, kw in ((ol.U8, False, {}), (ol.S8, True, {}), (ol.U8, True, {"relu_hi": 200.0})):
        res = run_and_compare(Layer(n, ic, oc, hw, stride=stride, out_type=out_type, with_sum=with_sum, out_nhwc=True,
                                    seed=330 + ic + out_type, **kw))
        if variant:
            assert res["conv"].kernel_name.startswith("k_gemm1x1_res")
    # what the lean epilogue does not cover goes through the general kernel
    res = run_and_compare(Layer(n, ic, oc, hw, stride=stride, out_type=ol.F32, out_nhwc=True, seed=331 + ic))
    assert res["conv"].kernel_name.startswith("k_gemm_u8s8")
    # and so does everything when the lean epilogue is switched off: the switch must reach the choice of kernel, not
    # only the launcher (this kernel's general epilogue writes blocked output only)
    monkeypatch.setenv("EHIP_LEAN_EPILOGUE", "0")
    res = run_and_compare(Layer(n, ic, oc, hw, stride=stride, out_type=ol.S8, with_sum=True, out_nhwc=True, seed=332 + ic))
    assert res["conv"].kernel_name.startswith("k_gemm_u8s8")


@pytest.mark.parametrize("variant", ["", "2", "4"])
@pytest.mark.parametrize("n,ic,oc,hw,stride", [(2, 256, 272, 14, 1), (3, 144, 80, 9, 1), (1, 512, 176, 14, 2), (2, 1024, 256, 7, 1),
                                               (1, 2048, 64, 5, 1)])
def test_conv1x1_resident_pixel_tile_kernel_nhwc_input(variant, n, ic, oc, hw, stride, monkeypatch):
    """nhwc input: the tile pixel-major in LDS (one pad cell per pixel); blocked output with every output
    type, nhwc output with the lean epilogue's cases; generic and unrolled K loops, stride 2, ragged tiles"""
    if variant:
        monkeypatch.setenv("EHIP_GEMM1X1_RES", variant)
    for out_type, with_sum in ((ol.U8, False), (ol.S8, True), (ol.F32, False), (ol.S32, False)):
        res = run_and_compare(Layer(n, ic, oc, hw, stride=stride, out_type=out_type, with_sum=with_sum, in_nhwc=True,
                                    seed=350 + ic + out_type))
        if variant:
            assert res["conv"].kernel_name.startswith("k_gemm1x1_res")
    for out_type, with_sum in ((ol.U8, True), (ol.S8, False)):
        res = run_and_compare(Layer(n, ic, oc, hw, stride=stride, out_type=out_type, with_sum=with_sum, in_nhwc=True,
                                    out_nhwc=True, seed=351 + ic + out_type))
        if variant:
            assert res["conv"].kernel_name.startswith("k_gemm1x1_res")
    monkeypatch.setenv("EHIP_GEMM1X1_UNROLL", "0")
    run_and_compare(Layer(n, ic, oc, hw, stride=stride, out_type=ol.U8, seed=352 + ic, in_nhwc=True))


@pytest.mark.parametrize("slots", ["", "8", "40"])
@pytest.mark.parametrize("n,ic,oc,hw,stride", [(2, 256, 256, 14, 1), (3, 256, 80, 9, 1), (1, 512, 272, 14, 2), (2, 1024, 128, 7, 1),
                                               (1, 512, 48, 5, 1), (3, 1024, 336, 9, 1), (5, 512, 128, 14, 1),
                                               (3, 128, 272, 11, 1), (2, 128, 512, 14, 2)])
def test_conv1x1_weights_resident_kernel(slots, n, ic, oc, hw, stride, monkeypatch):
    """the 1x1 kernel with the weights in registers and the pixels streamed through a ring of LDS stages: 128 / 256 / 512 /
    1024 input channels, ragged channel and pixel counts, stride 2, u8 / s8 with and without the sum, other ReLU
    bounds, blocked and nhwc output; few workgroup slots make the runs longer than the ring, so stages are reused"""
    monkeypatch.setenv("EHIP_GEMM1X1_WRES", "1")
    if slots:
        monkeypatch.setenv("EHIP_WRES_SLOTS", slots)
    for out_type, with_sum, kw in ((ol.U8, False, {}), (ol.S8, True, {}), (ol.U8, True, {"relu_hi": 200.0}), (ol.S8, False, {}),
                                   (ol.S8, True, {"out_nhwc": True}), (ol.U8, False, {"out_nhwc": True})):
        res = run_and_compare(Layer(n, ic, oc, hw, stride=stride, out_type=out_type, with_sum=with_sum,
                                    seed=700 + ic + oc + out_type, **kw))
        assert res["conv"].kernel_name == "k_gemm1x1_wres"
    # what the lean epilogue does not cover stays with the other kernels
    res = run_and_compare(Layer(n, ic, oc, hw, stride=stride, out_type=ol.F32, seed=701 + ic))
    assert res["conv"].kernel_name != "k_gemm1x1_wres"


@pytest.mark.parametrize("nbuf", ["3", "4"])
def test_conv1x1_weights_resident_kernel_ring_depths(nbuf, monkeypatch):
    monkeypatch.setenv("EHIP_GEMM1X1_WRES", "1")
    monkeypatch.setenv("EHIP_WRES_SLOTS", "16")
    monkeypatch.setenv("EHIP_WRES_NBUF", nbuf)
    for ic, with_sum in ((128, True), (256, True), (512, False), (1024, True)):
        res = run_and_compare(Layer(4, ic, 256, 14, out_type=ol.S8, with_sum=with_sum, seed=710 + ic))
        assert res["conv"].kernel_name == "k_gemm1x1_wres"


def test_conv1x1_weights_resident_kernel_can_be_switched_off(monkeypatch):
    # (256 -> 1024 at 14 x 14, N = 64: runs of three tiles per workgroup, the launcher's own choice)
    monkeypatch.setenv("EHIP_GEMM1X1_WRES", "0")
    res = run_and_compare(Layer(64, 256, 1024, 14, out_type=ol.S8, with_sum=True, seed=720))
    assert res["conv"].kernel_name != "k_gemm1x1_wres"
    monkeypatch.delenv("EHIP_GEMM1X1_WRES")
    res = run_and_compare(Layer(64, 256, 1024, 14, out_type=ol.S8, with_sum=True, seed=720))
    assert res["conv"].kernel_name == "k_gemm1x1_wres"


def test_conv1x1_resident_pixel_tile_kernel_can_be_switched_off(monkeypatch):
    monkeypatch.setenv("EHIP_GEMM1X1_RES", "0")
    run_and_compare(Layer(2, 256, 256, 14, out_type=ol.S8, with_sum=True, seed=302))


def test_conv1x1_lazy_first_run_and_no_bias():
    run_and_compare(Layer(1, 64, 32, 6, out_type=ol.U8, with_bias=False, seed=8), lazy=True)


@pytest.mark.parametrize("variant", range(7))
def test_conv1x1_every_kernel_variant(variant, monkeypatch):
    monkeypatch.setenv("EHIP_GEMM_VARIANT", str(variant))
    monkeypatch.setenv("EHIP_GEMM1X1_RES", "0")   # the general kernel, not the one with the resident pixel tile
    res = run_and_compare(Layer(2, 144, 80, 11, out_type=ol.S8, with_sum=True, seed=40 + variant))
    assert res["conv"].kernel_name.startswith("k_gemm_u8s8")


# layers with at most 128 input channels take the weights-in-registers kernel
@pytest.mark.parametrize("out_type", [ol.S32, ol.U8, ol.S8, ol.F32])
@pytest.mark.parametrize("n,ic,oc,hw,stride,nhwc", [(2, 64, 256, 9, 1, False), (3, 32, 64, 7, 1, False), (1, 128, 512, 6, 1, True),
                                                    (2, 16, 16, 5, 1, False), (2, 96, 48, 9, 2, False), (1, 8, 40, 33, 1, False),
                                                    (2, 128, 144, 8, 2, True)])
def test_conv1x1_few_input_channels(out_type, n, ic, oc, hw, stride, nhwc):
    if nhwc and oc % 16:
        pytest.skip("nhwc needs whole channel blocks")
    res = run_and_compare(Layer(n, ic, oc, hw, stride=stride, out_type=out_type, seed=170 + ic + oc,
                                with_sum=out_type in (ol.U8, ol.S8), in_nhwc=nhwc, out_nhwc=nhwc))
    assert res["conv"].kernel_name.startswith("k_gemm_smallk")


@pytest.mark.parametrize("out_type,with_sum", [(ol.U8, False), (ol.S8, True), (ol.S8, False)])
@pytest.mark.parametrize("n,ic,oc,hw,stride", [(2, 32, 256, 12, 1), (1, 32, 128, 17, 1), (2, 64, 128, 11, 1), (2, 64, 256, 14, 1),
                                               (1, 128, 144, 13, 1), (3, 128, 64, 9, 1), (2, 64, 80, 10, 1), (2, 128, 512, 12, 2),
                                               (1, 48, 272, 15, 1)])
def test_conv1x1_few_input_channels_several_channel_tiles_per_wave(out_type, with_sum, n, ic, oc, hw, stride):
    """u8 / s8 blocked output with ReLU: a wave keeps the weights of 2 or 4 tiles of 32 output channels and
    reads every pixel tile once; channel counts that leave the last wave group partly or wholly past the real
    channels included"""
    res = run_and_compare(Layer(n, ic, oc, hw, stride=stride, out_type=out_type, seed=510 + ic + oc, with_sum=with_sum))
    assert res["conv"].kernel_name.startswith("k_gemm_smallk_lean")


def test_conv1x1_few_input_channels_can_be_switched_off(monkeypatch):
    monkeypatch.setenv("EHIP_GEMM_SMALLK", "0")
    res = run_and_compare(Layer(2, 64, 96, 9, out_type=ol.U8, seed=177))
    assert res["conv"].kernel_name.startswith("k_gemm_u8s8")


# nhwc activations on either side (src/elx_int8_conv_direct_1x1.cpp:374-396,417-468); the expected
# values are the oracle's, moved through the closed-form index map [n][c/16][h][w][16] -> [n][h][w][c]
@pytest.mark.parametrize("in_nhwc,out_nhwc", [(True, True), (True, False), (False, True)])
@pytest.mark.parametrize("out_type", [ol.S32, ol.U8, ol.S8, ol.F32])
def test_conv1x1_nhwc(in_nhwc, out_nhwc, out_type):
    run_and_compare(Layer(3, 128, 272 if not out_nhwc else 176, 5, out_type=out_type, seed=70 + out_type,
                          in_nhwc=in_nhwc, out_nhwc=out_nhwc))


@pytest.mark.parametrize("stride", [1, 2])
def test_conv1x1_nhwc_sum_relu(stride):
    run_and_compare(Layer(2, 96, 64, 14, stride=stride, out_type=ol.S8, with_sum=True, seed=75, in_nhwc=True, out_nhwc=True))


@pytest.mark.parametrize("variant", range(7))
def test_conv1x1_nhwc_every_kernel_variant(variant, monkeypatch):
    monkeypatch.setenv("EHIP_GEMM_VARIANT", str(variant))
    run_and_compare(Layer(2, 144, 80, 11, out_type=ol.U8, with_sum=True, seed=80 + variant, in_nhwc=True, out_nhwc=True))


def test_nhwc_is_refused_where_it_is_not_built():
    E = pkg()
    d = E.make_desc(1, 40, 64, 8, 8, algorithm=E.CONV_DIRECT_1X1)
    d.input_fmt = E.NHWC   # channel tail
    with pytest.raises(E.EulerHipError):
        E.Conv(d)
    d = E.make_desc(1, 64, 64, 8, 8, 3, 3, 1, g=64, algorithm=E.CONV_DIRECT)
    d.input_fmt = E.NHWC   # nhwc input of a depthwise layer
    with pytest.raises(E.EulerHipError):
        E.Conv(d)


@pytest.mark.parametrize("k,pad,stride", [(3, 1, 1), (3, 1, 2), (7, 3, 2)])
def test_direct_kxk_nhwc_output(k, pad, stride):
    res = run_and_compare(Layer(2, 32, 48, 13, k=k, pad=pad, stride=stride, out_type=ol.S8, seed=160 + k + stride, out_nhwc=True))
    assert res["conv"].kernel_name.startswith("k_gemm_u8s8")


# nhwc INPUT of a k x k layer (src/elx_int8_conv_direct.cpp:596-668, input_as_bfmt_ false): the tap offset
# is a whole channel vector per pixel, every thread keeps the valid-tap mask of each pixel it stages
@pytest.mark.parametrize("in_z", [0.0, 128.0])
@pytest.mark.parametrize("out_nhwc", [False, True])
@pytest.mark.parametrize("n,ic,oc,hw,k,pad,stride", [(2, 32, 48, 13, 3, 1, 1), (1, 64, 64, 14, 3, 1, 2), (2, 16, 32, 17, 7, 3, 2),
                                                     (1, 144, 32, 9, 5, 2, 1), (2, 48, 80, 12, 3, 0, 1)])
def test_direct_kxk_nhwc_input(in_z, out_nhwc, n, ic, oc, hw, k, pad, stride):
    res = run_and_compare(Layer(n, ic, oc, hw, k=k, pad=pad, stride=stride, out_type=ol.U8, seed=260 + k + stride + ic,
                                in_nhwc=True, out_nhwc=out_nhwc, in_z=in_z))
    assert res["conv"].kernel_name.startswith("k_gemm_u8s8")


@pytest.mark.parametrize("variant", range(7))
def test_direct_kxk_nhwc_input_every_kernel_variant(variant, monkeypatch):
    monkeypatch.setenv("EHIP_GEMM_VARIANT", str(variant))
    run_and_compare(Layer(2, 80, 96, 13, k=3, pad=1, stride=2, out_type=ol.S8, seed=270 + variant, in_nhwc=True))


# ---- 3x3 direct (c160) ------------------------------------------------------------------------------
@pytest.mark.parametrize("out_type", [ol.S32, ol.U8, ol.S8, ol.F32])
@pytest.mark.parametrize("n,ic,oc,hw", [(2, 32, 32, 14), (1, 128, 128, 28), (2, 48, 80, 10), (1, 64, 16, 7)])
def test_conv3x3(out_type, n, ic, oc, hw):
    run_and_compare(Layer(n, ic, oc, hw, k=3, pad=1, out_type=out_type, seed=21 + hw + out_type))


def test_conv3x3_no_padding():
    run_and_compare(Layer(2, 32, 32, 12, k=3, pad=0, out_type=ol.U8, seed=3))


@pytest.mark.parametrize("variant", range(20))
@pytest.mark.parametrize("ic", [64, 96, 128, 256])
def test_conv3x3_every_virtual_row_kernel_variant(variant, ic, monkeypatch):
    """every tile shape, with the K loop as a loop (96 channels: 3 unit pairs) and as straight-line code
    (2, 4, 8 pairs); variants 15 and up deal a wave's pixels to its lanes with a stride"""
    monkeypatch.setenv("EHIP_CONV3X3V_VARIANT", str(variant))
    res = run_and_compare(Layer(2, ic, 144, 13, k=3, pad=1, out_type=ol.U8, seed=80 + variant + ic))
    assert res["conv"].kernel_name.startswith("k_conv3x3v_u8s8")


@pytest.mark.parametrize("split", ["0", "1"])
@pytest.mark.parametrize("variant", [9, 13])
@pytest.mark.parametrize("out_type,relu_hi", [(ol.U8, None), (ol.U8, 200.0), (ol.S8, None)])
@pytest.mark.parametrize("n,ic,oc,hw", [(2, 64, 144, 13), (3, 128, 128, 28), (1, 256, 80, 14)])
def test_conv3x3_split_last_pair(split, variant, out_type, relu_hi, n, ic, oc, hw, monkeypatch):
    """u8 / s8 output with ReLU: the last channel pair multiplied tile pair by tile pair with half of the
    epilogue behind its MFMAs (2, 4, 8 unit pairs; with and without a clamp), and the same layers in tap order"""
    monkeypatch.setenv("EHIP_CONV3X3V_VARIANT", str(variant))
    monkeypatch.setenv("EHIP_CONV3X3V_SPLIT_LAST", split)
    kw = {} if relu_hi is None else {"relu_hi": relu_hi}
    res = run_and_compare(Layer(n, ic, oc, hw, k=3, pad=1, out_type=out_type, seed=640 + ic + out_type, **kw))
    assert res["conv"].kernel_name.startswith("k_conv3x3v_u8s8")


@pytest.mark.parametrize("variant", [15, 16, 17, 18, 19])
@pytest.mark.parametrize("out_type", [ol.S32, ol.S8, ol.F32])
def test_conv3x3_strided_pixels_output_types(variant, out_type, monkeypatch):
    monkeypatch.setenv("EHIP_CONV3X3V_VARIANT", str(variant))
    run_and_compare(Layer(3, 128, 80, 28, k=3, pad=1, out_type=out_type, seed=60 + variant + out_type))
    monkeypatch.setenv("EHIP_CONV3X3V_UNROLL", "0")
    run_and_compare(Layer(1, 128, 80, 9, k=3, pad=0, out_type=out_type, seed=61 + variant + out_type))


def test_conv3x3_virtual_rows_many_channels_restage():
    # 1040 input channels = 65 units: more than one LDS fill of the virtual-row kernel, odd unit count
    res = run_and_compare(Layer(1, 1040, 48, 9, k=3, pad=1, out_type=ol.S8, seed=91, w_sigma=0.02))
    assert res["conv"].kernel_name.startswith("k_conv3x3v_u8s8")


@pytest.mark.parametrize("unroll", ["0", "1"])
@pytest.mark.parametrize("variant,ic", [(9, 512), (9, 768), (13, 256), (10, 1024), (12, 192), (2, 512)])
def test_conv3x3_several_fills_of_whole_pairs(variant, ic, unroll, monkeypatch):
    """more input channels than one LDS fill holds, in whole fills of 2, 4 or 8 unit pairs (512 channels in the
    128 x 128 tile: two fills of eight pairs; 768: three): whichever form of the K loop the launcher picks for them,
    and the loop form forced"""
    monkeypatch.setenv("EHIP_CONV3X3V_VARIANT", str(variant))
    monkeypatch.setenv("EHIP_CONV3X3V_UNROLL", unroll)
    res = run_and_compare(Layer(2, ic, 144, 13, k=3, pad=1, out_type=ol.S8, seed=95 + variant + ic, w_sigma=0.02))
    assert res["conv"].kernel_name.startswith("k_conv3x3v_u8s8")


def test_conv3x3_wide_rows():
    run_and_compare(Layer(1, 16, 32, 70, k=3, pad=1, out_type=ol.U8, seed=92))


# ---- k x k direct as a GEMM over [tap][unit]: stride 2, 5x5 / 7x7, one-sided pads (c160 shapes,
# src/elx_int8_conv_direct.cpp:66-77) ----------------------------------------------------------------
@pytest.mark.parametrize("out_type", [ol.S32, ol.U8, ol.S8, ol.F32])
@pytest.mark.parametrize("n,ic,oc,hw,k,pad,stride,out_hw", [
    (2, 32, 32, 15, 3, 0, 2, None),     # pre-padded input, as the tuned ResNet-v1.5 run feeds it
    (2, 64, 48, 14, 3, 1, 2, None),     # pad 1 on every side
    (1, 48, 80, 14, 3, 0, 2, 7),        # pads only right / bottom (output size fixes them)
    (1, 32, 32, 12, 5, 2, 1, None),
    (1, 16, 32, 17, 7, 3, 2, None),
    (2, 128, 64, 9, 5, 1, 2, None),
])
def test_direct_kxk_strided(out_type, n, ic, oc, hw, k, pad, stride, out_hw):
    res = run_and_compare(Layer(n, ic, oc, hw, k=k, pad=pad, stride=stride, out_type=out_type, seed=90 + k + stride,
                                out_hw=out_hw))
    # 3x3 stride 2 has a form of the 3x3 kernel (four phase planes of the input); the rest walks [tap][unit] in the GEMM
    assert res["conv"].kernel_name.startswith("k_conv3x3v_u8s8" if (k, stride) == (3, 2) else "k_gemm_u8s8")


@pytest.mark.parametrize("variant", ["", "20", "21", "22", "23"])
@pytest.mark.parametrize("n,ic,oc,hw,pad,out_hw", [
    (2, 128, 128, 30, 0, None),    # pre-padded input, 128 channels: the straight-line K loop of four unit pairs
    (3, 64, 80, 15, 1, None),      # two unit pairs, ragged channels, odd size
    (2, 256, 64, 14, 1, None),     # two fills
    (1, 48, 272, 14, 0, 7),        # pads only right / bottom, three units
    (2, 32, 32, 57, 1, None),      # output rows of 29 pixels: the widest the 128-pixel tiles take
    (1, 16, 16, 8, 1, None),
])
def test_direct_3x3_stride2_phase_planes(variant, n, ic, oc, hw, pad, out_hw, monkeypatch):
    """3x3 stride 2 through the 3x3 kernel: the staged input as four phase planes, every tile variant, every output type"""
    if variant:
        monkeypatch.setenv("EHIP_CONV3X3V_VARIANT", variant)
    for out_type in (ol.U8, ol.S8, ol.F32, ol.S32):
        res = run_and_compare(Layer(n, ic, oc, hw, k=3, pad=pad, stride=2, out_type=out_type, seed=95 + ic + hw + out_type,
                                    out_hw=out_hw))
        assert "s2" in res["conv"].kernel_name


def test_direct_3x3_stride2_phase_planes_can_be_switched_off(monkeypatch):
    monkeypatch.setenv("EHIP_CONV3X3V_S2", "0")
    res = run_and_compare(Layer(2, 64, 48, 14, k=3, pad=1, stride=2, out_type=ol.S8, seed=97))
    assert res["conv"].kernel_name.startswith("k_gemm_u8s8")


# non-zero input zero point with padding (the "U8...z" data-type configurations of the reference's
# first layers, src/elx_int8_conv_direct.cpp:227-423): one shift per class of border pixels
@pytest.mark.parametrize("out_type", [ol.U8, ol.S8, ol.F32])
@pytest.mark.parametrize("n,ic,oc,hw,k,pad,stride,out_hw", [
    (2, 3, 64, 30, 7, 3, 2, None),      # ResNet-50 conv1 shape family: 7x7 s2 p3, three input channels
    (2, 3, 32, 16, 3, 0, 2, 8),         # MobileNet Conv__224 family: 3x3 s2, pads only right / bottom
    (1, 32, 48, 9, 3, 1, 1, None),      # 3x3 s1 p1 takes the GEMM form when a zero point meets padding
    (1, 24, 16, 11, 5, 2, 2, None),
    (2, 16, 16, 8, 3, 0, 1, None),      # no padding: one class, plain shift
])
def test_direct_zero_point_with_padding(out_type, n, ic, oc, hw, k, pad, stride, out_hw):
    res = run_and_compare(Layer(n, ic, oc, hw, k=k, pad=pad, stride=stride, out_type=out_type, seed=140 + k + stride,
                                out_hw=out_hw, in_z=128.0, with_relu=(out_type != ol.F32)))
    if pad or out_hw:
        assert res["conv"].kernel_name.startswith("k_conv_fewch" if ic <= 4 else "k_gemm_u8s8")


# at most four input channels (first layers; the reference feeds them 3-channel nhwc,
# scripts/best_configs/resnetv1_5-n64-clx-1s-int8.sh:12): 16 / ic pixels per operand cell, a kernel row
# is ceil(kw / (16 / ic)) cells, input rows staged compactly in LDS
FEWCH_SHAPES = [
    (2, 3, 64, 38, 7, 3, 2, None),      # 7x7: two cells of five pixels per kernel row; rows of 114 bytes
    (2, 3, 32, 24, 3, 0, 2, 12),        # 3x3 s2, pads only right / bottom: one cell per kernel row
    (1, 4, 16, 13, 5, 2, 1, None),      # four channels: four pixels per cell, two cells per row
    (2, 1, 32, 17, 3, 1, 1, None),      # one channel: sixteen pixels per cell, rows of 17 bytes
    (1, 2, 48, 21, 7, 2, 2, None),      # pads k/2 - 1
    (3, 3, 16, 9, 3, 1, 2, None),       # rows of 27 bytes: every image and row starts at another byte phase
    (2, 3, 96, 15, 5, 2, 1, None),      # three 32-channel tiles
    (1, 3, 128, 11, 3, 1, 1, None),     # four channel tiles: one per wave
]


@pytest.mark.parametrize("in_nhwc", [False, True])
@pytest.mark.parametrize("in_z", [0.0, 128.0])
@pytest.mark.parametrize("n,ic,oc,hw,k,pad,stride,out_hw", FEWCH_SHAPES)
def test_direct_few_input_channels(in_z, in_nhwc, n, ic, oc, hw, k, pad, stride, out_hw, monkeypatch):
    layer = dict(k=k, pad=pad, stride=stride, out_type=ol.U8, seed=170 + k + ic, out_hw=out_hw, in_z=in_z)
    res = run_and_compare(Layer(n, ic, oc, hw, in_nhwc=in_nhwc, **layer))
    assert res["conv"].kernel_name.startswith("k_conv_fewch")
    if not in_nhwc:
        monkeypatch.setenv("EHIP_FEWCH", "0")     # the general kernels give the same bytes
        res2 = run_and_compare(Layer(n, ic, oc, hw, **layer))
        assert not res2["conv"].kernel_name.startswith("k_conv_fewch")


@pytest.mark.parametrize("out_type,out_nhwc", [(ol.S32, False), (ol.F32, False), (ol.S8, False), (ol.S8, True),
                                               (ol.F32, True), (ol.U8, True)])
def test_direct_few_input_channels_output_types(out_type, out_nhwc):
    run_and_compare(Layer(2, 3, 64, 19, k=7, pad=3, stride=2, out_type=out_type, seed=181 + out_type, in_z=128.0,
                          in_nhwc=True, out_nhwc=out_nhwc, with_relu=(out_type != ol.F32)))
    run_and_compare(Layer(1, 3, 32, 12, k=3, pad=1, stride=1, out_type=out_type, seed=183 + out_type,
                          in_nhwc=False, out_nhwc=out_nhwc))


@pytest.mark.parametrize("pad_pixel", ["0", "1"])
@pytest.mark.parametrize("in_nhwc", [False, True])
def test_direct_three_channels_padded_to_four_or_not(pad_pixel, in_nhwc, monkeypatch):
    # three channels take four bytes per pixel in the staged rows and the cells (every cell starts on a dword;
    # the default wherever it costs no extra cell per kernel row), or three: the same bytes either way
    monkeypatch.setenv("EHIP_FEWCH_PAD_PIXEL", pad_pixel)
    for n, hw, k, pad, stride, oc, in_z in [(3, 37, 7, 3, 2, 64, 128.0), (2, 23, 3, 1, 2, 32, 128.0), (3, 9, 3, 1, 1, 16, 0.0),
                                            (1, 29, 7, 2, 2, 32, 0.0), (2, 16, 5, 2, 1, 16, 0.0)]:
        res = run_and_compare(Layer(n, 3, oc, hw, k=k, pad=pad, stride=stride, out_type=ol.U8, seed=197 + k + hw,
                                    in_z=in_z, in_nhwc=in_nhwc))
        assert res["conv"].kernel_name.startswith("k_conv_fewch")


@pytest.mark.parametrize("lean_kernel", ["0", "1"])
@pytest.mark.parametrize("out_type,out_nhwc,with_relu", [(ol.U8, False, True), (ol.S8, True, True), (ol.U8, True, True),
                                                         (ol.S8, False, True), (ol.S8, False, False)])
def test_direct_few_input_channels_lean_kernel(lean_kernel, out_type, out_nhwc, with_relu, monkeypatch):
    # u8 / s8 output with ReLU has a kernel of its own (straight-line tile loop, the next tile's cells read during
    # the epilogue); EHIP_FEWCH_LEAN_KERNEL=0 sends those layers through the general one: the same bytes.  With and
    # without border classes (input zero point), every number of cells per tile, channel tiles over several waves.
    monkeypatch.setenv("EHIP_FEWCH_LEAN_KERNEL", lean_kernel)
    want = "k_conv_fewch_lean" if (lean_kernel == "1" and with_relu) else "k_conv_fewch_u8s8"
    for n, ic, oc, hw, k, pad, stride, in_z, in_nhwc in [(2, 3, 64, 37, 7, 3, 2, 128.0, True), (2, 3, 32, 23, 3, 1, 2, 128.0, True),
                                                         (1, 4, 16, 13, 5, 2, 1, 0.0, False), (2, 1, 96, 17, 3, 1, 1, 3.0, True),
                                                         (1, 2, 128, 21, 7, 3, 2, 0.0, True), (3, 3, 16, 9, 5, 2, 1, 128.0, False)]:
        res = run_and_compare(Layer(n, ic, oc, hw, k=k, pad=pad, stride=stride, out_type=out_type, seed=230 + k + ic,
                                    in_z=in_z, in_nhwc=in_nhwc, out_nhwc=out_nhwc, with_relu=with_relu))
        assert res["conv"].kernel_name == want


@pytest.mark.parametrize("rows", [1, 2, 3, 5, 16])
def test_direct_few_input_channels_strip_heights(rows, monkeypatch):
    # output rows per workgroup, including strips that end below the image
    monkeypatch.setenv("EHIP_FEWCH_ROWS", str(rows))
    run_and_compare(Layer(2, 3, 64, 27, k=7, pad=3, stride=2, out_type=ol.S8, seed=190 + rows, in_z=128.0, in_nhwc=True))
    run_and_compare(Layer(2, 3, 32, 13, k=3, pad=1, stride=1, out_type=ol.U8, seed=195 + rows, in_nhwc=True))


def test_direct_few_input_channels_rows_too_wide_for_lds():
    """7 staged rows of a 3000-pixel image do not fit the first-layer kernel's LDS: blocked input takes the
    general k x k form, compact nhwc input is refused (nothing else reads that layout)."""
    E = pkg()
    d = E.make_desc(1, 3, 16, 8, 3000, 7, 7, 3, algorithm=E.CONV_DIRECT, output_type=E.U8, output_quant=(0.05, 0.0),
                    input_quant=(1.0 / 255.0, 128.0))
    conv = E.Conv(d)
    assert conv.kernel_name.startswith("k_gemm_u8s8")
    d.input_fmt = E.NHWC
    with pytest.raises(E.EulerHipError):
        E.Conv(d)


@pytest.mark.parametrize("variant", range(7))
def test_direct_3x3_stride2_every_kernel_variant(variant, monkeypatch):
    monkeypatch.setenv("EHIP_GEMM_VARIANT", str(variant))
    monkeypatch.setenv("EHIP_CONV3X3V_S2", "0")   # the GEMM form
    run_and_compare(Layer(2, 80, 96, 13, k=3, pad=1, stride=2, out_type=ol.U8, seed=120 + variant))


def test_direct_3x3_very_wide_rows():
    run_and_compare(Layer(1, 16, 16, 240, k=3, pad=1, out_type=ol.U8, seed=130))


# ---- depthwise 3x3 ----------------------------------------------------------------------------------
@pytest.mark.parametrize("out_type", [ol.U8, ol.S8])
@pytest.mark.parametrize("g,hw,T", [(32, 14, 7), (144, 56, 14), (64, 7, 7), (16, 28, 11), (32, 9, 4), (32, 5, 0)])
def test_depthwise(out_type, g, hw, T):
    n = 2 if hw < 56 else 1
    run_and_compare(Layer(n, g, g, hw, k=3, pad=1, out_type=out_type, depthwise=True, seed=g + hw + T, w_sigma=0.1,
                          T=T))


@pytest.mark.parametrize("relu_hi,with_relu", [(200.0, True), (ol.FLT_MAX, True), (255.0, False)])
def test_depthwise_u8_other_bounds(relu_hi, with_relu):
    # bounds other than [0, 255] leave the one-instruction narrowing and take the general epilogue
    run_and_compare(Layer(2, 48, 48, 14, k=3, pad=1, out_type=ol.U8, depthwise=True, seed=17, w_sigma=0.1, T=7,
                          relu_hi=relu_hi, with_relu=with_relu))


@pytest.mark.parametrize("g,hw,pad,T,relu_hi,in_z", [
    (32, 28, 1, 14, 255.0, 0.0), (144, 56, 1, 14, 255.0, 0.0), (16, 70, 1, 7, 255.0, 0.0), (16, 112, 1, 28, 255.0, 0.0),
    (32, 30, 1, 11, 255.0, 0.0), (48, 9, 1, 4, 255.0, 0.0), (32, 13, 0, 0, 255.0, 0.0), (16, 37, 0, 5, 200.0, 0.0),
    (32, 28, 1, 7, 100.0, 0.0), (48, 14, 1, 14, 255.0, 37.0), (16, 128, 1, 16, 255.0, 0.0), (32, 5, 1, 5, 255.0, 0.0),
])
def test_depthwise_on_the_matrix_cores(g, hw, pad, T, relu_hi, in_z, monkeypatch):
    """k_depthwise3x3_mfma (stride 1, u8 output, ReLU inside the code range) forced onto every shape it accepts:
    1 to 4 chunks of 32 columns, widths and heights that fill neither the last chunk nor the last strip of
    8 rows, no padding, both clamp forms, width-block sizes that split lanes into floor and round columns."""
    monkeypatch.setenv("EHIP_DW_MFMA", "1")
    n = 2 if hw < 56 else 1
    layer = Layer(n, g, g, hw, k=3, pad=pad, out_type=ol.U8, depthwise=True, seed=g + hw + T + 11, w_sigma=0.1, T=T,
                  relu_hi=relu_hi, in_z=in_z)
    res = run_and_compare(layer)
    if res is not None:
        assert res["conv"].kernel_name == "k_depthwise3x3_mfma"


def test_depthwise_matrix_core_kernel_is_the_default_where_it_fits(monkeypatch):
    monkeypatch.delenv("EHIP_DW_MFMA", raising=False)
    E = pkg()
    names = {}
    for hw in (7, 14, 28, 56, 112):
        d = E.make_desc(1, 32, 32, hw, hw, 3, 3, pad=1, g=32, output_type=E.U8, relu_bound=(0.0, 255.0), flatting_t=7,
                        output_quant=(0.02, 0.0))
        names[hw] = E.Conv(d).kernel_name
    assert names[112] == names[56] == names[28] == "k_depthwise3x3_mfma"
    assert names[7] == names[14] == "k_depthwise3x3_u8s8"   # half-empty chunks and strips: the dot4 kernel


# stride 2 (MobileNet's down-sampling layers, scripts/best_configs/mobilenetv1-n64-clx-1s-int8.sh:48:
# pad 0 with the output size asking for one pad row / column at the bottom / right)
@pytest.mark.parametrize("out_type", [ol.U8, ol.S8])
@pytest.mark.parametrize("g,hw,pad,out_hw,T", [(32, 14, 0, 7, 7), (64, 28, 1, None, 14), (16, 15, 0, None, 7), (48, 13, 1, None, 4),
                                               (32, 56, 0, 28, 28), (32, 6, 1, None, 0)])
def test_depthwise_stride2(out_type, g, hw, pad, out_hw, T):
    run_and_compare(Layer(2, g, g, hw, k=3, pad=pad, stride=2, out_type=out_type, depthwise=True, seed=g + hw + T + 3,
                          w_sigma=0.1, T=T, out_hw=out_hw))


@pytest.mark.parametrize("stride,pad,hw", [(1, 1, 14), (1, 0, 9), (2, 1, 15), (2, 0, 14)])
@pytest.mark.parametrize("out_type", [ol.U8, ol.S8])
def test_depthwise_input_zero_point(out_type, stride, pad, hw):
    """z != 0: the shift takes z x all nine weights, padded taps add nothing
    (src/elx_int8_conv_direct_depthwise.cpp:247-289): the reference's values, border included."""
    run_and_compare(Layer(2, 48, 48, hw, k=3, pad=pad, stride=stride, out_type=out_type, depthwise=True,
                          seed=hw + stride + out_type, w_sigma=0.1, T=0, in_z=37.0))


def test_depthwise_stride2_raw_sums():
    run_and_compare(Layer(1, 32, 32, 11, k=3, pad=1, stride=2, out_type=ol.S32, depthwise=True, seed=78, w_sigma=0.1, T=3))


def test_depthwise_odd_width_and_raw_sums():
    run_and_compare(Layer(1, 32, 32, 13, k=3, pad=1, out_type=ol.S32, depthwise=True, seed=23, w_sigma=0.1, T=13))
    run_and_compare(Layer(2, 16, 16, 11, k=3, pad=0, out_type=ol.U8, depthwise=True, seed=29, w_sigma=0.1, T=3))


# ---- input quantizer and reorders ---------------------------------------------------------------------
def test_quantize_input_u8():
    import torch
    E = pkg()
    rng = np.random.default_rng(1)
    x = rng.uniform(0, 1, 1 << 16).astype(np.float32)
    x[:8] = [0.0, 1.0, 0.5 / 255, 1.5 / 255, 2.5 / 255, 254.5 / 255, 0.999999, 1e-9]
    for count in (x.size, x.size - 3, 5):
        d_x = dev(x[:count])
        d_q = torch.zeros(count, dtype=torch.uint8, device="cuda")
        E.quantize_input_u8(d_q, d_x, count, 1.0 / 255.0, 0.0)
        torch.cuda.synchronize()
        assert np.array_equal(host(d_q), ol.quantize_input_u8(x[:count], 1.0 / 255.0, 0.0))
    # exact ties go to the odd neighbour, as in the reference's helper
    t = np.array([0.5, 1.5, 2.5, 3.5, 4.5], np.float32)
    d_q = torch.zeros(5, dtype=torch.uint8, device="cuda")
    E.quantize_input_u8(d_q, dev(t), 5, 1.0, 0.0)
    assert host(d_q).tolist() == [1, 1, 3, 3, 5]


def test_device_reorders():
    import torch
    E = pkg()
    rng = np.random.default_rng(2)
    x = rng.normal(size=(2, 20, 5, 3)).astype(np.float32)
    d = torch.zeros((2, 2, 5, 3, 16), dtype=torch.float32, device="cuda")
    E.reorder_nchw_to_blocked(d, dev(x), 4, 2, 20, 5, 3)
    assert np.array_equal(host(d), ol.to_blocked(x))
    back = torch.zeros((2, 20, 5, 3), dtype=torch.float32, device="cuda")
    E.reorder_blocked_to_nchw(back, d, 4, 2, 20, 5, 3)
    assert np.array_equal(host(back), x)
    u = rng.integers(0, 256, (1, 17, 4, 4)).astype(np.uint8)
    du = torch.zeros((1, 2, 4, 4, 16), dtype=torch.uint8, device="cuda")
    E.reorder_nchw_to_blocked(du, dev(u), 1, 1, 17, 4, 4)
    assert np.array_equal(host(du), ol.to_blocked(u))
    w = rng.normal(size=(20, 35, 3, 3)).astype(np.float32)
    dw = torch.zeros((2, 3, 3, 3, 16, 16), dtype=torch.float32, device="cuda")
    E.reorder_oihw_to_blocked(dw, dev(w), 20, 35, 3, 3)
    assert np.array_equal(host(dw), ol.weights_to_blocked(w))


# ---- layers chained on the device (the reference's --output-as-input, tests/elt_conv.cpp:407-410):
# the u8 output of one layer is the next layer's input without leaving the GPU; requantization to
# the next layer's input scale is the producing layer's own epilogue ------------------------------------
def test_three_layers_chained_on_the_device():
    import torch
    E = pkg()
    l1 = Layer(2, 64, 96, 14, k=3, pad=1, out_type=ol.U8, seed=301, T=14)
    o1 = l1.oracle()["out"]
    l2 = Layer(2, 96, 96, 14, k=3, pad=1, out_type=ol.U8, depthwise=True, seed=302, w_sigma=0.1, T=14, x_blocked=o1)
    o2 = l2.oracle()["out"]
    l3 = Layer(2, 96, 48, 14, stride=2, out_type=ol.S8, seed=303, x_blocked=o2)
    o3 = l3.oracle()["out"]
    convs, bufs = [], []
    for l in (l1, l2, l3):
        c = E.Conv(l.desc)
        c.prepare(dev(l.wb), dev(l.bias))
        convs.append(c)
        bufs.append(torch.zeros(tuple(l.oracle()["out"].shape), dtype=torch.int8 if l.p.out_type == ol.S8 else torch.uint8,
                                device="cuda"))
    x = dev(l1.xb)
    convs[0].execute(bufs[0], x)
    convs[1].execute(bufs[1], bufs[0])
    convs[2].execute(bufs[2], bufs[1])
    torch.cuda.synchronize()
    assert np.array_equal(host(bufs[0]), o1)
    assert np.array_equal(host(bufs[1]), o2)
    assert np.array_equal(host(bufs[2]), o3)


def test_chain_replayed_from_a_hip_graph():
    """execute() of a prepared handle only launches kernels (no allocation, no memset, no synchronisation), so a
    chain of layers can be captured into a HIP graph: three replays with fresh inputs, eager work and
    synchronisations between them, each compared with the eager chain on the same input."""
    import torch
    E = pkg()
    rng = np.random.default_rng(5)
    l1 = Layer(2, 64, 96, 14, k=3, pad=1, out_type=ol.U8, seed=311, T=14)
    l2 = Layer(2, 96, 96, 14, k=3, pad=1, out_type=ol.U8, depthwise=True, seed=312, w_sigma=0.1, T=14)
    l3 = Layer(2, 96, 48, 14, stride=2, out_type=ol.S8, seed=313)
    l4 = Layer(2, 48, 64, 7, k=3, pad=1, stride=1, out_type=ol.F32, seed=314, in_nhwc=False)
    layers = (l1, l2, l3, l4)
    convs, bufs = [], []
    for l in layers:
        c = E.Conv(l.desc)
        c.prepare(dev(l.wb), dev(l.bias))
        convs.append(c)
        shape = (l.p.n, ol.up16(l.p.oc) // 16, l.p.oh, l.p.ow, 16)
        bufs.append(torch.zeros(shape, dtype={ol.S8: torch.int8, ol.U8: torch.uint8, ol.F32: torch.float32}[l.p.out_type],
                                device="cuda"))
    x = dev(l1.xb)

    def chain(stream=0):
        src = x
        for c, l, b in zip(convs, layers, bufs):
            # the s8 codes of layer 3 are layer 4's u8 input bytes as they are: only the chaining is under test
            c.execute(b, src, stream=stream)
            src = b

    inputs = [rng.integers(0, 256, l1.xb.shape).astype(np.uint8) for _ in range(3)]
    eager = []
    for xi in inputs:
        x.copy_(dev(xi))
        chain()
        torch.cuda.synchronize()
        eager.append([host(b).copy() for b in bufs])
    assert not np.array_equal(eager[0][3], eager[1][3])
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        chain(torch.cuda.current_stream().cuda_stream)
    for xi, exp in zip(inputs, eager):
        x.copy_(dev(xi))
        for b in bufs:
            b.fill_(7)                       # eager work between the replays
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        for b, e in zip(bufs, exp):
            assert np.array_equal(bits(host(b)), bits(e))


# ---- error behaviour of setup ---------------------------------------------------------------------------
def test_setup_rejects_what_the_reference_rejects():
    E = pkg()
    bad = [
        E.make_desc(1, 64, 64, 8, 8, 1, 1, pad=1, algorithm=E.CONV_DIRECT_1X1),            # padding in 1x1
        E.make_desc(1, 64, 64, 8, 8, 3, 3, pad=1, algorithm=E.CONV_DIRECT_1X1),            # not a 1x1
        E.make_desc(1, 64, 64, 9, 9, 3, 3, pad=1, stride=3, algorithm=E.CONV_DIRECT),      # stride 3
        E.make_desc(1, 64, 64, 8, 8, 5, 5, pad=0, algorithm=E.CONV_DIRECT),                # pad below k/2 - 1
        E.make_desc(1, 64, 64, 8, 8, 3, 3, pad=1, algorithm=E.CONV_DIRECT, sampling_kind=E.FINE),
        E.make_desc(1, 24, 24, 8, 8, 3, 3, pad=1, g=24, algorithm=E.CONV_DIRECT),          # g % 16
        E.make_desc(1, 64, 64, 8, 8, 1, 1, algorithm=E.CONV_DIRECT_1X1, output_type=E.F32),
    ]
    for d in bad:
        with pytest.raises(E.EulerHipError) as ei:
            E.Conv(d)
        assert ei.value.code in (E.EHIP_UNIMPLEMENTED, E.EHIP_GENERAL_ERROR)
    conv = E.Conv(E.make_desc(1, 64, 64, 8, 8))
    with pytest.raises(E.EulerHipError):
        conv.execute(None, None)


def test_setup_refuses_what_no_kernel_can_address():
    """Limits of the kernels' packed arguments and 32-bit offsets are applied when the handle is created (nothing is
    allocated yet), so that a handle that exists also executes: a depthwise layer of 2^30 output cells is refused
    with a message, not created and then failed at every execute."""
    E = pkg()
    d = E.make_desc(4096, 1024, 1024, 64, 64, 3, 3, pad=1, g=1024, algorithm=E.CONV_DIRECT, flatting_t=16)
    with pytest.raises(E.EulerHipError) as ei:
        E.Conv(d)
    assert ei.value.code == E.EHIP_UNIMPLEMENTED and "tensor too large" in str(ei.value)


@pytest.mark.parametrize("kind", ["1x1 many channels", "1x1 many channels, sum, nhwc", "1x1 few channels", "1x1 few channels f32", "3x3",
                                  "3x3 stride 2", "depthwise 56", "depthwise 7", "depthwise stride 2", "first layer", "first layer f32"])
def test_prepared_handle_on_other_buffers(kind):
    # a handle keeps its launch (kernel, grid, derived and leading scalar arguments) from the first execute; the
    # next execute must run on the tensors it is given: same bytes into a fresh output at another address
    layer = {
        "1x1 many channels": lambda: Layer(2, 256, 144, 14, out_type=ol.U8, seed=501),
        "1x1 many channels, sum, nhwc": lambda: Layer(2, 512, 256, 14, stride=2, out_type=ol.S8, with_sum=True, in_nhwc=True,
                                                      out_nhwc=True, seed=502),
        "1x1 few channels": lambda: Layer(2, 64, 128, 14, out_type=ol.U8, seed=503),
        "1x1 few channels f32": lambda: Layer(1, 32, 48, 9, out_type=ol.F32, seed=504),
        "3x3": lambda: Layer(2, 64, 64, 14, k=3, pad=1, out_type=ol.U8, seed=505),
        "3x3 stride 2": lambda: Layer(2, 32, 32, 15, k=3, pad=1, stride=2, out_type=ol.S8, seed=506),
        "depthwise 56": lambda: Layer(2, 32, 32, 56, k=3, pad=1, depthwise=True, out_type=ol.U8, seed=507, T=14, relu_hi=255.0),
        "depthwise 7": lambda: Layer(3, 48, 48, 7, k=3, pad=1, depthwise=True, out_type=ol.U8, seed=508, T=7, relu_hi=255.0),
        "depthwise stride 2": lambda: Layer(2, 32, 32, 28, k=3, pad=1, stride=2, depthwise=True, out_type=ol.S8, seed=509, T=7),
        "first layer": lambda: Layer(2, 3, 64, 37, k=7, pad=3, stride=2, out_type=ol.S8, seed=510, in_z=128.0, in_nhwc=True, out_nhwc=True),
        "first layer f32": lambda: Layer(2, 3, 32, 23, k=3, pad=1, stride=2, out_type=ol.F32, seed=511, in_nhwc=True, with_relu=False),
    }[kind]()
    res = run_and_compare(layer)
    again = layer.rerun_gpu(res["conv"])
    assert again.shape == res["out"].shape and (again == res["out"]).all(), kind
