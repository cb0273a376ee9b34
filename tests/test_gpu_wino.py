"""GPU parity of the Winograd F(4x4,3x3) int8 pipeline, stage by stage, against the CPU oracle:
calibration range, transformed+quantized weights, u8 transformed input, f32 GEMM result and the
final fp32 output -- all compared bit for bit (the north-star tolerance for fp32 is 1 ULP)."""
import numpy as np
import pytest

import oracle_lib as ol
from gpu_common import bits, dev, host, pkg

pytestmark = pytest.mark.gpu
f32 = np.float32


def make_wino(n, ic, oc, hw, seed, with_bias=True, with_relu=True, tile=6):
    E = pkg()
    rng = np.random.default_rng(seed)
    x = rng.uniform(0, 1, (n, ic, hw, hw)).astype(f32)
    w = rng.normal(0, 0.02, (oc, ic, 3, 3)).astype(f32)
    bias = np.zeros(ol.up16(oc), f32)
    bias[:oc] = rng.normal(0, 0.01, oc)
    xb, wb = ol.to_blocked(x), ol.weights_to_blocked(w)
    p = ol.make_params(n, ic, oc, hw, hw, 3, 3, 1, out_type=ol.F32, in_scale=1.0, with_bias=with_bias,
                       with_relu=with_relu, wino_tile=tile)
    d = E.make_desc(n, ic, oc, hw, hw, 3, 3, 1, algorithm=E.CONV_WINOGRAD, input_type=E.F32, output_type=E.F32,
                    with_bias=with_bias, with_relu=with_relu, input_quant=(1.0, 0.0), tile_size=tile,
                    execution_mode=0xa161, wino_tinput_quant=(1.0, 0.0))
    return E, p, d, xb, wb, bias


@pytest.mark.parametrize("tile", [6, 4, 5])
@pytest.mark.parametrize("n,ic,oc,hw", [(2, 32, 32, 10), (1, 64, 48, 12), (3, 16, 80, 7), (1, 32, 32, 28)])
def test_wino_pipeline(n, ic, oc, hw, tile, monkeypatch):
    """tile 6 = F(4x4,3x3), 4 = F(2x2,3x3), 5 = F(3x3,3x3) (src/eld_conv.cpp:257-270)"""
    import torch
    monkeypatch.setenv("EHIP_WINO_FUSED", "0")   # three kernels: every stage can be inspected
    E, p, d, xb, wb, bias = make_wino(n, ic, oc, hw, seed=n * 100 + hw, tile=tile)
    d_x = dev(xb)
    # calibration of wino_tinput_quant from the fp32 transformed input
    mn, mx = E.wino_tinput_range(d, d_x)
    omn, omx = ol.wino_tinput_range(p, xb)
    assert (f32(mn), f32(mx)) == (f32(omn), f32(omx))
    diff = f32(mx) - f32(mn) + f32(0.000001)
    s_t, z_t = float(diff / f32(255.0)), float(-f32(mn) * f32(255.0) / diff)
    p.tin_scale, p.tin_z = s_t, z_t
    d.tinput_scale, d.tinput_z = s_t, z_t

    twq, tscale, tshift = ol.wino_prepare(p, wb)
    tin = ol.wino_trans_input(p, xb)
    tout, _ = ol.wino_gemm(p, tin, twq, tscale, tshift)
    exp = ol.wino_trans_output(p, tout, bias)

    conv = E.Conv(d)
    d_w, d_b = dev(wb), dev(bias)
    d_out = torch.full(exp.shape, -7.0, dtype=torch.float32, device="cuda")
    conv.prepare(d_w, d_b)
    conv.execute(d_out, d_x, None, d_b)
    torch.cuda.synchronize()
    assert np.array_equal(conv.query(E.Q_WEIGHTS_S8), twq.ravel()), "transformed weights differ"
    assert np.array_equal(bits(conv.query(E.Q_SCALE)), bits(tscale))
    assert np.array_equal(bits(conv.query(E.Q_SHIFT)), bits(tshift))
    g_tin = conv.query(E.Q_TINPUT_U8).reshape(tin.shape)
    assert np.array_equal(g_tin, tin), "u8 transformed input differs at %d cells" % int((g_tin != tin).sum())
    g_tout = conv.query(E.Q_TOUTPUT_F32).reshape(tout.shape)
    assert np.array_equal(bits(g_tout), bits(tout)), "GEMM result differs"
    got = host(d_out)
    assert np.array_equal(bits(got), bits(exp)), "output differs at %d" % int((got != exp).sum())


@pytest.mark.parametrize("tile", [6, 4, 5])
@pytest.mark.parametrize("buf_gather", ["0", "1"])
def test_wino_tinput_under_range_and_both_gathers(tile, buf_gather, monkeypatch):
    """A tinput zero point too small for the data: transformed values below -0.5 end as code 255
    (src/elx_conv_wino_trans_input.cpp:643-650 converts through an unsigned integer), which the input
    transform handles in a second pass of the wave; and the gather with plain loads (what a tensor of 4 GB
    or more takes) next to the one with buffer loads."""
    import torch
    monkeypatch.setenv("EHIP_WINO_FUSED", "0")
    monkeypatch.setenv("EHIP_WINO_BUF_GATHER", buf_gather)
    E, p, d, xb, wb, bias = make_wino(2, 32, 32, 13, seed=77 + tile, tile=tile)
    mn, mx = ol.wino_tinput_range(p, xb)
    s_t = float((f32(mx) - f32(mn)) / f32(255.0))
    z_t = float(-f32(mn) / f32(s_t)) * 0.5      # half of what the range needs
    p.tin_scale, p.tin_z = s_t, z_t
    d.tinput_scale, d.tinput_z = s_t, z_t
    tin = ol.wino_trans_input(p, xb)
    assert (tin == 255).sum() > 300 and (tin == 0).sum() < tin.size // 2
    conv = E.Conv(d)
    d_b = dev(bias)
    d_out = torch.zeros((2, 2, 13, 13, 16), dtype=torch.float32, device="cuda")
    conv.execute(d_out, dev(xb), dev(wb), d_b)
    torch.cuda.synchronize()
    g_tin = conv.query(E.Q_TINPUT_U8).reshape(tin.shape)
    assert np.array_equal(g_tin, tin), "u8 transformed input differs at %d cells" % int((g_tin != tin).sum())


@pytest.mark.parametrize("n,ic,oc,hw", [(2, 32, 32, 10), (1, 64, 48, 12), (3, 16, 80, 7), (1, 32, 144, 28),
                                        (2, 256, 64, 9), (1, 272, 32, 6)])
def test_wino_fused_gemm_and_output_transform(n, ic, oc, hw):
    """Default schedule: GEMM + output transform in one kernel; final output bit for bit."""
    _fused(n, ic, oc, hw)


@pytest.mark.parametrize("ring", ["2", "4", "8"])
def test_wino_fused_every_operand_ring_depth(ring, monkeypatch):
    """256 input channels = 8 k-steps per position: the fused kernel with its operands requested 2, 4 and 8
    k-steps ahead (three instantiations; 4 is the default where it divides the k-steps)"""
    monkeypatch.setenv("EHIP_WINO_KS", ring)
    _fused(2, 256, 80, 9)


@pytest.mark.parametrize("halves", ["1", "2"])
@pytest.mark.parametrize("n,ic,oc,hw", [(2, 256, 80, 9), (1, 64, 144, 13), (3, 32, 64, 7)])
def test_wino_fused_channels_per_workgroup(halves, n, ic, oc, hw, monkeypatch):
    """the fused kernel with workgroups of 32 channels (what layers of few tiles get, so that every CU has a
    workgroup) and of 64; ragged channel counts leave the last workgroup partly past the real channels"""
    monkeypatch.setenv("EHIP_WINO_HALVES", halves)
    _fused(n, ic, oc, hw)


@pytest.mark.parametrize("flat", ["0", "1"])
@pytest.mark.parametrize("tile", [6, 5, 4])
@pytest.mark.parametrize("ic", [64, 128, 48])
def test_wino_fused_few_input_channels(flat, tile, ic, monkeypatch):
    """64 / 128 input channels (2 / 4 k-steps per position): the operand ring running ahead over the positions as one
    flat sequence of steps, and filled position by position; 48 channels (padded to 64) as well"""
    monkeypatch.setenv("EHIP_WINO_FLAT", flat)
    import torch
    E, p, d, xq, wb, bias = make_wino_u8(2, ic, 80, 13, seed=31 + tile + ic, out_type=ol.S8, tile=tile)
    p.tin_scale, p.tin_z = 22.0 / 255.0, 104.0
    d.tinput_scale, d.tinput_z = p.tin_scale, p.tin_z
    _, exp = _oracle_u8(p, xq, wb, bias)
    conv = E.Conv(d)
    assert conv.kernel_name.endswith("k_wino_gemm_output")
    d_b = dev(bias)
    d_out = torch.zeros(exp.shape, dtype=torch.int8, device="cuda")
    conv.prepare(dev(wb), d_b)
    conv.execute(d_out, dev(xq), None, d_b)
    torch.cuda.synchronize()
    got = host(d_out)
    assert np.array_equal(bits(got), bits(exp)), "output differs at %d of %d" % (int((got != exp).sum()), got.size)


@pytest.mark.parametrize("lanes", ["1", "0"])
@pytest.mark.parametrize("tile", [6, 5, 4])
@pytest.mark.parametrize("out_type", [ol.U8, ol.S8])
@pytest.mark.parametrize("n,ic,oc,hw,with_relu", [(2, 64, 80, 13, True), (1, 128, 48, 9, False), (3, 256, 32, 7, True),
                                                  (1, 48, 144, 28, True), (2, 192, 64, 10, True)])
def test_wino_fused_lanes_form(lanes, tile, out_type, n, ic, oc, hw, with_relu, monkeypatch):
    """up to 256 input channels with u8 / s8 output: the fused stage whose lanes own a tile x four channels at every
    position (16 x 16 x 64 matrix instruction, no exchange through LDS), and the general form on the same layers; one,
    two and four k-steps of 64 channels per position, channel counts that leave units, rows and tiles unused"""
    import torch
    monkeypatch.setenv("EHIP_WINO_LANES", lanes)
    E, p, d, xq, wb, bias = make_wino_u8(n, ic, oc, hw, seed=41 + tile + ic + out_type, out_type=out_type, tile=tile,
                                         with_relu=with_relu, out_z=0.0 if out_type == ol.S8 else 2.4)
    p.tin_scale, p.tin_z = 22.0 / 255.0, 104.0
    d.tinput_scale, d.tinput_z = p.tin_scale, p.tin_z
    _, exp = _oracle_u8(p, xq, wb, bias)
    conv = E.Conv(d)
    d_b = dev(bias)
    d_out = torch.zeros(exp.shape, dtype=torch.uint8 if out_type == ol.U8 else torch.int8, device="cuda")
    conv.prepare(dev(wb), d_b)
    conv.execute(d_out, dev(xq), None, d_b)
    torch.cuda.synchronize()
    got = host(d_out)
    assert np.array_equal(bits(got), bits(exp)), "output differs at %d of %d" % (int((got != exp).sum()), got.size)


@pytest.mark.parametrize("slots", ["1", ""])
@pytest.mark.parametrize("wres", ["1", "0"])
@pytest.mark.parametrize("tile", [6, 5, 4])
@pytest.mark.parametrize("out_type,with_sum", [(ol.U8, 0), (ol.S8, 1), (ol.U8, 1)])
@pytest.mark.parametrize("n,ic,oc,hw,with_relu", [(5, 64, 48, 64, True), (1, 128, 32, 36, False), (2, 48, 16, 40, True),
                                                  (3, 128, 80, 30, True)])
def test_wino_fused_lanes_weights_resident(slots, wres, tile, out_type, with_sum, n, ic, oc, hw, with_relu, monkeypatch):
    """at most 128 input channels with u8 / s8 output: workgroups that keep the weights of 16 channels in LDS and walk
    over blocks of 64 tiles, the operand ring running on from one block into the next (one workgroup per XCD and
    channel block, so that every workgroup takes several blocks, and the default grid); an odd number of blocks of 32
    tiles, channels and tiles that leave lanes unused, the in-place sum; and the form that streams both operands"""
    import torch
    monkeypatch.setenv("EHIP_WINO_LANES_WRES", wres)
    if slots:
        monkeypatch.setenv("EHIP_WINO_LANES_SLOTS", slots)
    E, p, d, xq, wb, bias = make_wino_u8(n, ic, oc, hw, seed=57 + tile + ic + out_type, out_type=out_type, tile=tile,
                                         with_relu=with_relu, out_z=0.0 if out_type == ol.S8 else 1.6)
    p.with_sum = with_sum
    d.with_ip_sum = with_sum
    p.tin_scale, p.tin_z = 22.0 / 255.0, 104.0
    d.tinput_scale, d.tinput_z = p.tin_scale, p.tin_z
    rng = np.random.default_rng(91 + tile + hw)
    shape = (n, ol.up16(oc) // 16, hw, hw, 16)
    old = rng.integers(-30 if out_type == ol.S8 else 0, 60, shape).astype(ol.NP_OF[out_type])
    twq, tscale, tshift = ol.wino_prepare(p, wb)
    tout, _ = ol.wino_gemm(p, ol.wino_trans_input(p, xq.astype(f32)), twq, tscale, tshift)
    exp = ol.wino_trans_output(p, tout, bias, out_init=old if with_sum else None)
    conv = E.Conv(d)
    d_out = dev(old)
    d_b = dev(bias)
    conv.prepare(dev(wb), d_b)
    conv.execute(d_out, dev(xq), None, d_b)
    torch.cuda.synchronize()
    got = host(d_out)
    assert np.array_equal(bits(got), bits(exp)), "output differs at %d of %d" % (int((got != exp).sum()), got.size)


@pytest.mark.parametrize("waves", ["4", "8"])
@pytest.mark.parametrize("slots", ["1", ""])
@pytest.mark.parametrize("tile", [6, 5, 4])
@pytest.mark.parametrize("out_type,with_sum", [(ol.S8, 0), (ol.U8, 1), (ol.F32, 0)])
@pytest.mark.parametrize("n,ic,oc,hw", [(2, 256, 48, 30), (1, 192, 32, 36), (3, 512, 32, 18)])
def test_wino_fused_lanes_weights_resident_many_channels(waves, slots, tile, out_type, with_sum, n, ic, oc, hw, monkeypatch):
    """192 / 256 input channels (three / four k-steps of 64 per position): the weights of 16 channels fill most of the
    LDS, one workgroup per CU, of four or of eight waves (64 / 128 tiles a block); 512 channels: with tile size 4 the
    same, with tile sizes 6 and 5 two passes over half of the columns each, the first pass's results parked in memory"""
    import torch
    monkeypatch.setenv("EHIP_WINO_LANES_WAVES", waves)
    monkeypatch.setenv("EHIP_WINO_LANES_TWO_PASS", "1")   # (by itself the library keeps so small a layer on the general kernel)
    if slots:
        monkeypatch.setenv("EHIP_WINO_LANES_SLOTS", slots)
    E, p, d, xq, wb, bias = make_wino_u8(n, ic, oc, hw, seed=63 + tile + ic + out_type, out_type=out_type, tile=tile,
                                         out_z=0.0 if out_type != ol.U8 else 1.6)
    p.with_sum = with_sum
    d.with_ip_sum = with_sum
    p.tin_scale, p.tin_z = 22.0 / 255.0, 104.0
    d.tinput_scale, d.tinput_z = p.tin_scale, p.tin_z
    rng = np.random.default_rng(93 + tile + hw)
    shape = (n, ol.up16(oc) // 16, hw, hw, 16)
    old = (rng.normal(0, 0.05, shape).astype(f32) if out_type == ol.F32 else
           rng.integers(-30 if out_type == ol.S8 else 0, 60, shape).astype(ol.NP_OF[out_type]))
    twq, tscale, tshift = ol.wino_prepare(p, wb)
    tout, _ = ol.wino_gemm(p, ol.wino_trans_input(p, xq.astype(f32)), twq, tscale, tshift)
    exp = ol.wino_trans_output(p, tout, bias, out_init=old if with_sum else None)
    conv = E.Conv(d)
    d_out = dev(old)
    d_b = dev(bias)
    conv.prepare(dev(wb), d_b)
    conv.execute(d_out, dev(xq), None, d_b)
    torch.cuda.synchronize()
    assert conv.kernel_name.endswith("k_wino_gemm_output_lanes_wres")
    got = host(d_out)
    assert np.array_equal(bits(got), bits(exp)), "output differs at %d of %d" % (int((got != exp).sum()), got.size)


@pytest.mark.parametrize("out_type", [ol.S8, ol.F32])
@pytest.mark.parametrize("n,ic,oc,hw", [(8, 64, 64, 224), (16, 128, 128, 112), (16, 256, 256, 56), (64, 512, 512, 28)])
def test_wino_fused_forms_agree_at_full_size(out_type, n, ic, oc, hw, monkeypatch):
    """the VGG layers at their real planes (a share of the batch), where the weights-resident workgroups take many blocks
    of tiles each: the three forms of the fused stage -- lanes with resident weights, lanes with both operands streamed,
    the general kernel -- written independently of each other, leave the same bytes (each is pinned against the oracle
    at sizes the oracle finishes in seconds by the tests above)"""
    import torch
    E = pkg()
    g = torch.Generator(device="cuda").manual_seed(1234 + ic + hw)
    x = torch.randint(0, 256, (n, ic // 16, hw, hw, 16), dtype=torch.uint8, device="cuda", generator=g)
    w = (torch.randn((oc // 16, ic // 16, 3, 3, 16, 16), device="cuda", generator=g) * 0.02).float()
    bias = (torch.randn(oc, device="cuda", generator=g) * 0.01).float()
    out_scale = 4.0 * 0.02 * np.sqrt(9 * ic / 3.0) / 127.0
    d = E.make_desc(n, ic, oc, hw, hw, 3, 3, 1, algorithm=E.CONV_WINOGRAD, input_type=E.U8, output_type=out_type,
                    with_bias=True, with_relu=True, input_quant=(1.0 / 255.0, 0.0), tile_size=6, execution_mode=0xa161,
                    wino_tinput_quant=(22.0 / 255.0, 104.0), output_quant=(out_scale, 0.0))
    outs = {}
    forms = [("resident", {}), ("streamed", {"EHIP_WINO_LANES_WRES": "0"}), ("general", {"EHIP_WINO_LANES": "0"})]
    if ic > 256:
        forms.pop(1)   # (the streamed form stops at 256 input channels; 512: two passes with resident weights)
    for name, env in forms:
        for k in ("EHIP_WINO_LANES_WRES", "EHIP_WINO_LANES"):
            monkeypatch.delenv(k, raising=False)
        for k, v in env.items():
            monkeypatch.setenv(k, v)
        conv = E.Conv(d)
        out = torch.zeros((n, oc // 16, hw, hw, 16), dtype=torch.float32 if out_type == ol.F32 else torch.int8, device="cuda")
        conv.prepare(w, bias)
        conv.execute(out, x, None, bias)
        torch.cuda.synchronize()
        outs[name] = (out, conv.kernel_name)
        del conv
    assert outs["resident"][1].endswith("k_wino_gemm_output_lanes_wres")
    if "streamed" in outs:
        assert outs["streamed"][1].endswith("k_wino_gemm_output_lanes")
    assert outs["general"][1].endswith("k_wino_gemm_output")
    ref = outs["general"][0]
    assert int((ref.view(torch.uint8) != 0).sum()) > ref.numel() // 8   # (not a layer of zeros)
    for name in ("resident", "streamed"):
        if name not in outs:
            continue
        got = outs[name][0]
        assert torch.equal(got.view(torch.uint8), ref.view(torch.uint8)), "%s differs from the general kernel at %d values" % (
            name, int((got != ref).sum()))


def _fused(n, ic, oc, hw):
    import torch
    E, p, d, xb, wb, bias = make_wino(n, ic, oc, hw, seed=n * 10 + hw + ic)
    s_t, z_t = 22.0 / 255.0, 104.0
    p.tin_scale, p.tin_z = s_t, z_t
    d.tinput_scale, d.tinput_z = s_t, z_t
    twq, tscale, tshift = ol.wino_prepare(p, wb)
    tin = ol.wino_trans_input(p, xb)
    tout, _ = ol.wino_gemm(p, tin, twq, tscale, tshift)
    exp = ol.wino_trans_output(p, tout, bias)
    conv = E.Conv(d)
    assert conv.kernel_name.endswith("k_wino_gemm_output")
    d_b = dev(bias)
    d_out = torch.full(exp.shape, -7.0, dtype=torch.float32, device="cuda")
    conv.prepare(dev(wb), d_b)
    conv.execute(d_out, dev(xb), None, d_b)
    torch.cuda.synchronize()
    assert np.array_equal(conv.query(E.Q_TINPUT_U8).reshape(tin.shape), tin)
    got = host(d_out)
    assert np.array_equal(bits(got), bits(exp)), "output differs at %d of %d" % (int((got != exp).sum()), got.size)


def make_wino_u8(n, ic, oc, hw, seed, out_type, with_bias=True, with_relu=True, out_scale=None, out_z=0.0, tile=6):
    """u8 user input (codes of U[0,1) at scale 1/255), f32 / u8 / s8 user output: the data-type
    configurations U8F32F32F32, U8F32U8F32, U8F32S8F32 of the reference (src/eld_conv.cpp:275-281)."""
    E = pkg()
    rng = np.random.default_rng(seed)
    x = rng.uniform(0, 1, (n, ic, hw, hw)).astype(f32)
    w = rng.normal(0, 0.02, (oc, ic, 3, 3)).astype(f32)
    bias = np.zeros(ol.up16(oc), f32)
    bias[:oc] = rng.normal(0, 0.01, oc)
    xq = ol.to_blocked(ol.quantize_input_u8(x, 1.0 / 255.0, 0.0))
    wb = ol.weights_to_blocked(w)
    if out_scale is None:
        out_scale = 4.0 * 0.02 * np.sqrt(9 * ic / 3.0) / (127.0 if out_type == ol.S8 else 255.0)
    p = ol.make_params(n, ic, oc, hw, hw, 3, 3, 1, out_type=out_type, in_scale=1.0 / 255.0, with_bias=with_bias,
                       with_relu=with_relu, out_scale=out_scale, out_z=out_z, wino_tile=tile)
    d = E.make_desc(n, ic, oc, hw, hw, 3, 3, 1, algorithm=E.CONV_WINOGRAD, input_type=E.U8, output_type=out_type,
                    with_bias=with_bias, with_relu=with_relu, input_quant=(1.0 / 255.0, 0.0), tile_size=tile,
                    execution_mode=0xa161, wino_tinput_quant=(1.0, 0.0), output_quant=(out_scale, out_z))
    return E, p, d, xq, wb, bias


def _oracle_u8(p, xq, wb, bias):
    # the reference transforms the u8 codes as floats (src/kernel/elk_conv_wino_4x4_3x3_input.hxx:40-47)
    xf = xq.astype(f32)
    twq, tscale, tshift = ol.wino_prepare(p, wb)
    tin = ol.wino_trans_input(p, xf)
    tout, _ = ol.wino_gemm(p, tin, twq, tscale, tshift)
    return tin, ol.wino_trans_output(p, tout, bias)


@pytest.mark.parametrize("fused", ["1", "0"])
@pytest.mark.parametrize("out_type", [ol.F32, ol.U8, ol.S8])
@pytest.mark.parametrize("n,ic,oc,hw", [(2, 32, 32, 10), (1, 64, 80, 12), (1, 48, 32, 7)])
def test_wino_u8_input_quantized_output(fused, out_type, n, ic, oc, hw, monkeypatch):
    import torch
    monkeypatch.setenv("EHIP_WINO_FUSED", fused)
    E, p, d, xq, wb, bias = make_wino_u8(n, ic, oc, hw, seed=7 * n + hw + ic + out_type, out_type=out_type)
    d_x = dev(xq)
    # calibration on the codes: the transformed-input range in code units, times the input scale
    mn, mx = E.wino_tinput_range(d, d_x)
    omn, omx = ol.wino_tinput_range(p, xq.astype(f32))
    assert (f32(mn), f32(mx)) == (f32(omn), f32(omx))
    diff = (f32(mx) - f32(mn)) * f32(1.0 / 255.0) + f32(0.000001)
    s_t, z_t = float(diff / f32(255.0)), float(-f32(mn) * f32(1.0 / 255.0) * f32(255.0) / diff)
    p.tin_scale, p.tin_z = s_t, z_t
    d.tinput_scale, d.tinput_z = s_t, z_t
    tin, exp = _oracle_u8(p, xq, wb, bias)
    conv = E.Conv(d)
    d_b = dev(bias)
    tdt = {ol.F32: torch.float32, ol.U8: torch.uint8, ol.S8: torch.int8}[out_type]
    d_out = torch.full(exp.shape, 5, dtype=tdt, device="cuda")
    conv.prepare(dev(wb), d_b)
    conv.execute(d_out, d_x, None, d_b)
    torch.cuda.synchronize()
    g_tin = conv.query(E.Q_TINPUT_U8).reshape(tin.shape)
    assert np.array_equal(g_tin, tin), "u8 transformed input differs at %d cells" % int((g_tin != tin).sum())
    got = host(d_out)
    assert got.dtype == exp.dtype
    assert np.array_equal(bits(got), bits(exp)), "output differs at %d of %d" % (int((got != exp).sum()), got.size)
    if out_type != ol.F32:   # the codes really use the range
        assert len(np.unique(got)) > 40


def test_wino_u8_output_without_relu_wraps_negatives_to_255():
    """No ReLU and u8 output: the reference's store converts through an unsigned integer, so negative
    values saturate to 255 (src/kernel/elk_conv_wino_4x4_3x3_output.hxx:97-101)."""
    import torch
    E, p, d, xq, wb, bias = make_wino_u8(1, 32, 32, 9, seed=11, out_type=ol.U8, with_relu=False, out_z=2.4)
    p.tin_scale, p.tin_z = 22.0 / 255.0, 104.0
    d.tinput_scale, d.tinput_z = p.tin_scale, p.tin_z
    _, exp = _oracle_u8(p, xq, wb, bias)
    conv = E.Conv(d)
    d_out = torch.zeros(exp.shape, dtype=torch.uint8, device="cuda")
    d_b = dev(bias)
    conv.execute(d_out, dev(xq), dev(wb), d_b)
    torch.cuda.synchronize()
    got = host(d_out)
    assert np.array_equal(got, exp)
    assert (exp == 255).sum() > exp.size // 10


def test_wino_no_bias_no_relu():
    import torch
    E, p, d, xb, wb, bias = make_wino(1, 32, 32, 9, seed=4, with_bias=False, with_relu=False)
    p.tin_scale, p.tin_z = 0.04, 100.3
    d.tinput_scale, d.tinput_z = 0.04, 100.3
    twq, tscale, tshift = ol.wino_prepare(p, wb)
    tout, _ = ol.wino_gemm(p, ol.wino_trans_input(p, xb), twq, tscale, tshift)
    exp = ol.wino_trans_output(p, tout, bias)
    conv = E.Conv(d)
    d_out = torch.zeros(exp.shape, dtype=torch.float32, device="cuda")
    conv.execute(d_out, dev(xb), dev(wb), None)
    torch.cuda.synchronize()
    assert np.array_equal(bits(host(d_out)), bits(exp))


# ---- tile sizes 4 (F(2x2,3x3)) and 5 (F(3x3,3x3)) with u8 input and every user output type ------------
@pytest.mark.parametrize("fused", ["1", "0"])
@pytest.mark.parametrize("tile", [4, 5])
@pytest.mark.parametrize("out_type", [ol.F32, ol.U8, ol.S8])
@pytest.mark.parametrize("n,ic,oc,hw,with_relu", [(2, 32, 32, 10, True), (1, 64, 80, 13, True), (1, 48, 32, 7, False),
                                                  (2, 16, 16, 4, True)])
def test_wino_other_tiles_u8_input_quantized_output(tile, out_type, n, ic, oc, hw, with_relu, fused, monkeypatch):
    """The F(2x2,3x3) store rounds toward minus infinity, the others to nearest even; without ReLU negative
    values of a u8 output end as 255 (src/kernel/elk_conv_wino_2x2_3x3_output.hxx:142-151,
    src/kernel/elk_conv_wino_3x3_3x3_output.hxx:74-86)."""
    import torch
    monkeypatch.setenv("EHIP_WINO_FUSED", fused)   # both schedules against the oracle: they are byte-identical
    E, p, d, xq, wb, bias = make_wino_u8(n, ic, oc, hw, seed=9 * n + hw + ic + out_type + tile, out_type=out_type,
                                         with_relu=with_relu, out_z=0.0 if out_type == ol.S8 else 2.4, tile=tile)
    d_x = dev(xq)
    mn, mx = E.wino_tinput_range(d, d_x)
    omn, omx = ol.wino_tinput_range(p, xq.astype(f32))
    assert (f32(mn), f32(mx)) == (f32(omn), f32(omx))
    diff = (f32(mx) - f32(mn)) * f32(1.0 / 255.0) + f32(0.000001)
    s_t, z_t = float(diff / f32(255.0)), float(-f32(mn) * f32(1.0 / 255.0) * f32(255.0) / diff)
    p.tin_scale, p.tin_z = s_t, z_t
    d.tinput_scale, d.tinput_z = s_t, z_t
    tin, exp = _oracle_u8(p, xq, wb, bias)
    assert tin.shape[0] == tile * tile
    conv = E.Conv(d)
    assert conv.kernel_name.endswith("k_wino_gemm_output" if fused == "1" else "k_wino_trans_output")
    tdt = {ol.F32: torch.float32, ol.U8: torch.uint8, ol.S8: torch.int8}[out_type]
    d_out = torch.full(exp.shape, 5, dtype=tdt, device="cuda")
    d_b = dev(bias)
    conv.execute(d_out, d_x, dev(wb), d_b)
    torch.cuda.synchronize()
    twq, tscale, tshift = ol.wino_prepare(p, wb)
    assert np.array_equal(conv.query(E.Q_WEIGHTS_S8), twq.ravel()), "transformed weights differ"
    assert np.array_equal(bits(conv.query(E.Q_SCALE)), bits(tscale))
    g_tin = conv.query(E.Q_TINPUT_U8).reshape(tin.shape)
    assert np.array_equal(g_tin, tin), "u8 transformed input differs at %d cells" % int((g_tin != tin).sum())
    got = host(d_out)
    assert np.array_equal(bits(got), bits(exp)), "output differs at %d of %d" % (int((got != exp).sum()), got.size)


def test_wino_automatic_tile_size():
    """tile_size 0: the reference picks 6 or 4 from the layer's multiply-accumulates per byte read
    (src/eld_conv.cpp:231-236); a small layer gets F(2x2,3x3)."""
    import torch
    E, p, d, xb, wb, bias = make_wino(1, 16, 16, 8, seed=3, tile=4)
    d.tile_size = 0
    p.tin_scale, p.tin_z = 6.0 / 255.0, 120.0
    d.tinput_scale, d.tinput_z = p.tin_scale, p.tin_z
    twq, tscale, tshift = ol.wino_prepare(p, wb)
    tout, _ = ol.wino_gemm(p, ol.wino_trans_input(p, xb), twq, tscale, tshift)
    exp = ol.wino_trans_output(p, tout, bias)
    conv = E.Conv(d)
    d_out = torch.zeros(exp.shape, dtype=torch.float32, device="cuda")
    d_b = dev(bias)
    conv.execute(d_out, dev(xb), dev(wb), d_b)
    torch.cuda.synchronize()
    assert conv.query(E.Q_WEIGHTS_S8).size == 16 * twq.shape[1] * twq.shape[2]
    assert np.array_equal(bits(host(d_out)), bits(exp))


# ---- in-place sum (with_ip_sum) in the output transform ------------------------------------------------
@pytest.mark.parametrize("fused", ["1", "0"])
@pytest.mark.parametrize("tile", [6, 4, 5])
@pytest.mark.parametrize("out_type", [ol.F32, ol.U8, ol.S8])
def test_wino_with_ip_sum(tile, out_type, fused, monkeypatch):
    """The old output (f32, or the u8 / s8 code as it is) is added after the output quantization and before
    the ReLU (src/kernel/elk_conv_wino_4x4_3x3_output.hxx:168-187)."""
    import torch
    monkeypatch.setenv("EHIP_WINO_FUSED", fused)
    n, ic, oc, hw = 2, 32, 48, 11
    E, p, d, xq, wb, bias = make_wino_u8(n, ic, oc, hw, seed=31 + tile + out_type, out_type=out_type,
                                         out_z=0.0 if out_type == ol.S8 else 1.6, tile=tile)
    p.with_sum = 1
    d.with_ip_sum = 1
    p.tin_scale, p.tin_z = 22.0 / 255.0, 104.0
    d.tinput_scale, d.tinput_z = p.tin_scale, p.tin_z
    rng = np.random.default_rng(77 + tile)
    shape = (n, ol.up16(oc) // 16, hw, hw, 16)
    if out_type == ol.F32:
        old = rng.normal(0, 0.05, shape).astype(f32)
    else:
        old = rng.integers(-30 if out_type == ol.S8 else 0, 60, shape).astype(ol.NP_OF[out_type])
    twq, tscale, tshift = ol.wino_prepare(p, wb)
    tout, _ = ol.wino_gemm(p, ol.wino_trans_input(p, xq.astype(f32)), twq, tscale, tshift)
    exp = ol.wino_trans_output(p, tout, bias, out_init=old)
    assert not np.array_equal(exp, ol.wino_trans_output(p, tout, bias))   # the sum operand matters
    conv = E.Conv(d)
    assert conv.kernel_name.endswith("k_wino_gemm_output" if fused == "1" else "k_wino_trans_output")
    d_out = dev(old)
    d_b = dev(bias)
    conv.execute(d_out, dev(xq), dev(wb), d_b)
    torch.cuda.synchronize()
    got = host(d_out)
    assert np.array_equal(bits(got), bits(exp)), "output differs at %d of %d" % (int((got != exp).sum()), got.size)


# ---- nhwc activations -----------------------------------------------------------------------------------
@pytest.mark.parametrize("fused", ["1", "0"])
@pytest.mark.parametrize("in_nhwc,out_nhwc", [(True, True), (True, False), (False, True)])
@pytest.mark.parametrize("tile,out_type,with_sum", [(6, ol.F32, 0), (6, ol.U8, 0), (6, ol.S8, 1), (4, ol.U8, 0),
                                                    (5, ol.F32, 1), (5, ol.S8, 0)])
def test_wino_nhwc_activations(tile, out_type, with_sum, in_nhwc, out_nhwc, fused, monkeypatch):
    """The transforms read and write [n][h][w][c] activations (the reference's nhwc variants of the
    Winograd transforms, src/elx_conv_wino_trans_input.cpp:226-262, src/elx_conv_wino_trans_output.cpp:136-190):
    the same values as with nChw16c, in the other layout."""
    import torch
    monkeypatch.setenv("EHIP_WINO_FUSED", fused)
    n, ic, oc, hw = 2, 48, 80, 13
    E, p, d, xq, wb, bias = make_wino_u8(n, ic, oc, hw, seed=91 + tile + out_type, out_type=out_type,
                                         out_z=0.0 if out_type == ol.S8 else 2.4, tile=tile)
    p.with_sum = with_sum
    d.with_ip_sum = with_sum
    p.tin_scale, p.tin_z = 22.0 / 255.0, 104.0
    d.tinput_scale, d.tinput_z = p.tin_scale, p.tin_z
    if in_nhwc:
        d.input_fmt = E.NHWC
    if out_nhwc:
        d.output_fmt = E.NHWC
    rng = np.random.default_rng(5 + tile)
    shape = (n, oc // 16, hw, hw, 16)
    if out_type == ol.F32:
        old = rng.normal(0, 0.05, shape).astype(f32)
    else:
        old = rng.integers(-30 if out_type == ol.S8 else 0, 60, shape).astype(ol.NP_OF[out_type])
    twq, tscale, tshift = ol.wino_prepare(p, wb)
    tout, _ = ol.wino_gemm(p, ol.wino_trans_input(p, xq.astype(f32)), twq, tscale, tshift)
    exp = ol.wino_trans_output(p, tout, bias, out_init=old if with_sum else None)
    conv = E.Conv(d)
    d_x = dev(ol.blocked_to_nhwc(xq, ic) if in_nhwc else xq)
    d_out = dev(ol.blocked_to_nhwc(old, oc) if out_nhwc else old)
    d_b = dev(bias)
    conv.execute(d_out, d_x, dev(wb), d_b)
    torch.cuda.synchronize()
    got = host(d_out)
    if out_nhwc:
        exp = ol.blocked_to_nhwc(exp, oc)
    assert got.shape == exp.shape
    assert np.array_equal(bits(got), bits(exp)), "output differs at %d of %d" % (int((got != exp).sum()), got.size)


def test_wino_nhwc_f32_input_and_range():
    """fp32 nhwc input: calibration range and the whole pipeline match the blocked layout's."""
    import torch
    E, p, d, xb, wb, bias = make_wino(2, 32, 48, 11, seed=3)
    p.tin_scale, p.tin_z = 9.0 / 255.0, 100.0
    d.tinput_scale, d.tinput_z = p.tin_scale, p.tin_z
    d.input_fmt = d.output_fmt = E.NHWC
    d_x = dev(ol.blocked_to_nhwc(xb, 32))
    mn, mx = E.wino_tinput_range(d, d_x)
    omn, omx = ol.wino_tinput_range(p, xb)
    assert (f32(mn), f32(mx)) == (f32(omn), f32(omx))
    twq, tscale, tshift = ol.wino_prepare(p, wb)
    tout, _ = ol.wino_gemm(p, ol.wino_trans_input(p, xb), twq, tscale, tshift)
    exp = ol.blocked_to_nhwc(ol.wino_trans_output(p, tout, bias), 48)
    conv = E.Conv(d)
    d_out = torch.zeros(exp.shape, dtype=torch.float32, device="cuda")
    d_b = dev(bias)
    conv.execute(d_out, d_x, dev(wb), d_b)
    torch.cuda.synchronize()
    assert np.array_equal(bits(host(d_out)), bits(exp))


def test_wino_nhwc_channel_tail_is_refused():
    E, p, d, xq, wb, bias = make_wino_u8(1, 24, 32, 8, seed=1, out_type=ol.U8)
    d.input_fmt = E.NHWC
    with pytest.raises(E.EulerHipError, match="channel tail"):
        E.Conv(d)


@pytest.mark.parametrize("tile", [6, 4])
def test_wino_replayed_from_a_hip_graph(tile):
    """The Winograd execute of a prepared handle (input transform, GEMMs, output transform over the handle's
    own workspace) launches kernels only, so it can be captured: three replays with fresh inputs, eager work
    and synchronisations between them, each equal to the eager result."""
    import torch
    E, p, d, xq, wb, bias = make_wino_u8(3, 48, 80, 13, seed=17 + tile, out_type=ol.S8, tile=tile)
    d.tinput_scale, d.tinput_z = 22.0 / 255.0, 104.0
    conv = E.Conv(d)
    d_b = dev(bias)
    conv.prepare(dev(wb), d_b)
    rng = np.random.default_rng(3)
    inputs = [rng.integers(0, 256, xq.shape).astype(np.uint8) for _ in range(3)]
    x = dev(xq)
    out = torch.zeros((3, 5, 13, 13, 16), dtype=torch.int8, device="cuda")
    eager = []
    for xi in inputs:
        x.copy_(dev(xi))
        conv.execute(out, x, None, d_b)
        torch.cuda.synchronize()
        eager.append(host(out).copy())
    assert not np.array_equal(eager[0], eager[1])
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        conv.execute(out, x, None, d_b, stream=torch.cuda.current_stream().cuda_stream)
    for xi, exp in zip(inputs, eager):
        x.copy_(dev(xi))
        out.fill_(9)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert np.array_equal(host(out), exp)
