"""The C++ surface (include/euler.hpp: eld_conv_t::setup + elx_conv on host buffers, reorder<>) end
to end: a prebuilt client program (tests/cxx/euler_api_check.cpp, compiled by build()) runs a layer
the way a program written against the reference does; its output is compared bit for bit with the
CPU oracle."""
import os
import subprocess

import numpy as np
import pytest

import oracle_lib as ol
from gpu_common import Layer, pkg

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CHECK = os.path.join(ROOT, "deep-learning-math-kernel-research_amd", "build", "euler_api_check")


def from_blocked(b, c):
    n, c2, h, w, _ = b.shape
    return np.ascontiguousarray(b.transpose(0, 1, 4, 2, 3).reshape(n, c2 * 16, h, w)[:, :c])


CASES = [
    dict(n=2, ic=64, oc=48, hw=12, k=3, pad=1, out_type=ol.U8, T=12),
    dict(n=2, ic=96, oc=64, hw=7, k=1, pad=0, out_type=ol.S8, with_sum=True),
    dict(n=1, ic=32, oc=80, hw=9, k=1, pad=0, out_type=ol.F32),
    dict(n=2, ic=32, oc=32, hw=14, k=3, pad=1, out_type=ol.U8, depthwise=True, T=7),
    dict(n=2, ic=64, oc=64, hw=14, k=3, pad=1, stride=2, out_type=ol.S8, T=7),
    dict(n=2, ic=32, oc=32, hw=14, k=3, pad=1, stride=2, out_type=ol.U8, depthwise=True, T=7),
    dict(n=2, ic=96, oc=64, hw=7, k=1, pad=0, out_type=ol.S8, with_sum=True, nhwc=True),
    dict(n=2, ic=3, oc=64, hw=22, k=7, pad=3, stride=2, out_type=ol.S8, nhwc=True),   # a first layer: 3-channel nhwc image
]


@pytest.mark.parametrize("case", CASES, ids=["3x3_u8", "1x1_s8_sum", "1x1_f32", "depthwise_u8", "3x3_s2_s8", "depthwise_s2_u8",
                                              "1x1_s8_sum_nhwc", "7x7_s2_3ch_nhwc"])
def test_elx_conv_on_host_buffers(case, tmp_path):
    assert os.path.exists(CHECK), "euler_api_check is not built (python -c 'import __graft_entry__ as g; g.build()')"
    c = dict(stride=1, with_sum=False, depthwise=False, T=0, nhwc=False)
    c.update(case)
    layer = Layer(c["n"], c["ic"], c["oc"], c["hw"], k=c["k"], pad=c["pad"], stride=c["stride"], out_type=c["out_type"],
                  with_sum=c["with_sum"], depthwise=c["depthwise"], seed=321 + c["ic"], T=c["T"],
                  w_sigma=0.1 if c["depthwise"] else 0.05)
    exp = from_blocked(layer.oracle()["out"], c["oc"])
    fin, fout = tmp_path / "in.bin", tmp_path / "out.bin"
    with open(fin, "wb") as f:
        f.write(np.ascontiguousarray(layer.x_u8).tobytes())
        f.write(np.ascontiguousarray(layer.w, dtype=np.float32).tobytes())
        f.write(np.ascontiguousarray(layer.bias[:c["oc"]], dtype=np.float32).tobytes())
        if c["with_sum"]:
            f.write(from_blocked(layer.old, c["oc"]).tobytes())
    d = layer.desc
    g = c["ic"] if c["depthwise"] else 1
    args = [CHECK, str(fin), str(fout)] + [str(v) for v in (
        c["n"], c["ic"], c["oc"], c["hw"], c["k"], c["pad"], c["stride"], c["out_type"], d.algorithm,
        int(c["with_sum"]), c["T"], repr(float(d.output_scale)), repr(float(d.sum_scale)), g, int(c["nhwc"]))]
    r = subprocess.run(args, capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, "rc=%d stdout=%s stderr=%s" % (r.returncode, r.stdout, r.stderr)
    got = np.fromfile(fout, dtype=exp.dtype).reshape(exp.shape)
    assert np.array_equal(got.view(np.uint8), exp.view(np.uint8)), "%d values differ" % int((got != exp).sum())
    if case is CASES[0] or case is CASES[1]:
        # eager mode with a managed output: the client reads the result on the host straight after elx_conv returns
        r = subprocess.run(args, capture_output=True, text=True, timeout=120,
                           env=dict(os.environ, EULER_CHECK_MANAGED_OUTPUT="1"))
        assert r.returncode == 0, "rc=%d stdout=%s stderr=%s" % (r.returncode, r.stdout, r.stderr)
        got = np.fromfile(fout, dtype=exp.dtype).reshape(exp.shape)
        assert np.array_equal(got.view(np.uint8), exp.view(np.uint8)), "managed output: %d values differ" % int((got != exp).sum())


@pytest.mark.parametrize("in_type,out_type,tile,mode", [
    (ol.F32, ol.F32, 6, 0xa161), (ol.F32, ol.F32, 6, 0xa133), (ol.U8, ol.S8, 6, 0xa161), (ol.U8, ol.F32, 4, 0xa161),
    (ol.F32, ol.F32, 0, 0xa161),
], ids=["f32_f32_a161", "f32_f32_a133", "u8_s8_a161", "u8_f32_tile4", "f32_f32_automatic_tile"])
def test_elx_conv_winograd_on_host_buffers(in_type, out_type, tile, mode, tmp_path):
    """eld_conv_t{CONV_WINOGRAD, tile_size, execution_mode, wino_tinput_quant} -> setup() -> elx_conv()
    (dispatch of src/eld_conv.cpp:273-305) with the data-type configurations F32F32F32F32 (int8 GEMM inside,
    as `--f16c-opt`-less int8 Winograd runs of the reference), U8F32S8F32 and U8F32F32F32."""
    assert os.path.exists(CHECK), "euler_api_check is not built (python -c 'import __graft_entry__ as g; g.build()')"
    n, ic, oc, hw = 2, 48, 80, 14
    rng = np.random.default_rng(90 + in_type + out_type + tile)
    x = rng.uniform(0, 1, (n, ic, hw, hw)).astype(np.float32)
    w = rng.normal(0, 0.02, (oc, ic, 3, 3)).astype(np.float32)
    bias = np.zeros(ol.up16(oc), np.float32)
    bias[:oc] = rng.normal(0, 0.01, oc)
    out_scale = 4.0 * 0.02 * np.sqrt(9 * ic / 3.0) / 127.0 if out_type == ol.S8 else 1.0
    in_scale = 1.0 if in_type == ol.F32 else 1.0 / 255.0
    # setup() picks the tile size itself when the descriptor leaves it 0 (src/eld_conv.cpp:231-236): this
    # shape has 2 * 4 * 4 = 32 tiles of F(4x4,3x3) and 80 output channels, 32 * 80 / (32 + 80) = 22.9
    # multiply-accumulates per read, below the threshold of 25 -> F(2x2,3x3), tile size 4
    p = ol.make_params(n, ic, oc, hw, hw, 3, 3, 1, out_type=out_type, in_scale=in_scale, out_scale=out_scale,
                       wino_tile=tile or 4, relu_hi=127.0 if out_type == ol.S8 else ol.FLT_MAX)
    if in_type == ol.F32:
        xin, xuser = ol.to_blocked(x), x
    else:
        xq = ol.quantize_input_u8(x, 1.0 / 255.0, 0.0)
        xin, xuser = ol.to_blocked(xq).astype(np.float32), xq   # the transform reads the codes as floats
    mn, mx = ol.wino_tinput_range(p, xin)
    diff = (np.float32(mx) - np.float32(mn)) * np.float32(in_scale) + np.float32(0.000001)
    p.tin_scale = float(diff / np.float32(255.0))
    p.tin_z = float(-np.float32(mn) * np.float32(in_scale) * np.float32(255.0) / diff)
    twq, tscale, tshift = ol.wino_prepare(p, ol.weights_to_blocked(w))
    tout, _ = ol.wino_gemm(p, ol.wino_trans_input(p, xin), twq, tscale, tshift)
    exp = from_blocked(ol.wino_trans_output(p, tout, bias), oc)
    fin, fout = tmp_path / "in.bin", tmp_path / "out.bin"
    with open(fin, "wb") as f:
        f.write(np.ascontiguousarray(xuser).tobytes())
        f.write(w.tobytes())
        f.write(bias[:oc].tobytes())
    E = pkg()
    args = [CHECK, str(fin), str(fout)] + [str(v) for v in (
        n, ic, oc, hw, 3, 1, 1, out_type, E.CONV_WINOGRAD, 0, 0, repr(float(out_scale)), 0.0, 1, 0,
        in_type, tile, hex(mode), repr(float(np.float32(p.tin_scale))), repr(float(np.float32(p.tin_z))))]
    r = subprocess.run(args, capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, "rc=%d stdout=%s stderr=%s" % (r.returncode, r.stdout, r.stderr)
    got = np.fromfile(fout, dtype=exp.dtype).reshape(exp.shape)
    assert np.array_equal(got.view(np.uint8), exp.view(np.uint8)), "%d values differ" % int((got != exp).sum())
    if out_type == ol.S8:
        assert len(np.unique(got)) > 40
