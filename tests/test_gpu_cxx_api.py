"""The C++ surface (include/euler.hpp: eld_conv_t::setup + elx_conv on host buffers, reorder<>) end
to end: a prebuilt client program (tests/cxx/euler_api_check.cpp, compiled by build()) runs a layer
the way a program written against the reference does; its output is compared bit for bit with the
CPU oracle."""
import os
import subprocess

import numpy as np
import pytest

import oracle_lib as ol
from gpu_common import Layer

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CHECK = os.path.join(ROOT, "deep-learning-math-kernel-research_amd", "build", "euler_api_check")


def from_blocked(b, c):
    n, c2, h, w, _ = b.shape
    return np.ascontiguousarray(b.transpose(0, 1, 4, 2, 3).reshape(n, c2 * 16, h, w)[:, :c])


@pytest.mark.parametrize("case", [
    dict(n=2, ic=64, oc=48, hw=12, k=3, pad=1, out_type=ol.U8, T=12),
    dict(n=2, ic=96, oc=64, hw=7, k=1, pad=0, out_type=ol.S8, with_sum=True),
    dict(n=1, ic=32, oc=80, hw=9, k=1, pad=0, out_type=ol.F32),
    dict(n=2, ic=32, oc=32, hw=14, k=3, pad=1, out_type=ol.U8, depthwise=True, T=7),
    dict(n=2, ic=64, oc=64, hw=14, k=3, pad=1, stride=2, out_type=ol.S8, T=7),
    dict(n=2, ic=32, oc=32, hw=14, k=3, pad=1, stride=2, out_type=ol.U8, depthwise=True, T=7),
    dict(n=2, ic=96, oc=64, hw=7, k=1, pad=0, out_type=ol.S8, with_sum=True, nhwc=True),
    dict(n=2, ic=3, oc=64, hw=22, k=7, pad=3, stride=2, out_type=ol.S8, nhwc=True),   # a first layer: 3-channel nhwc image
], ids=["3x3_u8", "1x1_s8_sum", "1x1_f32", "depthwise_u8", "3x3_s2_s8", "depthwise_s2_u8", "1x1_s8_sum_nhwc",
        "7x7_s2_3ch_nhwc"])
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
