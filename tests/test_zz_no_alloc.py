"""The allocation-free entry point ehip_wino_tinput_range_noalloc against ehip_wino_tinput_range.

It keeps its partial results in a static device array of the library instead of in memory from
hipMalloc, leaves the result in device memory and synchronises nothing.  Both entry points must give
the same two floats, bit for bit, on calls in a row that share the array: the second call has a smaller
input (fewer channels, fewer tiles, a narrower range), so anything left over from the first would show."""
import ctypes

import numpy as np
import pytest

import oracle_lib as ol
from gpu_common import dev, pkg

pytestmark = pytest.mark.gpu
f32 = np.float32


def _case(E, n, ic, hw, seed, lo, hi, tile=6, u8=False):
    rng = np.random.default_rng(seed)
    x = rng.uniform(lo, hi, (n, ic, hw, hw)).astype(f32)
    if u8:
        x = np.rint(x).astype(np.uint8)
    xb = ol.to_blocked(x)
    d = E.make_desc(n, ic, 32, hw, hw, 3, 3, 1, algorithm=E.CONV_WINOGRAD, input_type=E.U8 if u8 else E.F32,
                    output_type=E.F32, input_quant=(1.0, 0.0), tile_size=tile, execution_mode=0xa161,
                    wino_tinput_quant=(1.0, 0.0))
    p = ol.make_params(n, ic, 32, hw, hw, 3, 3, 1, out_type=ol.F32, in_scale=1.0, wino_tile=tile)
    return d, p, xb


def test_range_without_allocation_matches_the_allocating_entry_point():
    import torch
    E = pkg()
    assert E.lib.ehip_init(0) == 0, E.lib.ehip_last_error()
    out = torch.full((2,), -1.0, dtype=torch.float32, device="cuda")
    # first call: the larger input with the wider range; second call: smaller in every respect
    cases = [_case(E, 3, 80, 20, 11, -4.0, 9.0), _case(E, 1, 24, 9, 12, 0.25, 0.75),
             _case(E, 2, 48, 13, 13, 0.0, 255.0, tile=4, u8=True), _case(E, 1, 16, 7, 14, 10.0, 20.0, tile=5, u8=True)]
    for d, p, xb in cases:
        d_x = dev(xb)
        E.wino_tinput_range_noalloc(d, d_x, out)
        got = out.cpu().numpy().copy()
        mn, mx = E.wino_tinput_range(d, d_x)
        assert got.view(np.uint32).tolist() == np.array([mn, mx], f32).view(np.uint32).tolist()
        omn, omx = ol.wino_tinput_range(p, xb.astype(f32))
        assert (f32(got[0]), f32(got[1])) == (f32(omn), f32(omx))


def test_range_without_allocation_on_a_side_stream_and_in_a_row():
    """Calls queued back to back on one stream, no synchronisation in between: each re-initialises the
    part of the array it uses."""
    import torch
    E = pkg()
    s = torch.cuda.Stream()
    outs = [torch.zeros(2, dtype=torch.float32, device="cuda") for _ in range(3)]
    cases = [_case(E, 2, 64, 16, 21, -1.0, 1.0), _case(E, 1, 16, 8, 22, 0.0, 0.5), _case(E, 2, 32, 12, 23, -3.0, 0.0)]
    xs = [dev(c[2]) for c in cases]
    torch.cuda.synchronize()
    for (d, _, _), x, o in zip(cases, xs, outs):
        E.wino_tinput_range_noalloc(d, x, o, stream=s.cuda_stream)
    s.synchronize()
    for (d, p, xb), x, o in zip(cases, xs, outs):
        mn, mx = E.wino_tinput_range(d, x)
        assert o.cpu().numpy().view(np.uint32).tolist() == np.array([mn, mx], f32).view(np.uint32).tolist()


def test_range_without_allocation_rejects_what_the_array_cannot_hold():
    E = pkg()
    d = E.make_desc(1, 16 * 4097, 32, 6, 6, 3, 3, 1, algorithm=E.CONV_WINOGRAD, input_type=E.U8, output_type=E.F32,
                    input_quant=(1.0, 0.0), tile_size=6, wino_tinput_quant=(1.0, 0.0))
    rc = E.lib.ehip_wino_tinput_range_noalloc(ctypes.byref(d), ctypes.c_void_p(256), ctypes.c_void_p(256), None)
    assert rc == E.EHIP_UNIMPLEMENTED
    assert b"at most 65536 input channels" in E.lib.ehip_last_error()


def test_range_without_allocation_under_graph_capture_and_without_any_allocation():
    """What the entry point is for: a stream under HIP graph capture.  After ehip_init (which resolves the static
    array's address for the device) the call is captured -- three kernels, no memset node, no allocation -- and the
    graph replayed three times on changing inputs, with the program's own eager work between the replays; every
    replay must give what the allocating entry point gives for the same input.  Device memory in use (torch's
    allocator and the driver's free-memory figure) is the same before and after the call."""
    import torch
    E = pkg()
    assert E.lib.ehip_init(0) == 0, E.lib.ehip_last_error()
    d, p, xb = _case(E, 2, 64, 16, 31, -2.0, 5.0)
    x = dev(xb)
    out = torch.zeros(2, dtype=torch.float32, device="cuda")
    torch.cuda.synchronize()
    # no allocation: an eager call first
    before_t = torch.cuda.memory_allocated()
    free0, _ = torch.cuda.mem_get_info()
    E.wino_tinput_range_noalloc(d, x, out)
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert torch.cuda.memory_allocated() == before_t
    assert free1 == free0
    # captured
    s = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.graph(g, stream=s):
        E.wino_tinput_range_noalloc(d, x, out, stream=torch.cuda.current_stream().cuda_stream)
    rng = np.random.default_rng(32)
    for rep in range(3):
        # other inputs at the same address; eager work of the program's own and a synchronisation in between
        xb2 = ol.to_blocked(rng.uniform(-1.0 - rep, 2.0 + 3 * rep, (2, 64, 16, 16)).astype(f32))
        x.copy_(torch.from_numpy(xb2))
        out.fill_(-7.0)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        got = out.cpu().numpy().copy()
        mn, mx = E.wino_tinput_range(d, x)
        assert got.view(np.uint32).tolist() == np.array([mn, mx], f32).view(np.uint32).tolist(), rep
        omn, omx = ol.wino_tinput_range(p, xb2)
        assert (f32(got[0]), f32(got[1])) == (f32(omn), f32(omx))


def test_range_without_allocation_as_the_first_call_of_a_process():
    """No ehip_init, no other entry point before it: the first call resolves the static array's address itself."""
    import os
    import subprocess
    import sys
    code = r'''
import sys, numpy as np
sys.path.insert(0, %r); sys.path.insert(0, %r)
import torch
import oracle_lib as ol
from gpu_common import dev, pkg
E = pkg()
rng = np.random.default_rng(41)
xb = ol.to_blocked(rng.uniform(-3.0, 4.0, (2, 32, 12, 12)).astype(np.float32))
d = E.make_desc(2, 32, 32, 12, 12, 3, 3, 1, algorithm=E.CONV_WINOGRAD, input_type=E.F32, output_type=E.F32,
                input_quant=(1.0, 0.0), tile_size=6, execution_mode=0xa161, wino_tinput_quant=(1.0, 0.0))
out = torch.zeros(2, dtype=torch.float32, device="cuda")
E.wino_tinput_range_noalloc(d, dev(xb), out)       # the process's first call into the library
torch.cuda.synchronize()
p = ol.make_params(2, 32, 32, 12, 12, 3, 3, 1, out_type=ol.F32, in_scale=1.0, wino_tile=6)
omn, omx = ol.wino_tinput_range(p, xb)
got = out.cpu().numpy()
assert (np.float32(got[0]), np.float32(got[1])) == (np.float32(omn), np.float32(omx)), (got, omn, omx)
print("ok")
''' % (os.path.dirname(os.path.dirname(os.path.abspath(__file__))), os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "ok" in r.stdout, "rc=%d stdout=%s stderr=%s" % (r.returncode, r.stdout, r.stderr[-2000:])
