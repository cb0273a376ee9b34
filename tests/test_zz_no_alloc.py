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
