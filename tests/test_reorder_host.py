"""The host-side reorder<T, dst, src> constructors of the C++ API (include/euler_reorder.hpp, the
counterparts of src/elx_reorder.cpp:11-232): all twelve format pairs, for float and uint8_t, against
numpy transposes -- including channel tails that do not fill a 16-block, tensors large enough to be
split over several host threads, and the round trip through the blocked formats."""
import ctypes
import os

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "deep-learning-math-kernel-research_amd", "build", "libreorder_check.so")

(NCHW_FROM_NHWC, NHWC_FROM_NCHW, NCHW_FROM_BLOCKED, BLOCKED_FROM_NCHW, WBLOCKED_FROM_OIHW, OIHW_FROM_WBLOCKED,
 GWBLOCKED_FROM_GOIHW, GOIHW_FROM_GWBLOCKED, OIHW_FROM_HWIO, HWIO_FROM_OIHW, GOIHW_FROM_GHWIO, GHWIO_FROM_GOIHW) = range(12)


@pytest.fixture(scope="module")
def lib():
    assert os.path.exists(LIB), "libreorder_check.so is not built (python -c 'import __graft_entry__ as g; g.build()')"
    l = ctypes.CDLL(LIB)
    l.reorder_check.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p] + [ctypes.c_int] * 5
    return l


def up16(x):
    return (x + 15) // 16 * 16


def run(lib, which, src, dst_shape, g, a, b, h, w):
    src = np.ascontiguousarray(src)
    fill = 0x5a if src.dtype == np.uint8 else -77.0   # a stale destination must be fully overwritten
    dst = np.full(dst_shape, fill, src.dtype)
    rc = lib.reorder_check(which, int(src.dtype == np.uint8), dst.ctypes.data, src.ctypes.data, g, a, b, h, w)
    assert rc == 0
    return dst


def data(rng, shape, dtype):
    if dtype == np.uint8:
        return rng.integers(0, 256, shape).astype(np.uint8)
    return rng.normal(0, 1, shape).astype(np.float32)


def blocked_act(x):
    n, c, h, w = x.shape
    xp = np.zeros((n, up16(c), h, w), x.dtype)
    xp[:, :c] = x
    return np.ascontiguousarray(xp.reshape(n, up16(c) // 16, 16, h, w).transpose(0, 1, 3, 4, 2))


def blocked_weights(wt):
    g, o, i, h, w = wt.shape
    wp = np.zeros((g, up16(o), up16(i), h, w), wt.dtype)
    wp[:, :o, :i] = wt
    return np.ascontiguousarray(wp.reshape(g, up16(o) // 16, 16, up16(i) // 16, 16, h, w).transpose(0, 1, 3, 5, 6, 4, 2))


# small, channel tails, and one large enough (> 32768 elements per thread) to be split over threads
ACT_SHAPES = [(1, 16, 3, 3), (2, 3, 5, 4), (3, 40, 7, 6), (2, 17, 1, 9), (8, 144, 28, 28)]
W_SHAPES = [(1, 16, 16, 1, 1), (1, 24, 40, 3, 3), (1, 3, 7, 7, 7), (1, 33, 16, 1, 1), (1, 256, 272, 3, 3)]
GW_SHAPES = [(2, 16, 16, 1, 1), (3, 24, 8, 3, 3), (32, 1, 1, 3, 3), (4, 48, 80, 3, 3)]


@pytest.mark.parametrize("dtype", [np.float32, np.uint8], ids=["float", "uint8"])
@pytest.mark.parametrize("shape", ACT_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_activation_reorders(lib, dtype, shape):
    n, c, h, w = shape
    rng = np.random.default_rng(sum(shape))
    x = data(rng, shape, dtype)
    nhwc = np.ascontiguousarray(x.transpose(0, 2, 3, 1))
    assert np.array_equal(run(lib, NHWC_FROM_NCHW, x, nhwc.shape, 1, n, c, h, w), nhwc)
    assert np.array_equal(run(lib, NCHW_FROM_NHWC, nhwc, x.shape, 1, n, c, h, w), x)
    xb = blocked_act(x)
    got = run(lib, BLOCKED_FROM_NCHW, x, xb.shape, 1, n, c, h, w)
    assert np.array_equal(got, xb), "nChw16c: the channel tail must be zero-filled"
    # on the way back the tail is dropped: poison it to show it is never read into the result
    xb_poisoned = xb.copy()
    if c % 16:
        xb_poisoned[:, -1, :, :, c % 16:] = 99
    assert np.array_equal(run(lib, NCHW_FROM_BLOCKED, xb_poisoned, x.shape, 1, n, c, h, w), x)


@pytest.mark.parametrize("dtype", [np.float32, np.uint8], ids=["float", "uint8"])
@pytest.mark.parametrize("shape", W_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_weight_reorders(lib, dtype, shape):
    _, o, i, h, w = shape
    rng = np.random.default_rng(sum(shape) + 1)
    wt = data(rng, shape, dtype)
    wb = blocked_weights(wt)
    assert np.array_equal(run(lib, WBLOCKED_FROM_OIHW, wt[0], wb[0].shape, 1, o, i, h, w), wb[0])
    assert np.array_equal(run(lib, OIHW_FROM_WBLOCKED, wb[0], wt[0].shape, 1, o, i, h, w), wt[0])
    hwio = np.ascontiguousarray(wt[0].transpose(2, 3, 1, 0))
    assert np.array_equal(run(lib, HWIO_FROM_OIHW, wt[0], hwio.shape, 1, o, i, h, w), hwio)
    assert np.array_equal(run(lib, OIHW_FROM_HWIO, hwio, wt[0].shape, 1, o, i, h, w), wt[0])


@pytest.mark.parametrize("dtype", [np.float32, np.uint8], ids=["float", "uint8"])
@pytest.mark.parametrize("shape", GW_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_grouped_weight_reorders(lib, dtype, shape):
    g, o, i, h, w = shape
    rng = np.random.default_rng(sum(shape) + 2)
    wt = data(rng, shape, dtype)
    wb = blocked_weights(wt)
    assert np.array_equal(run(lib, GWBLOCKED_FROM_GOIHW, wt, wb.shape, g, o, i, h, w), wb)
    assert np.array_equal(run(lib, GOIHW_FROM_GWBLOCKED, wb, wt.shape, g, o, i, h, w), wt)
    ghwio = np.ascontiguousarray(wt.transpose(0, 3, 4, 2, 1))
    assert np.array_equal(run(lib, GHWIO_FROM_GOIHW, wt, ghwio.shape, g, o, i, h, w), ghwio)
    assert np.array_equal(run(lib, GOIHW_FROM_GHWIO, ghwio, wt.shape, g, o, i, h, w), wt)


def test_thread_count_does_not_change_the_result(lib, monkeypatch):
    """the reorders split their outer loop over host threads (OMP_NUM_THREADS caps the count)"""
    n, c, h, w = 4, 100, 30, 30
    x = data(np.random.default_rng(5), (n, c, h, w), np.float32)
    outs = []
    for threads in ("1", "3", "8"):
        monkeypatch.setenv("OMP_NUM_THREADS", threads)
        outs.append(run(lib, BLOCKED_FROM_NCHW, x, blocked_act(x).shape, 1, n, c, h, w))
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2])
    assert np.array_equal(outs[0], blocked_act(x))
