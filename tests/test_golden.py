"""The CPU oracle against the committed golden vectors (tests/golden/*.npz: outputs of the
reference's own micro-kernel templates, compiled from its sources by tests/golden/make_golden.py).
Needs neither the reference tree nor its build, so it also pins the oracle on the GPU box."""
import glob
import os
import sys

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))
import cases  # noqa: E402

FILES = sorted(glob.glob(os.path.join(HERE, "golden", "*.npz")))


def test_every_case_has_a_fixture():
    have = {os.path.basename(f)[:-4] for f in FILES}
    assert have == set(cases.CASES), (sorted(set(cases.CASES) - have), sorted(have - set(cases.CASES)))


@pytest.mark.parametrize("path", FILES, ids=lambda p: os.path.basename(p)[:-4])
def test_oracle_matches_golden(path):
    name = os.path.basename(path)[:-4]
    with np.load(path, allow_pickle=False) as z:
        d = {k: z[k] for k in z.files}
    expected = d.pop("expected")
    got = cases.CASES[name][2](d)
    assert got.shape == expected.shape and got.dtype == expected.dtype
    assert np.array_equal(np.ascontiguousarray(got).view(np.uint8), np.ascontiguousarray(expected).view(np.uint8))
    # the stored inputs are the seeded ones (guards against fixtures and generator drifting apart)
    fresh = cases.CASES[name][0]()
    for k, v in fresh.items():
        assert np.array_equal(np.asarray(v), d[k]), k


@pytest.mark.parametrize("A", [6, 4, 5])
def test_tie_fixtures_tell_the_fused_quantization_from_the_unfused(A):
    """wino_glue_input*_ties: every injected value reaches position (A-1, A-1) of its tile unchanged, and the
    stored code of the reference's compiled transform is the one of fma(v, mrepS, mz) -- never that of
    (v * mrepS) + mz, which these values were searched to separate."""
    path = os.path.join(HERE, "golden", "wino_glue_input%d_ties.npz" % A)
    with np.load(path, allow_pickle=False) as z:
        d = {k: z[k] for k in z.files}
    f32, L = np.float32, np.longdouble
    M, hw = A - 2, int(d["hw"])
    wt = (hw + M - 1) // M
    m = f32(1.0) * (f32(1.0) / f32(d["tin_scale"]))
    mz = f32(np.ceil(d["tin_z"]))
    x = d["x"].transpose(0, 1, 4, 2, 3).reshape(1, 16, hw, hw)
    sites = 0
    for h, w in cases.glue_ties_sites(A, hw):
        t = ((h + 1 - (A - 1)) // M) * wt + (w + 1 - (A - 1)) // M
        for c in range(16):
            v = x[0, c, h, w]
            if v == 0:
                continue
            fused = int(np.clip(np.rint((L(v) * L(m) + L(mz)).astype(f32)), 0, 255))
            unfused = int(np.clip(np.rint(f32(v * m) + mz), 0, 255))
            assert fused != unfused
            assert int(d["expected"][A * A - 1, 0, t, c]) == fused
            sites += 1
    assert sites >= 32
