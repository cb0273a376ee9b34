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
