#!/usr/bin/env python3
"""Writes tests/golden/*.npz: seeded inputs plus the outputs of the reference's micro-kernel
templates compiled from /root/reference (oracle/Makefile target `ref`).  Run in the build
container only (needs oracle/_ref and an AVX-512-VNNI host):

    python tests/golden/make_golden.py [prefix]     (prefix: only the cases whose names start with it)

The harness_* cases hold tensors that the reference's harness draws itself (partly seeded from the clock), so
writing them again gives new fixtures rather than the same bytes.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, HERE)
import oracle_lib as ol  # noqa: E402
import cases  # noqa: E402


def main():
    ref = ol.ref_kernels()
    if ref is None:
        sys.exit("oracle/_ref is not built (make -C oracle ref) or the host lacks AVX-512-VNNI")
    prefix = sys.argv[1] if len(sys.argv) > 1 else ""
    for name, (make_inputs, run_reference, _) in sorted(cases.CASES.items()):
        if not name.startswith(prefix):
            continue
        d = make_inputs()
        out = run_reference(d, ref)
        np.savez_compressed(os.path.join(HERE, name + ".npz"), expected=out, **d)
        print("%-32s %8d bytes out" % (name, out.nbytes))


if __name__ == "__main__":
    main()
