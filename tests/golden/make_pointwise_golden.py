"""Writes tests/golden/pointwise_reference_vectors.npz: the outputs of the REFERENCE library's CPU backend
(oracle/_ref/libfkl_ref.so) for every chain of tests/cases/pointwise_chains.h on the seeded 5 x 9 inputs of
tests/pointwise_cases.py.  Data only; run in the build container:  python tests/golden/make_pointwise_golden.py"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(HERE)), "tests"))

import oracle_lib as ol  # noqa: E402
import pointwise_cases as pc  # noqa: E402


def main():
    assert ol.have_ref(), "build oracle/_ref first (make -C oracle ref)"
    po = ol.pointwise_oracle()
    out = {}
    for which in sorted(po.CASES):
        src = pc.inputs(which, po.CASES, 5, 9, 0)
        out[f"in_{which}"] = src
        out[f"out_{which}"] = ol.ref_pointwise(which, src, pc.constants(which), pc.MATRIX)
    np.savez_compressed(os.path.join(HERE, "pointwise_reference_vectors.npz"), **out)
    print("wrote", len(out), "arrays")


if __name__ == "__main__":
    main()
