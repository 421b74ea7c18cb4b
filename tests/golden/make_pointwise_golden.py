"""Writes tests/golden/pointwise_reference_vectors.npz: the outputs of the REFERENCE library's CPU backend
(oracle/_ref/libfkl_ref.so) for every chain of tests/cases/pointwise_chains.h (per-channel Operations, two-image chains, SplitWrite) on small seeded
inputs (tests/pointwise_cases.py, tests/test_oracle_pointwise.py).  Data only; run in the build container:  python tests/golden/make_pointwise_golden.py"""
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
    # the two-image chains and the SplitWrite chains of the same header
    import test_oracle_pointwise as t
    for which in sorted(po.DUAL_CASES):
        a, b = pc.dual_inputs(which, po.DUAL_CASES, 6, 11, 0)
        out[f"dual_a_{which}"], out[f"dual_b_{which}"] = a, b
        out[f"dual_out_{which}"] = ol.ref_dual(which, a, b)
    for which in sorted(ol.SPLIT_WRITE_CASES):
        src = t._split_input(which, 24, 40, 0)
        out[f"split_in_{which}"] = src
        for k, plane in enumerate(ol.ref_split_write(which, src, (29, 17) if which == 3 else None, (0.5, -2.0, 3.25, 0))):
            out[f"split_out_{which}_{k}"] = plane
    np.savez_compressed(os.path.join(HERE, "pointwise_reference_vectors.npz"), **out)
    print("wrote", len(out), "arrays")


if __name__ == "__main__":
    main()
