"""Writes tests/golden/resize_geometry_reference_vectors.json: target rectangle and source conversion factors the
REFERENCE library computes (Resize<INTER_LINEAR, AR>::build on its CPU side, oracle/_ref/libfkl_ref.so) for the
aspect-ratio modes PRESERVE_AR, PRESERVE_AR_RN_EVEN and PRESERVE_AR_LEFT on a list of source and destination sizes.
Data only; run in the build container:  python tests/golden/make_resize_geometry_golden.py"""
import ctypes as C
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(HERE)), "tests"))

import oracle_lib as ol  # noqa: E402

SIZES = [((60, 40), (128, 64)), ((130, 140), (128, 64)), ((100, 35), (128, 64)), ((40, 15), (128, 64)), ((1920, 1080), (128, 64)),
         ((7, 300), (128, 64)), ((300, 7), (128, 64)), ((333, 111), (224, 224)), ((111, 333), (224, 224)), ((1920, 1080), (640, 640)),
         ((1279, 719), (416, 416)), ((50, 50), (63, 63)), ((3, 2), (5, 5)), ((101, 67), (97, 33)), ((67, 101), (33, 97))]


def main():
    assert ol.have_ref(), "build oracle/_ref first (make -C oracle ref)"
    out = {}
    for ar in (0, 2, 3):
        for (sw, sh), (dw, dh) in SIZES:
            o4 = (C.c_int32 * 4)()
            f2 = (C.c_float * 2)()
            assert ol.ref().fklref_resize_params_ar(ar, sw, sh, dw, dh, o4, f2) == 0
            out[f"{ar}:{sw}x{sh}->{dw}x{dh}"] = {"rect": list(o4), "fx": float(np.float32(f2[0])), "fy": float(np.float32(f2[1]))}
    with open(os.path.join(HERE, "resize_geometry_reference_vectors.json"), "w") as f:
        json.dump(out, f, indent=0, sort_keys=True)
    print("wrote", len(out), "entries")


if __name__ == "__main__":
    main()
