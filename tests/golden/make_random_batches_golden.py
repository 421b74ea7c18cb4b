"""Writes tests/golden/random_batches_reference_digests.json: SHA-256 of what the REFERENCE library's CPU backend
(oracle/_ref/libfkl_ref.so, built from the reference's headers by oracle/Makefile) returns for the seeded random cases of
tests/random_cases.py.  Data only; run in the build container:  python tests/golden/make_random_batches_golden.py"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))

import oracle_lib as ol  # noqa: E402
import random_cases as rc  # noqa: E402


def reference_outputs():
    for seed, batch, size, pad, least, dst in rc.NORMALISE:
        backing, rects, sub, div = rc.normalise_inputs(seed, batch, size, pad, least)
        yield f"normalise:{seed}", ol.ref_crop_resize_norm_split(rc.image_of(backing, size[0]), rects, dst, sub, div)
    for seed, size, pad, dst in rc.LETTERBOX:
        backing, rects, bg, mul, sub = rc.letterbox_inputs(seed, size, pad)
        yield f"letterbox:{seed}", ol.ref_crop_resize_par_u8(rc.image_of(backing, size[0]), rects, dst, bg, mul, sub)
    for seed, size, pad, dst in rc.FRAMES:
        backing, scale = rc.frame_inputs(seed, size, pad)
        yield f"frame:{seed}", ol.ref_nv12_rgb_resize_split(backing[:, :size[0]], size[0], size[1], dst, scale)


def main():
    assert ol.have_ref(), "build oracle/_ref first (make -C oracle ref)"
    out = {key: rc.digest(value) for key, value in reference_outputs()}
    with open(os.path.join(HERE, "random_batches_reference_digests.json"), "w") as f:
        json.dump(out, f, indent=0, sort_keys=True)
    print("wrote", len(out), "digests")


if __name__ == "__main__":
    main()
