"""The oracle on the seeded random cases of tests/random_cases.py: equal, bit for bit, to the digests the reference CPU
backend gave (tests/golden/random_batches_reference_digests.json) and, where the reference backend is built, to its
live output."""
import json
import os

import numpy as np
import pytest

import oracle_lib as ol
import random_cases as rc

with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "random_batches_reference_digests.json")) as f:
    REFERENCE = json.load(f)


def _check(key, want, live):
    assert rc.digest(want) == REFERENCE[key], key
    if ol.have_ref():
        got = live()
        assert got.tobytes() == want.tobytes(), key


@pytest.mark.parametrize("seed,batch,size,pad,least,dst", rc.NORMALISE)
def test_oracle_on_random_batches(seed, batch, size, pad, least, dst):
    backing, rects, sub, div = rc.normalise_inputs(seed, batch, size, pad, least)
    img = rc.image_of(backing, size[0])
    want = ol.oracle_crop_resize_norm_split(np.ascontiguousarray(img), rects, dst, sub, div)
    _check(f"normalise:{seed}", want, lambda: ol.ref_crop_resize_norm_split(img, rects, dst, sub, div))


@pytest.mark.parametrize("seed,size,pad,dst", rc.LETTERBOX)
def test_oracle_on_random_letterboxed_batches(seed, size, pad, dst):
    backing, rects, bg, mul, sub = rc.letterbox_inputs(seed, size, pad)
    img = rc.image_of(backing, size[0])
    want = ol.oracle_crop_resize_par_u8(np.ascontiguousarray(img), rects, dst, bg, mul, sub)
    _check(f"letterbox:{seed}", want, lambda: ol.ref_crop_resize_par_u8(img, rects, dst, bg, mul, sub))


@pytest.mark.parametrize("seed,size,pad,dst", rc.FRAMES)
def test_oracle_on_random_nv12_frames(seed, size, pad, dst):
    backing, scale = rc.frame_inputs(seed, size, pad)
    w, h = size
    want = ol.oracle_nv12_rgb_resize_split(np.ascontiguousarray(backing[:, :w]), w, h, dst, scale)
    _check(f"frame:{seed}", want, lambda: ol.ref_nv12_rgb_resize_split(backing[:, :w], w, h, dst, scale))


def test_every_case_has_a_reference_digest():
    keys = {f"normalise:{c[0]}" for c in rc.NORMALISE} | {f"letterbox:{c[0]}" for c in rc.LETTERBOX} | {f"frame:{c[0]}" for c in rc.FRAMES}
    assert keys == set(REFERENCE)


def test_oracle_equals_the_reference_backend_on_the_sweep():
    # the 1 500 cases of the sweep the GPU test runs, against the live reference CPU backend
    if not ol.have_ref():
        pytest.skip("the reference CPU backend is not built here")
    for i in range(1500):
        family, c = rc.sweep_case(i)
        backing, w, dst = c["backing"], c["w"], c["dst"]
        if family == 0:
            img = rc.image_of(backing, w)
            want = ol.oracle_crop_resize_norm_split(np.ascontiguousarray(img), c["rects"], dst, c["sub"], c["div"])
            got = ol.ref_crop_resize_norm_split(img, c["rects"], dst, c["sub"], c["div"])
        elif family == 1:
            img = rc.image_of(backing, w)
            want = ol.oracle_crop_resize_par_u8(np.ascontiguousarray(img), c["rects"], dst, c["bg"], c["mul"], c["sub"])
            got = ol.ref_crop_resize_par_u8(img, c["rects"], dst, c["bg"], c["mul"], c["sub"])
        else:
            want = ol.oracle_nv12_rgb_resize_split(np.ascontiguousarray(backing[:, :w]), w, c["h"], dst, c["scale"])
            got = ol.ref_nv12_rgb_resize_split(backing[:, :w], w, c["h"], dst, c["scale"])
        assert got.tobytes() == want.tobytes(), f"case {i} (family {family})"


def test_oracle_equals_the_reference_backend_on_the_reader_sweep():
    # the cases of the reader sweep the GPU test runs that the reference harness has a chain for (uchar3 Warping and
    # Deinterlace, BorderReader of both element types), against the live reference CPU backend
    if not ol.have_ref():
        pytest.skip("the reference CPU backend is not built here")
    borders = [ol.BORDER_CONSTANT, ol.BORDER_REPLICATE, ol.BORDER_REFLECT, ol.BORDER_WRAP, ol.BORDER_REFLECT_101]
    for i in range(1000):
        family, c = rc.reader_sweep_case(i)
        img = c["img"]
        if family == 0:
            want = ol.oracle_warp(img, 3, c["matrix"], c["dst"], c["perspective"])
            got = ol.ref_warp_u8x3(img, c["matrix"], c["dst"], c["perspective"])
        elif family == 2:
            want = ol.oracle_deinterlace(img, 3, c["mode"])
            got = ol.ref_deinterlace_u8x3(img, c["mode"])
            if c["mode"] == ol.DEINTERLACE_LINEAR_ODD and img.shape[0] % 2:
                # outside the reference's domain: its last line reads past the image (here it is defined as the last line)
                want, got = want[:-1], got[:-1]
        elif family == 3:
            want = ol.oracle_pad(img, borders[c["border"]], c["left"], c["top"], c["out_w"], c["out_h"], value=c["value"])
            got = ol.ref_pad(img, borders[c["border"]], c["left"], c["top"], c["out_w"], c["out_h"], value=c["value"])
        else:
            continue
        assert got.tobytes() == want.tobytes(), f"case {i} (family {family})"


def test_oracle_equals_the_reference_backend_on_the_chain_sweep():
    # the 1 200 cases of the chain sweep the GPU test runs, against the live reference CPU backend
    if not ol.have_ref():
        pytest.skip("the reference CPU backend is not built here")
    for i in range(1200):
        family, c = rc.chain_sweep_case(i)
        if family == 0:
            src = c["src"][:, :c["w"]]
            same = ol.oracle_add_mul_chain(np.ascontiguousarray(src), c["n"], 0.5, 1.0001).tobytes() == \
                ol.ref_add_mul_chain(src, c["n"], 0.5, 1.0001, c["tf"]).tobytes()
        elif family == 1:
            imgs = [rc.image_of(b, c["w"]) for b in c["backings"]]
            want = ol.oracle_batch_muladd_sat([np.ascontiguousarray(x) for x in imgs], c["mul"], c["add"])
            same = np.stack(ol.ref_batch_muladd_sat(imgs, c["mul"], c["add"])).tobytes() == np.stack(want).tobytes()
        elif family == 2:
            args = (c["img"], c["rects"], c["dst"], c["used"], c["default"], c["sub"], c["div"])
            same = ol.oracle_crop_resize_default_norm_split(*args).tobytes() == ol.ref_crop_resize_default_norm_split(*args).tobytes()
        else:
            args = (c["imgs"], c["active"], (7, 200, 33), (0.5, 2.0, 1.25))
            same = ol.oracle_batch_default_cast_mul(*args).tobytes() == ol.ref_batch_default_cast_mul(*args).tobytes()
        assert same, f"case {i} (family {family})"
