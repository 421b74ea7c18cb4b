"""CPU tests that pin the oracle's BorderReader (reference border_reader.h:177-327): numpy.pad gives the textbook
result of each border type while the padding stays within one image size; the reference's CPU backend, running the
same chain text (tests/cases/border_chains.h), gives the result everywhere, including paddings several images wide,
where the reference's index arithmetic is its own."""
import numpy as np
import pytest

import oracle_lib as ol

needs_ref = pytest.mark.skipif(not ol.have_ref(), reason="reference CPU backend (oracle/_ref) not built here")
NUMPY_MODE = {ol.BORDER_CONSTANT: "constant", ol.BORDER_REPLICATE: "edge", ol.BORDER_REFLECT: "symmetric", ol.BORDER_WRAP: "wrap",
              ol.BORDER_REFLECT_101: "reflect"}


def images():
    r = np.random.default_rng(11)
    return [r.integers(0, 256, (9, 14, 3), dtype=np.uint8), (r.random((7, 5), dtype=np.float32) * 50 - 25).astype(np.float32),
            r.integers(0, 256, (6, 11, 4), dtype=np.uint8), r.integers(0, 1000, (8, 7, 3)).astype(np.uint16),
            r.integers(0, 256, (5, 9), dtype=np.uint8), (r.random((6, 8, 3), dtype=np.float32) * 50 - 25).astype(np.float32)]


@pytest.mark.parametrize("bt", sorted(NUMPY_MODE))
def test_padding_within_one_image_size_is_numpy_pad(bt):
    for img in images():
        h, w = img.shape[:2]
        for (left, top, right, bottom) in ((3, 2, 4, 1), (0, 0, 0, 0), (w - 1, h - 1, w - 1, h - 1), (0, 3, 2, 0)):
            pads = ((top, bottom), (left, right)) + (((0, 0),) if img.ndim == 3 else ())
            kw = {"constant_values": 7} if bt == ol.BORDER_CONSTANT else {}
            want = np.pad(img, pads, mode=NUMPY_MODE[bt], **kw)
            got = ol.oracle_pad(img, bt, left, top, w + left + right, h + top + bottom, value=(7, 7, 7, 7))
            assert got.tobytes() == want.tobytes(), (bt, left, top, right, bottom)


def test_a_crop_inside_the_image_is_untouched_by_any_border():
    img = images()[0]
    for bt in sorted(NUMPY_MODE):
        assert np.array_equal(ol.oracle_pad(img, bt, -2, -1, 6, 5), img[1:6, 2:8])


@needs_ref
@pytest.mark.parametrize("bt", sorted(NUMPY_MODE))
def test_padding_matches_reference_backend(bt):
    for img in images():
        h, w = img.shape[:2]
        for (left, top, ow, oh) in ((3, 2, w + 7, h + 3), (2 * w + 3, 3 * h + 1, 5 * w + 2, 7 * h), (-1, -2, 4, 3), (w, h, 3 * w, 3 * h)):
            a = ol.oracle_pad(img, bt, left, top, ow, oh, value=(9, 8, 7, 6))
            b = ol.ref_pad(img, bt, left, top, ow, oh, value=(9, 8, 7, 6))
            assert a.tobytes() == b.tobytes(), (bt, left, top, ow, oh)
