"""Oracle restatement of SaturateDepth, DenormalizePixel, SaturateDenormalizePixel, Saturate, SaturateFloat
(reference color_conversion.h:96-148, saturate.h:38-64) and of the transposed tensor forms TensorTSplit / TensorTPack /
CircularTensor<..., ColorPlanes::Transposed> (memory_operations.h:214-241, 292-327, circular_tensor.h:84-168), held
against: the values of the reference's own unit tests (utests/algorithm/image_processing/utest_color_conversion.h:248-297),
what the operations mean (written out with numpy, without the oracle's expressions), and the reference's CPU backend
running the same chain text (tests/cases/color_chains.h, circular_chains.h)."""
import numpy as np
import pytest

import oracle_lib as ol

needs_ref = pytest.mark.skipif(not ol.have_ref(), reason="reference CPU backend (oracle/_ref) not built here")

SPECIAL = np.array([np.nan, -np.inf, np.inf, -0.0, 0.0, 1.0, 255.0, 256.0, -1e-30, 1e-45, 0.5, 0.99999994, 1.0000001,
                    1023.0, 1023.5, 4095.0, -3.0, 2.0], np.float32)


def float_image(which, h, w, seed):
    """Inputs that make sense for operation `which`: anything for the saturating ones, [0, 1] for the plain casts."""
    cn = ol.DEPTH_OPS[which][0]
    r = np.random.default_rng(seed)
    shape = (h, w, cn) if cn > 1 else (h, w)
    if which in (2, 3, 8):                                  # DenormalizePixel: product must fit the output type
        a = r.random(shape, dtype=np.float32)
        a.reshape(-1)[:4] = [0.0, 1.0, 0.5, 0.25]
        return a
    a = (r.random(shape, dtype=np.float32) * 3.0 - 1.0).astype(np.float32)
    if which in (0, 1, 7):
        a *= 700.0
    flat = a.reshape(-1)
    flat[: SPECIAL.size] = SPECIAL
    return a


def test_values_of_the_reference_unit_tests():
    # utest_color_conversion.h:248-264
    src = np.array([[[0.0, 0.5, 1.0], [0.25, 0.75, 0.9]]], np.float32)
    assert ol.oracle_depth_ops(3, src).tolist() == [[[0.0, 127.5, 255.0], [63.75, 191.25, 229.5]]]
    # utest_color_conversion.h:282-297.  The second pixel is the test's own; for the first, that file expects {0, 128, 255}
    # while the operation it tests is a C cast of 0.5 * 255 = 127.5, which is 127 (the reference's CPU backend agrees:
    # test_depth_operations_match_reference_backend below runs this very input).
    src = np.array([[[-0.5, 0.5, 1.5], [0.25, 0.75, 0.9]]], np.float32)
    assert ol.oracle_depth_ops(4, src).tolist() == [[[0, 127, 255], [63, 191, 229]]]


@pytest.mark.parametrize("which", sorted(ol.DEPTH_OPS))
def test_depth_operations_are_what_they_mean(which):
    src = float_image(which, 7, 13, which)
    got = ol.oracle_depth_ops(which, src, -2.5, 9.25)
    with np.errstate(invalid="ignore"):
        if which in (0, 1, 7):
            lo, hi = {0: (0.0, 255.0), 1: (0.0, 1023.0), 7: (-2.5, 9.25)}[which]
            want = np.where(np.isnan(src), src, np.clip(src, np.float32(lo), np.float32(hi)))
            assert np.array_equal(got, want, equal_nan=True)
            return
        # NaN -> 1; below zero -> +0; above one -> 1; everything else (-0 included) as it is
        unit = np.where(np.isnan(src), np.float32(1.0), np.where(src < 0, np.float32(0.0), np.where(src > 1, np.float32(1.0), src)))
        if which == 6:
            assert got.tobytes() == unit.astype(np.float32).tobytes()
            return
        scale = {2: 255, 3: 255, 4: 255, 5: 1023, 8: 4095, 9: 255}[which]
        v = (src if which in (2, 3, 8) else unit).astype(np.float32) * np.float32(scale)
        want = v if which == 3 else np.trunc(v).astype(got.dtype)
        assert np.array_equal(got, want)


@needs_ref
@pytest.mark.parametrize("which", sorted(ol.DEPTH_OPS))
def test_depth_operations_match_reference_backend(which):
    for seed, (h, w) in enumerate([(5, 9), (16, 33)]):
        src = float_image(which, h, w, 10 * which + seed)
        assert ol.oracle_depth_ops(which, src, -2.5, 9.25).tobytes() == ol.ref_depth_ops(which, src, -2.5, 9.25).tobytes(), (which, h, w)
    if which == 4:
        src = np.array([[[-0.5, 0.5, 1.5], [0.25, 0.75, 0.9]]], np.float32)
        assert ol.ref_depth_ops(4, src).tolist() == [[[0, 127, 255], [63, 191, 229]]]


def images(n, w, h, seed):
    r = np.random.default_rng(seed)
    return [r.integers(0, 256, (h, w, 3), dtype=np.uint8) for _ in range(n)]


def test_transposed_tensor_layout():
    imgs = images(3, 10, 6, 1)
    tensor_t, packed = ol.oracle_transposed_round_trip(imgs, 0.5, 3.0)
    for z, img in enumerate(imgs):
        for c in range(3):
            assert np.array_equal(tensor_t[c, z], img[:, :, c].astype(np.float32) * np.float32(0.5))      # channel planes outermost
        assert np.array_equal(packed[z], img.astype(np.float32) * np.float32(0.5) * np.float32(3.0))


@needs_ref
@pytest.mark.parametrize("planes,w,h", [(1, 8, 4), (3, 10, 6), (4, 33, 5)])
def test_transposed_tensor_matches_reference_backend(planes, w, h):
    imgs = images(planes, w, h, planes)
    a = ol.oracle_transposed_round_trip(imgs, 1.25, 0.75)
    b = ol.ref_transposed_round_trip(imgs, 1.25, 0.75)
    assert a[0].tobytes() == b[0].tobytes() and a[1].tobytes() == b[1].tobytes()


@needs_ref
@pytest.mark.parametrize("batch", [2, 3, 5])
@pytest.mark.parametrize("oldest_first", [False, True])
def test_transposed_window_matches_reference_backend(batch, oldest_first):
    # the window's logical content does not depend on where its channel planes lie: the restatement of the standard
    # window (OracleWindow) is the expectation, the chain gathers the transposed window into the same order
    imgs = images(batch + 4, 11, 6, 60 + batch)
    a = ol.oracle_circular(batch, oldest_first, imgs, 10.0)
    b = ol.ref_circular_transposed(batch, oldest_first, imgs, 10.0)
    defined = ~np.isnan(a)
    assert defined.any() and np.array_equal(a[defined], b[defined])
    assert defined[batch - 1:].all()
