"""CPU tests that pin the colour part of the oracle (pixel-format readers/writers, YCbCr<->RGB for every depth, range
and set of primaries, gray, alpha, normalisation):

  * against the literal values the reference's own unit test holds (tests/golden/color_conversion_reference_vectors.json,
    transcribed from utests/algorithm/image_processing/utest_color_conversion.h),
  * against the reference's CPU backend compiled from its own headers (oracle/_ref), when that is built,
  * against what the mathematics fixes (neutral chroma gives gray, the two matrices are inverses, round trips).
"""
from __future__ import annotations

import json
import os

import numpy as np
import pytest

import oracle_lib as ol

GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "color_conversion_reference_vectors.json")))
needs_ref = pytest.mark.skipif(not ol.have_ref(), reason="reference CPU backend (oracle/_ref) not built here")

PRIMARIES = {"bt601": ol.CP_BT601, "bt709": ol.CP_BT709, "bt2020": ol.CP_BT2020}
RANGES = {"limited": ol.CR_LIMITED, "full": ol.CR_FULL}
LIMITS = {ol.CD_P10: (1023.0, 876.0, 896.0), ol.CD_P12: (4095.0, 3504.0, 3584.0)}


def rng(seed):
    return np.random.default_rng(seed)


def frame(pf, w, h, seed, pad=0):
    """Random frame in pixel format pf; 10-bit formats hold 10-bit values.  `pad` extra samples per row (pitch > width)."""
    rows, cols = ol.frame_shape(pf, w, h)
    if ol.PF_WIDE[pf]:
        a = rng(seed).integers(0, 1024, (rows, cols + pad), dtype=np.uint16)
    else:
        a = rng(seed).integers(0, 256, (rows, cols + pad), dtype=np.uint8)
    return a


# ---- matrices --------------------------------------------------------------------------------------------

def golden_matrix(cd, cr_name, cp_name, to_rgb):
    """The literal the reference's unit test expects, following its aliasing rules for the other depths."""
    direction = "to_rgb" if to_rgb else "to_yuv"
    base = cd % 3
    if cr_name == "full" or base == ol.CD_P8:
        return np.array(GOLDEN["matrices_p8bit"][cp_name][cr_name][direction], np.float32)
    full = np.array(GOLDEN["matrices_p8bit"][cp_name]["full"][direction], np.float32).reshape(3, 3)
    mx, ly, lc = (np.float32(v) for v in LIMITS[base])
    if to_rgb:
        f = np.array([mx / ly, mx / lc, mx / lc], np.float32)
        return (full * f[None, :]).astype(np.float32).ravel()
    f = np.array([ly / mx, lc / mx, lc / mx], np.float32)
    return (full * f[:, None]).astype(np.float32).ravel()


@pytest.mark.parametrize("cd", range(6))
def test_matrices_equal_the_reference_unit_test_literals(cd):
    for cp_name, cp in PRIMARIES.items():
        for cr_name, cr in RANGES.items():
            for to_rgb in (True, False):
                got = ol.oracle_color_matrix(cd, cr, cp, to_rgb)
                want = golden_matrix(cd, cr_name, cp_name, to_rgb)
                assert got.tobytes() == want.tobytes(), (cd, cr_name, cp_name, to_rgb, got, want)


@needs_ref
def test_matrices_equal_the_reference_constexpr_matrices():
    for cd in range(6):
        for cr in (0, 1):
            for cp in (0, 1, 2):
                for to_rgb in (True, False):
                    assert ol.oracle_color_matrix(cd, cr, cp, to_rgb).tobytes() == ol.ref_color_matrix(cd, cr, cp, to_rgb).tobytes(), (cd, cr, cp, to_rgb)


def test_the_two_directions_are_inverse_matrices():
    for cd in range(6):
        for cr in (0, 1):
            for cp in (0, 1, 2):
                a = ol.oracle_color_matrix(cd, cr, cp, True).astype(np.float64).reshape(3, 3)
                b = ol.oracle_color_matrix(cd, cr, cp, False).astype(np.float64).reshape(3, 3)
                assert np.allclose(a @ b, np.eye(3), atol=2e-6), (cd, cr, cp)


def test_depth_constants():
    mx, lu, ch = (ol.C.c_float(), ol.C.c_float(), ol.C.c_float())
    want = {0: (255, 16, 128), 1: (1023, 64, 512), 2: (4095, 256, 2048)}
    for cd in range(6):
        assert ol.oracle().fklo_depth_constants(cd, mx, lu, ch) == 0
        m, l, c = want[cd % 3]
        if cd < 3:
            assert (mx.value, lu.value, ch.value) == (m, l, c)
        else:
            assert mx.value == 1.0 and lu.value == np.float32(l) / np.float32(m) and ch.value == np.float32(c) / np.float32(m)


# ---- readers ---------------------------------------------------------------------------------------------

def _read_only(pf, buf, w, h):
    dt = np.uint16 if ol.PF_WIDE[pf] else np.uint8
    out = np.zeros((h, w, 3), dt)
    ol.execute([ol.read_yuv(pf, buf, w, h)], [], [ol.write(ol.WRITE_2D, out, 3, w, h)])
    return out


def test_uyvy_reader_on_the_reference_unit_test_vectors():
    for case in GOLDEN["uyvy"]:
        w, h = case["width"], case["height"]
        if "bytes" in case:
            buf = np.array(case["bytes"], np.uint8).reshape(h, 2 * w)
            want = np.array(case["yuv"], np.uint8).reshape(h, w, 3)
        else:
            buf = np.array([case["row_bytes_even"] if y % 2 == 0 else case["row_bytes_odd"] for y in range(h)], np.uint8)
            want = np.array([case["row_yuv_even"] if y % 2 == 0 else case["row_yuv_odd"] for y in range(h)], np.uint8)
        assert np.array_equal(_read_only(ol.PF_UYVY, buf, w, h), want)


@pytest.mark.parametrize("pf", [ol.PF_NV12, ol.PF_NV21, ol.PF_P010, ol.PF_P210, ol.PF_Y210, ol.PF_UYVY])
def test_readers_against_numpy_indexing(pf):
    w, h = 14, 6
    buf = frame(pf, w, h, 100 + pf, pad=3)
    got = _read_only(pf, buf, w, h)
    want = np.zeros_like(got)
    for y in range(h):
        for x in range(w):
            if pf in (ol.PF_NV12, ol.PF_NV21, ol.PF_P010, ol.PF_P210):
                cy = y if pf == ol.PF_P210 else y // 2
                pair = buf[h + cy, 2 * (x // 2): 2 * (x // 2) + 2]
                u, v = (pair[1], pair[0]) if pf == ol.PF_NV21 else (pair[0], pair[1])
                want[y, x] = (buf[y, x], u, v)
            else:
                g = buf[y, 4 * (x // 2): 4 * (x // 2) + 4]
                want[y, x] = (g[1 + 2 * (x % 2)], g[0], g[2]) if pf == ol.PF_UYVY else (g[2 * (x % 2)], g[1], g[3])
    assert np.array_equal(got, want)


# ---- conversions: golden vectors of the reference's unit test --------------------------------------------

def _pixels(rows, dtype):
    a = np.array(rows, dtype)
    return a.reshape(1, a.shape[0], -1) if a.ndim == 2 else a.reshape(1, -1)


def test_gray_alpha_and_swap_codes_on_the_reference_unit_test_vectors():
    g = GOLDEN
    assert np.array_equal(ol.oracle_convert_code(5, _pixels(g["rgb2gray_u8"]["in"], np.uint8))[0], np.array(g["rgb2gray_u8"]["out"], np.uint8))
    assert np.array_equal(ol.oracle_convert_code(0, _pixels(g["bgr2bgra"]["in"], np.uint8))[0], np.array(g["bgr2bgra"]["out"], np.uint8))
    assert np.array_equal(ol.oracle_convert_code(6, _pixels(g["bgr2gray"]["in"], np.uint8))[0], np.array(g["bgr2gray"]["out"], np.uint8))
    assert np.array_equal(ol.oracle_convert_code(8, _pixels(g["bgra2gray"]["in"], np.uint8))[0], np.array(g["bgra2gray"]["out"], np.uint8))
    assert np.array_equal(ol.oracle_convert_code(2, _pixels(g["bgr2rgba"]["in"], np.uint8))[0], np.array(g["bgr2rgba"]["out"], np.uint8))
    assert np.array_equal(ol.oracle_convert_code(3, _pixels(g["bgra2rgb"]["in"], np.uint8))[0], np.array(g["bgra2rgb"]["out"], np.uint8))


def test_normalize_on_the_reference_unit_test_vectors():
    src = _pixels([[0, 128, 255], [64, 192, 32]], np.uint8)
    want = np.array([[0.0, np.float32(128.0) / np.float32(255.0), 1.0],
                     [np.float32(64.0) / np.float32(255.0), np.float32(192.0) / np.float32(255.0), np.float32(32.0) / np.float32(255.0)]], np.float32)
    assert ol.oracle_normalize(0, src)[0].tobytes() == want.tobytes()


# ---- conversions: closed forms ----------------------------------------------------------------------------

def test_neutral_chroma_gives_gray_of_the_scaled_luma():
    # U = V = chroma offset: R = G = B = (Y - luma offset) * max/limitY for limited range, Y for full range
    for cd, dt, mx, lu, ch, ly in ((ol.CD_P8, np.uint8, 255.0, 16.0, 128, 219.0), (ol.CD_P10, np.uint16, 1023.0, 64.0, 512, 876.0)):
        ys = np.arange(0, int(mx) + 1, 7, dtype=dt)
        src = np.stack([ys, np.full_like(ys, ch), np.full_like(ys, ch)], axis=-1).reshape(1, -1, 3)
        for cp in (0, 1, 2):
            full = ol.oracle_convert_depth(cd, ol.CR_FULL, cp, True, src)[0]
            assert np.array_equal(full, np.repeat(ys.astype(np.float32)[:, None], 3, axis=1))
            lim = ol.oracle_convert_depth(cd, ol.CR_LIMITED, cp, True, src)[0]
            want = (ys.astype(np.float32) - np.float32(lu)) * (np.float32(mx) / np.float32(ly))
            assert np.array_equal(lim, np.repeat(want[:, None], 3, axis=1))


def test_gray_rgb_gives_neutral_chroma_and_round_trip_returns_the_input():
    r = rng(7)
    for cd, dt, mx, ch in ((ol.CD_P8, np.uint8, 255, 128.0), (ol.CD_P12, np.uint16, 4095, 2048.0), (ol.CD_FN10, np.float32, 1.0, 512.0 / 1023.0)):
        if dt == np.float32:
            src = r.random((4, 33, 3), dtype=np.float32)
            gray = np.repeat(r.random((4, 33, 1), dtype=np.float32), 3, axis=2)
        else:
            src = r.integers(0, mx + 1, (4, 33, 3)).astype(dt)
            gray = np.repeat(r.integers(0, mx + 1, (4, 33, 1)).astype(dt), 3, axis=2)
        for cr in (0, 1):
            for cp in (0, 1, 2):
                yuv = ol.oracle_convert_depth(cd, cr, cp, False, gray)
                assert np.allclose(yuv[..., 1:], ch, atol=float(mx) * 1e-6 + 1e-7), (cd, cr, cp)
                back = ol.oracle_convert_depth(cd + 3 if cd < 3 else cd, cr, cp, True,
                                               (ol.oracle_convert_depth(cd, cr, cp, False, src) / np.float32(mx if cd < 3 else 1.0)).astype(np.float32))
                assert np.allclose(back * (mx if cd < 3 else 1.0), src.astype(np.float32), atol=float(mx) * 2e-5), (cd, cr, cp)


def test_gray_formula_rounds_half_to_even_and_ignores_alpha():
    src = rng(3).integers(0, 256, (5, 40, 4), dtype=np.uint8)
    lum = (src[..., 0].astype(np.float32) * np.float32(0.299) + src[..., 1].astype(np.float32) * np.float32(0.587)) + \
        src[..., 2].astype(np.float32) * np.float32(0.114)
    assert np.array_equal(ol.oracle_convert_code(7, src), np.rint(lum).astype(np.uint8))
    assert np.array_equal(ol.oracle_convert_code(5, np.ascontiguousarray(src[..., :3])), np.rint(lum).astype(np.uint8))
    f = rng(4).random((3, 17, 3), dtype=np.float32)
    # a float output is rounded too: the reference's type test takes float for a signed type
    assert ol.oracle_convert_code(9, f * np.float32(200.0)).tobytes() == np.rint((f[..., 0] * np.float32(200.0) * np.float32(0.299) + f[..., 1] * np.float32(200.0) * np.float32(0.587)) + f[..., 2] * np.float32(200.0) * np.float32(0.114)).astype(np.float32).tobytes()


# ---- writers ----------------------------------------------------------------------------------------------

@pytest.mark.parametrize("pf", [ol.PF_NV12, ol.PF_NV21, ol.PF_P010, ol.PF_P210, ol.PF_Y210, ol.PF_UYVY])
@pytest.mark.parametrize("size", [(16, 8), (13, 7)])
def test_write_then_read_returns_the_stored_samples(pf, size):
    """Luma survives exactly; chroma of a pixel is that of the pixel the writer takes the block's pair from."""
    w, h = size
    dt = np.uint16 if ol.PF_WIDE[pf] else np.uint8
    yuv = rng(50 + pf).integers(0, 1024 if ol.PF_WIDE[pf] else 256, (h, w, 3)).astype(dt)
    rows, cols = ol.frame_shape(pf, w + (w & 1), h + (h & 1))
    buf = np.full((rows, cols), 7, dt)
    # the stored frame keeps the even-size backing array; width/height passed are the odd ones
    wr = ol.write_yuv(pf, buf, w, h)
    if pf in (ol.PF_NV12, ol.PF_NV21, ol.PF_P010, ol.PF_P210):
        wr.height = h       # chroma base = pitch * height: keep the plane right after the luma rows
    ol.execute([ol.read_2d(yuv, 3)], [], [wr])
    rd = ol.read_yuv(pf, buf, w, h)
    back = np.zeros((h, w, 3), dt)
    ol.execute([rd], [], [ol.write(ol.WRITE_2D, back, 3, w, h)])
    assert np.array_equal(back[..., 0], yuv[..., 0])
    for y in range(h):
        for x in range(w):
            bx = x - (x & 1)
            if pf in (ol.PF_NV12, ol.PF_P010):
                sx, sy = bx, y - (y & 1)
            elif pf == ol.PF_NV21:
                sx, sy = min(bx + 1, w - 1), min(y - (y & 1) + 1, h - 1)
            else:
                sx, sy = bx, y
            assert tuple(back[y, x, 1:]) == tuple(yuv[sy, sx, 1:]), (pf, x, y)


# ---- the oracle against the reference's CPU backend -------------------------------------------------------

Y2R = [(ol.PF_NV12, 0, 0), (ol.PF_NV12, 1, 0), (ol.PF_NV12, 0, 1), (ol.PF_NV12, 0, 2), (ol.PF_NV12, 1, 2), (ol.PF_NV21, 1, 1),
       (ol.PF_NV21, 0, 0), (ol.PF_P010, 0, 2), (ol.PF_P210, 1, 1), (ol.PF_Y210, 0, 1), (ol.PF_UYVY, 0, 0), (ol.PF_UYVY, 1, 1)]
R2Y = [(ol.PF_NV12, 0, 1), (ol.PF_NV21, 1, 0), (ol.PF_P010, 0, 2), (ol.PF_P210, 1, 1), (ol.PF_Y210, 0, 0), (ol.PF_UYVY, 1, 2)]
DEPTHS = [(0, 0, 2), (2, 0, 0), (2, 1, 1), (3, 0, 1), (4, 1, 0), (5, 0, 2)]


@needs_ref
@pytest.mark.parametrize("pf,cr,cp", Y2R)
def test_yuv_to_rgb_matches_reference_backend(pf, cr, cp):
    w, h = 38, 12
    buf = frame(pf, w, h, 200 + pf * 7 + cr * 3 + cp, pad=5)
    assert ol.oracle_yuv_to_rgb(pf, cr, cp, buf, w, h).tobytes() == ol.ref_yuv_to_rgb(pf, cr, cp, buf, w, h).tobytes()


@needs_ref
@pytest.mark.parametrize("pf,cr,cp", R2Y)
def test_rgb_to_yuv_matches_reference_backend(pf, cr, cp):
    w, h = 36, 10
    dt = np.uint16 if ol.PF_WIDE[pf] else np.uint8
    rgb = rng(300 + pf).integers(0, 1024 if ol.PF_WIDE[pf] else 256, (h, w, 3)).astype(dt)
    rows, cols = ol.frame_shape(pf, w, h)
    a = ol.oracle_rgb_to_yuv(pf, cr, cp, rgb, np.full((rows, cols + 4), 9, dt))
    b = ol.ref_rgb_to_yuv(pf, cr, cp, rgb, np.full((rows, cols + 4), 9, dt))
    assert np.array_equal(a, b)


@needs_ref
@pytest.mark.parametrize("pf", [ol.PF_NV21, ol.PF_UYVY, ol.PF_P010])
def test_yuv_resize_matches_reference_backend(pf):
    w, h = 46, 20
    buf = frame(pf, w, h, 400 + pf)
    for dst in ((17, 9), (60, 31)):
        assert ol.oracle_yuv_resize(pf, buf, w, h, dst, 0.5).tobytes() == ol.ref_yuv_resize(pf, buf, w, h, dst, 0.5).tobytes()


@needs_ref
@pytest.mark.parametrize("cd,cr,cp", DEPTHS)
def test_depth_conversions_match_reference_backend(cd, cr, cp):
    r = rng(500 + cd)
    if cd >= 3:
        src = (r.random((9, 31, 3), dtype=np.float32) * np.float32(1.2) - np.float32(0.1)).astype(np.float32)
    elif cd == 0:
        src = r.integers(0, 256, (9, 31, 3), dtype=np.uint8)
    else:
        src = r.integers(0, 4096, (9, 31, 3)).astype(np.uint16)
    for to_rgb in (True, False):
        assert ol.oracle_convert_depth(cd, cr, cp, to_rgb, src).tobytes() == ol.ref_convert_depth(cd, cr, cp, to_rgb, src).tobytes()


@needs_ref
@pytest.mark.parametrize("which", sorted(ol.COLOR_CODES))
def test_color_codes_match_reference_backend(which):
    idt, cin, _, _, _ = ol.COLOR_CODES[which]
    r = rng(600 + which)
    if idt == np.float32:
        src = (r.random((7, 29, cin), dtype=np.float32) * np.float32(255.0)).astype(np.float32)
    else:
        src = r.integers(0, 256 if idt == np.uint8 else 1024, (7, 29, cin)).astype(idt)
    assert ol.oracle_convert_code(which, src).tobytes() == ol.ref_convert_code(which, src).tobytes()


@needs_ref
@pytest.mark.parametrize("which", [0, 1])
def test_normalize_matches_reference_backend(which):
    dt, mx = ol.NORMALIZE[which]
    src = rng(700 + which).integers(0, int(mx) + 1, (6, 27, 3)).astype(dt)
    assert ol.oracle_normalize(which, src).tobytes() == ol.ref_normalize(which, src).tobytes()


@needs_ref
def test_oracle_equals_the_reference_backend_on_the_sweep_of_random_sizes():
    # the 900 cases tests/test_gpu_color.py runs on the GPU (tests/random_cases.py); RGB -> YUV only at even sizes, odd
    # ones being outside what the reference's writers define
    import random_cases as rc
    for i in range(900):
        family, c = rc.color_sweep_case(i, Y2R, R2Y, [ol.PF_NV21, ol.PF_UYVY, ol.PF_P010])
        pf = c["pf"]
        if family == 0:
            same = ol.oracle_yuv_to_rgb(pf, c["cr"], c["cp"], c["frame"], c["w"], c["h"]).tobytes() == \
                ol.ref_yuv_to_rgb(pf, c["cr"], c["cp"], c["frame"], c["w"], c["h"]).tobytes()
        elif family == 1:
            h, w = c["rgb"].shape[:2]
            if (w | h) & 1:
                continue
            same = np.array_equal(ol.oracle_rgb_to_yuv(pf, c["cr"], c["cp"], c["rgb"], c["start"].copy()),
                                  ol.ref_rgb_to_yuv(pf, c["cr"], c["cp"], c["rgb"], c["start"].copy()))
        else:
            same = ol.oracle_yuv_resize(pf, c["frame"], c["w"], c["h"], c["dst"], 0.5).tobytes() == \
                ol.ref_yuv_resize(pf, c["frame"], c["w"], c["h"], c["dst"], 0.5).tobytes()
        assert same, f"case {i} (family {family})"
