"""CPU tests that pin the plain-C oracle (oracle/fkl_oracle.c).

Three kinds of evidence, none of which re-types the oracle's own formulas:
  1. known answers the reference's unit tests hold (saturate cast, BT.709 matrix, BGR swap, round),
  2. golden fixtures produced by the reference's own CPU backend (tests/golden/, made by make_golden.py),
     and the live reference build oracle/_ref when it is present,
  3. closed forms and brute force: ramp images, identity / exact-2x resize, constant chroma, letterbox bands,
     index-encoding address checks, numpy restatements of the pointwise chains.
"""
import ctypes as C
import hashlib
import json
import os

import numpy as np
import pytest

import oracle_lib as ol
import workloads as wl

HERE = os.path.dirname(os.path.abspath(__file__))
GOLD = np.load(os.path.join(HERE, "golden", "golden_outputs.npz"))
META = json.load(open(os.path.join(HERE, "golden", "golden_digests.json")))
DIG = META["digests"]
CASES = META["cases"]


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def bits_equal(a, b):
    return a.shape == b.shape and a.dtype == b.dtype and a.tobytes() == b.tobytes()


# ---- 1. known answers held by the reference's own tests --------------------------------------------------

def test_saturate_cast_known_answers():
    # utests/algorithm/image_processing/utest_saturate/utest_saturate_common.h:36-90 (0.5->0, 1.5->2, 2.5->2, ...)
    # and the values the reference build returns for the same inputs (golden_digests.json).
    o = ol.oracle()
    table = {0.5: 0, 1.5: 2, 2.5: 2, 3.5: 4, 254.5: 254, 255.5: 255, -0.5: 0, -3.0: 0, 1e9: 255,
             float("inf"): 255, float("-inf"): 0, float("nan"): 0}
    for v, want in table.items():
        assert o.fklo_saturate_cast_u8(v) == want, v
    for s, want in zip(DIG["saturate_inputs"], DIG["saturate_outputs"]):
        assert o.fklo_saturate_cast_u8(float(s)) == want, s


def test_saturate_cast_matches_numpy_rint_everywhere_it_matters():
    o = ol.oracle()
    rng = np.random.RandomState(7)
    vals = np.concatenate([np.arange(-4, 260, 0.5, dtype=np.float32), rng.uniform(-300, 600, 20000).astype(np.float32),
                           np.nextafter(np.arange(0, 256, dtype=np.float32) + np.float32(0.5), np.float32(1000)),
                           np.nextafter(np.arange(0, 256, dtype=np.float32) + np.float32(0.5), np.float32(-1000))])
    want = np.clip(np.rint(vals), 0, 255).astype(np.uint8)
    got = np.array([o.fklo_saturate_cast_u8(float(v)) for v in vals], np.uint8)
    assert np.array_equal(got, want)


def test_round_half_away_known_answers():
    # utests/core/constexpr_libs/utest_constexpr_cmath.h:246-259: equals std::round at +-1.4/1.5/1.6 ...
    o = ol.oracle()
    for v, want in {1.4: 1, 1.5: 2, 1.6: 2, -1.4: -1, -1.5: -2, -1.6: -2, 2.5: 3, -2.5: -3, 0.0: 0, 0.49999997: 0}.items():
        assert o.fklo_round_half_away(v) == want


def test_bt709_full_matrix_known_answer():
    # utests/algorithm/image_processing/utest_color_conversion.h:441-447: {1,0,1.5748} {1,-0.187324256,-0.468124270} {1,1.8556,0}
    m = (C.c_float * 9)()
    ol.oracle().fklo_yuv2rgb_709_full_matrix(m)
    want = np.array([1, 0, 1.574800014, 1, -0.187324256, -0.468124270, 1, 1.855599999, 0], np.float32)
    assert np.array_equal(np.array(list(m), np.float32), want)
    assert [float(np.float32(v)) for v in m] == DIG["bt709_full_matrix"]


def test_bgr_swap_known_answer():
    # utest_color_conversion.h:90-101: {100,150,200} -> {200,150,100}, {50,75,125} -> {125,75,50}
    src = np.array([[[100, 150, 200], [50, 75, 125]]], np.uint8)
    out = np.zeros_like(src)
    ol.execute([ol.read_2d(src, 3)], [ol.op(ol.REORDER, idx=(2, 1, 0, 0))], [ol.write(ol.WRITE_2D, out, 3, 2, 1)])
    assert out.tolist() == [[[200, 150, 100], [125, 75, 50]]]


def test_nv12_constant_chroma_gives_gray():
    # U = V = 128 makes both chroma terms exactly zero: R = G = B = Y.
    w, h = 16, 8
    buf = np.full((h * 3 // 2, w), 128, np.uint8)
    buf[:h] = np.arange(w * h, dtype=np.uint8).reshape(h, w)
    out = np.zeros((h, w, 3), np.float32)
    ol.execute([ol.read_nv12(buf, w, h, tap_ops=[ol.op(ol.YUV2RGB_709_FULL)])], [], [ol.write(ol.WRITE_2D, out, 3, w, h)])
    y = buf[:h].astype(np.float32)
    for c in range(3):
        assert np.array_equal(out[..., c], y)


def test_mt19937_known_answers():
    # std::mt19937 default-seeded: first output 3499211612, 10000th 4123659995 (C++ standard, [rand.predef]).
    g = ol.MT()
    ol.oracle().fklo_mt_seed(C.byref(g), 5489)
    vals = [ol.oracle().fklo_mt_next(C.byref(g)) for _ in range(10000)]
    assert vals[0] == 3499211612 and vals[-1] == 4123659995
    assert np.array_equal(np.array(vals, np.uint32), wl.RawMT(5489).u32(10000))


def test_workload_generators_match_the_c_generator():
    g = ol.MT()
    ol.oracle().fklo_mt_seed(C.byref(g), 3)
    a = np.zeros(1000, np.uint8)
    ol.oracle().fklo_mt_fill_bytes(C.byref(g), a.ctypes.data_as(C.c_void_p), 1000)
    assert np.array_equal(a, wl.RawMT(3).bytes(1000))
    ol.oracle().fklo_mt_seed(C.byref(g), 2)
    f = np.zeros(1000, np.float32)
    ol.oracle().fklo_mt_fill_unit_floats(C.byref(g), f.ctypes.data_as(C.c_void_p), 1000)
    assert np.array_equal(f, wl.RawMT(2).unit_floats(1000)) and f.min() >= -1 and f.max() < 1
    ol.oracle().fklo_mt_seed(C.byref(g), 44)
    ol.oracle().fklo_mt_fill_range_floats(C.byref(g), f.ctypes.data_as(C.c_void_p), 1000, -64.0, 64.0)
    assert np.array_equal(f, wl.RawMT(44).range_floats(1000, -64.0, 64.0))


# ---- 2. golden fixtures from the reference's CPU backend -------------------------------------------------

def test_letterbox_geometry_matches_reference():
    for key, want in DIG["letterbox"].items():
        size = key.split("->")[0]
        sw, sh = (int(v) for v in size.split("x"))
        rp = ol.ResizeParams()
        ol.oracle().fklo_compute_resize_params(sw, sh, 128, 64, ol.PRESERVE_AR, C.byref(rp))
        assert [rp.x1, rp.y1, rp.x2, rp.y2] == want["rect"], key
        assert float(np.float32(rp.fx)) == want["fx"] and float(np.float32(rp.fy)) == want["fy"], key


def _geometry_of_the_oracle(ar, sw, sh, dw, dh):
    rp = ol.ResizeParams()
    ol.oracle().fklo_compute_resize_params(sw, sh, dw, dh, ar, C.byref(rp))
    return [rp.x1, rp.y1, rp.x2, rp.y2], float(np.float32(rp.fx)), float(np.float32(rp.fy))


def test_aspect_ratio_modes_match_the_committed_reference_vectors():
    # PRESERVE_AR (0), PRESERVE_AR_RN_EVEN (2), PRESERVE_AR_LEFT (3): tests/golden/resize_geometry_reference_vectors.json
    with open(os.path.join(HERE, "golden", "resize_geometry_reference_vectors.json")) as f:
        vectors = json.load(f)
    assert len(vectors) == 45
    for key, want in vectors.items():
        ar, rest = key.split(":")
        src, dst = rest.split("->")
        (sw, sh), (dw, dh) = (tuple(int(v) for v in t.split("x")) for t in (src, dst))
        rect, fx, fy = _geometry_of_the_oracle(int(ar), sw, sh, dw, dh)
        assert rect == want["rect"] and fx == want["fx"] and fy == want["fy"], key
        if int(ar) == 2:
            assert (rect[2] - rect[0] + 1) % 2 == 0 or (rect[3] - rect[1] + 1) % 2 == 0       # one side made even
        if int(ar) == 3:
            assert rect[0] == 0


@pytest.mark.skipif(not ol.have_ref(), reason="oracle/_ref not built")
def test_aspect_ratio_modes_match_the_live_reference_on_random_sizes():
    rng = np.random.default_rng(77)
    for _ in range(300):
        sw, sh, dw, dh = (int(v) for v in rng.integers(2, 700, 4))
        for ar in (0, 2, 3):
            o4 = (C.c_int32 * 4)()
            f2 = (C.c_float * 2)()
            assert ol.ref().fklref_resize_params_ar(ar, sw, sh, dw, dh, o4, f2) == 0
            rect, fx, fy = _geometry_of_the_oracle(ar, sw, sh, dw, dh)
            assert rect == list(o4) and fx == float(np.float32(f2[0])) and fy == float(np.float32(f2[1])), (ar, sw, sh, dw, dh)


def test_golden_c1():
    c = wl.config1(**CASES["c1_small"])
    rects = np.array(META["c1_small_rects"], np.int32)
    assert bits_equal(ol.oracle_crop_resize_par_u8(c["src"], rects, c["dst"], c["bg"], c["mul"], c["sub"]), GOLD["c1_small"])
    c = wl.config1()
    got = ol.oracle_crop_resize_par_u8(c["src"], c["rects"], c["dst"], c["bg"], c["mul"], c["sub"])
    assert bits_equal(got, GOLD["c1_full"]) and sha(got) == DIG["c1_full"]


@pytest.mark.parametrize("n", [1, 2, 3, 10, 50, 100])
def test_golden_c2_small(n):
    c = wl.config2(**CASES["c2_small"])
    assert bits_equal(ol.oracle_add_mul_chain(c["src"], n, c["add"], c["mul"]), GOLD[f"c2_small_n{n}"])


def test_golden_c2_full_n10():
    c = wl.config2()
    assert sha(ol.oracle_add_mul_chain(c["src"], 10, c["add"], c["mul"])) == DIG["c2_full_n10"]


def test_golden_c3():
    c = wl.config3(**CASES["c3_small"])
    assert bits_equal(ol.oracle_crop_resize_norm_split(c["src"], c["rects"], c["dst"], c["sub"], c["div"]), GOLD["c3_small"])
    c = wl.config3()
    assert sha(c["rects"]) == DIG["c3_rects"]
    assert sha(ol.oracle_crop_resize_norm_split(c["src"], c["rects"], c["dst"], c["sub"], c["div"])) == DIG["c3_full"]


def test_golden_c4():
    c = wl.config4(**CASES["c4_small"])
    assert bits_equal(np.stack(ol.oracle_batch_muladd_sat(c["srcs"], c["mul"], c["add"])), GOLD["c4_small"])


def test_golden_c5():
    for name in ("c5_small", "c5_odd"):
        c = wl.config5(**CASES[name])
        assert bits_equal(ol.oracle_nv12_rgb_resize_split(c["nv12"], c["width"], c["height"], c["dst"], c["scale"]), GOLD[name]), name
    c = wl.config5()
    assert sha(ol.oracle_nv12_rgb_resize_split(c["nv12"], c["width"], c["height"], c["dst"], c["scale"])) == DIG["c5_full"]


@pytest.mark.skipif(not ol.have_ref(), reason="reference CPU backend (oracle/_ref) not built here")
def test_oracle_equals_live_reference_on_random_cases():
    rng = np.random.RandomState(123)
    for trial in range(6):
        w, h = int(rng.randint(80, 400)), int(rng.randint(60, 300))
        src = rng.randint(0, 256, (h, w, 3)).astype(np.uint8)
        rects = []
        for _ in range(8):
            x, y = int(rng.randint(0, w - 8)), int(rng.randint(0, h - 8))
            rects.append((x, y, int(rng.randint(1, w - x + 1)), int(rng.randint(1, h - y + 1))))
        rects = np.array(rects, np.int32)
        dst = (int(rng.randint(1, 200)), int(rng.randint(1, 200)))
        sub, div = rng.uniform(0, 255, 3).astype(np.float32), rng.uniform(0.5, 80, 3).astype(np.float32)
        assert bits_equal(ol.oracle_crop_resize_norm_split(src, rects, dst, sub, div),
                          ol.ref_crop_resize_norm_split(src, rects, dst, sub, div)), (trial, "ignore_ar")
        bg, mul = rng.uniform(0, 255, 3).astype(np.float32), rng.uniform(0.2, 3, 3).astype(np.float32)
        assert bits_equal(ol.oracle_crop_resize_par_u8(src, rects[:5], dst, bg, mul, sub),
                          ol.ref_crop_resize_par_u8(src, rects[:5], dst, bg, mul, sub)), (trial, "preserve_ar")
        same = rects[:4].copy()
        same[:, 2], same[:, 3] = 7 + trial, 5 + trial
        same[:, 0] = np.minimum(same[:, 0], w - same[:, 2])
        same[:, 1] = np.minimum(same[:, 1], h - same[:, 3])
        assert bits_equal(ol.oracle_crop_swap_u8(src, same), ol.ref_crop_swap_u8(src, same)), (trial, "int-only")
        ew, eh = 2 * int(rng.randint(8, 100)), 2 * int(rng.randint(8, 60))
        nv12 = rng.randint(0, 256, (eh * 3 // 2, ew)).astype(np.uint8)
        d5 = (int(rng.randint(1, 150)), int(rng.randint(1, 90)))
        assert bits_equal(ol.oracle_nv12_rgb_resize_split(nv12, ew, eh, d5, np.float32(1 / 255)),
                          ol.ref_nv12_rgb_resize_split(nv12, ew, eh, d5, np.float32(1 / 255))), (trial, "nv12")


# ---- 3. closed forms and brute force ----------------------------------------------------------------------

def _ramp(w, h):
    img = np.zeros((h, w, 2), np.float32)
    img[..., 0] = np.arange(w, dtype=np.float32)[None, :]
    img[..., 1] = np.arange(h, dtype=np.float32)[:, None]
    return img


def test_bilinear_of_a_ramp_is_the_source_coordinate():
    # Bilinear interpolation of an affine image is affine: out(i, j) = (x0 + i*fx, y0 + j*fy) wherever no tap is
    # clamped (interpolation.h:100-103).  Factors 0.5 and 4 keep every product exact.
    img = _ramp(64, 48)
    x0, y0, cw, ch = 8, 4, 16, 12
    for dw, dh in ((32, 24), (4, 3)):
        out = np.zeros((dh, dw, 2), np.float32)
        ol.execute([ol.read_2d(img, 2, crop=(x0, y0, cw, ch), resize=(dw, dh))], [], [ol.write(ol.WRITE_2D, out, 2, dw, dh)])
        fx, fy = cw / dw, ch / dh
        for j in range(dh):
            for i in range(dw):
                if i * fx <= cw - 1 and j * fy <= ch - 1 and (i * fx) % 1 == 0 or fx < 1:
                    if (np.floor(i * fx) + 1 <= cw - 1) and (np.floor(j * fy) + 1 <= ch - 1):
                        assert out[j, i, 0] == np.float32(x0 + i * fx) and out[j, i, 1] == np.float32(y0 + j * fy), (dw, i, j)


def test_identity_resize_returns_the_input_as_float():
    rng = np.random.RandomState(3)
    src = rng.randint(0, 256, (20, 30, 3)).astype(np.uint8)
    out = np.zeros((20, 30, 3), np.float32)
    ol.execute([ol.read_2d(src, 3, resize=(30, 20))], [], [ol.write(ol.WRITE_2D, out, 3, 30, 20)])
    assert np.array_equal(out, src.astype(np.float32))


def test_exact_2x_downscale_picks_even_pixels():
    rng = np.random.RandomState(4)
    src = rng.randint(0, 256, (40, 60, 3)).astype(np.uint8)
    out = np.zeros((20, 30, 3), np.float32)
    ol.execute([ol.read_2d(src, 3, resize=(30, 20))], [], [ol.write(ol.WRITE_2D, out, 3, 30, 20)])
    assert np.array_equal(out, src[::2, ::2].astype(np.float32))


def test_right_and_bottom_edge_taps_are_clamped_but_weighted_unclamped():
    # 2x upscale of a 2x2 image: the last column/row weights use x2 = x1 + 1 while the tap re-reads the edge pixel,
    # so out = edge*(w_left) + edge*(w_right) and the value stays the edge value.
    src = np.array([[[10.0], [20.0]], [[30.0], [40.0]]], np.float32).reshape(2, 2)
    out = np.zeros((4, 4), np.float32)
    ol.execute([ol.read_2d(src, 1, resize=(4, 4))], [], [ol.write(ol.WRITE_2D, out, 1, 4, 4)])
    want = np.array([[10, 15, 20, 20], [20, 25, 30, 30], [30, 35, 40, 40], [30, 35, 40, 40]], np.float32)
    assert np.array_equal(out, want)


def test_letterbox_band_is_exactly_the_background():
    rng = np.random.RandomState(5)
    src = rng.randint(0, 256, (40, 60, 3)).astype(np.uint8)
    bg = (7.0, 8.0, 9.0)
    out = np.zeros((64, 128, 3), np.float32)
    ol.execute([ol.read_2d(src, 3, resize=(128, 64), ar=ol.PRESERVE_AR, bg=bg)], [], [ol.write(ol.WRITE_2D, out, 3, 128, 64)])
    rp = ol.ResizeParams()
    ol.oracle().fklo_compute_resize_params(60, 40, 128, 64, ol.PRESERVE_AR, C.byref(rp))
    assert (rp.x1, rp.y1, rp.x2, rp.y2) == (16, 0, 111, 63)
    assert np.all(out[:, :16] == np.array(bg, np.float32)) and np.all(out[:, 112:] == np.array(bg, np.float32))
    assert np.array_equal(out[0, 16], src[0, 0].astype(np.float32))


def test_tensor_write_and_split_addressing():
    # Values encode (x, y, z, c); the expected layouts are plain numpy reshapes.
    b, h, w = 3, 4, 5
    srcs = []
    for z in range(b):
        a = np.zeros((h, w, 3), np.float32)
        for c in range(3):
            a[..., c] = 1000 * z + 100 * c + 10 * np.arange(h)[:, None] + np.arange(w)[None, :]
        srcs.append(a)
    aos = np.zeros((b, h, w, 3), np.float32)
    ol.execute([ol.read_2d(s, 3) for s in srcs], [], [ol.write(ol.TENSOR_WRITE, aos, 3, w, h, b, 1)])
    assert np.array_equal(aos, np.stack(srcs))
    planar = np.zeros((b, 3, h, w), np.float32)
    ol.execute([ol.read_2d(s, 3) for s in srcs], [], [ol.write(ol.TENSOR_SPLIT, planar, 3, w, h, b, 3)])
    assert np.array_equal(planar, np.stack(srcs).transpose(0, 3, 1, 2))


def test_pointwise_chains_against_numpy():
    c = wl.config2(width=97, height=13, seed=21)
    want = c["src"].copy()
    for i in range(10):
        want = (want + np.float32(0.5)).astype(np.float32) if i % 2 == 0 else (want * np.float32(1.0001)).astype(np.float32)
    assert np.array_equal(ol.oracle_add_mul_chain(c["src"], 10, c["add"], c["mul"]), want)
    c = wl.config4(batch=3, width=50, height=20, seed=22, param_seed=23)
    got = ol.oracle_batch_muladd_sat(c["srcs"], c["mul"], c["add"])
    for i in range(3):
        v = (c["srcs"][i].astype(np.float32) * c["mul"][i]).astype(np.float32) + c["add"][i]
        assert np.array_equal(got[i], np.clip(np.rint(v.astype(np.float32)), 0, 255).astype(np.uint8))


def test_pitched_source_rows():
    rng = np.random.RandomState(6)
    padded = rng.randint(0, 256, (10, 64)).astype(np.uint8)   # 64-byte pitch, 17 pixels of 3 bytes used
    out = np.zeros((10, 17, 3), np.uint8)
    ol.execute([ol.read_2d(padded, 3, width=17)], [], [ol.write(ol.WRITE_2D, out, 3, 17, 10)])
    assert np.array_equal(out, padded[:, :51].reshape(10, 17, 3))


def test_divergent_plane_sizes_are_rejected():
    src = np.zeros((20, 20, 3), np.uint8)
    out = np.zeros((2, 8, 8, 3), np.uint8)
    with pytest.raises(RuntimeError):
        ol.execute([ol.read_2d(src, 3, crop=(0, 0, 8, 8)), ol.read_2d(src, 3, crop=(0, 0, 6, 8))], [],
                   [ol.write(ol.TENSOR_WRITE, out, 3, 8, 8, 2, 1)])


@pytest.mark.skipif(not ol.have_ref(), reason="reference CPU backend not built (needs the reference tree)")
def test_default_planes_match_reference_backend():
    """BatchRead<CONDITIONAL_WITH_DEFAULT> (batch_operations.h:221-281): planes >= usedPlanes yield the default value."""
    rng = np.random.RandomState(3)
    src = rng.randint(0, 256, (120, 200, 3)).astype(np.uint8)
    rects = np.array([[0, 0, 50, 40], [10, 10, 100, 80], [150, 80, 50, 40], [5, 5, 20, 100], [0, 0, 200, 120], [100, 60, 3, 2],
                      [20, 30, 64, 64], [1, 2, 77, 33]], np.int32)
    mean, std = (123.675, 116.28, 103.53), (58.395, 57.12, 57.375)
    for used in (0, 3, 8):
        a = ol.oracle_crop_resize_default_norm_split(src, rects, (32, 24), used, (1.5, -2.0, 300.0), mean, std)
        b = ol.ref_crop_resize_default_norm_split(src, rects, (32, 24), used, (1.5, -2.0, 300.0), mean, std)
        assert a.tobytes() == b.tobytes()
    srcs = [rng.randint(0, 256, (30, 41, 3)).astype(np.uint8) for _ in range(4)]
    for active in (0, 2, 4):
        a = ol.oracle_batch_default_cast_mul(srcs, active, (7, 200, 33), (0.5, 2.0, 1.25))
        b = ol.ref_batch_default_cast_mul(srcs, active, (7, 200, 33), (0.5, 2.0, 1.25))
        assert a.tobytes() == b.tobytes()


def test_default_planes_closed_form():
    """A default plane holds compute(default) everywhere, whatever the source: checked without the reference."""
    src = np.full((40, 50, 3), 9, np.uint8)
    rects = np.array([[0, 0, 10, 10]] * 8, np.int32)
    out = ol.oracle_crop_resize_default_norm_split(src, rects, (6, 5), 2, (10.0, 20.0, 40.0), (1.0, 2.0, 3.0), (2.0, 4.0, 8.0))
    # BGR->RGB swaps the default too: (40, 20, 10), then (x - sub) / div
    assert np.all(out[2:, 0] == np.float32((40.0 - 1.0) / 2.0)) and np.all(out[2:, 1] == np.float32((20.0 - 2.0) / 4.0))
    assert np.all(out[2:, 2] == np.float32((10.0 - 3.0) / 8.0))
    assert np.all(out[:2, 0] == np.float32((9.0 - 1.0) / 2.0))


@pytest.mark.skipif(not ol.have_ref(), reason="reference CPU backend not built (needs the reference tree)")
def test_warp_matches_reference_backend():
    """Warping<Affine|Perspective> (warping.h:42-96) on a uchar3 image."""
    import math
    rng = np.random.RandomState(5)
    src = rng.randint(0, 256, (90, 131, 3)).astype(np.uint8)
    th = math.radians(17)
    affine = [[1.3 * math.cos(th), -1.3 * math.sin(th), 20.5], [1.3 * math.sin(th), 1.3 * math.cos(th), -7.25]]
    persp = [[1.1, 0.05, -3.0], [0.02, 0.9, 4.0], [0.0008, -0.0005, 1.0]]
    for matrix, p, dst in ((affine, False, (100, 70)), (persp, True, (160, 120)), ([[1, 0, 0], [0, 1, 0]], False, (131, 90))):
        a = ol.oracle_warp(src, 3, matrix, dst, p)
        b = ol.ref_warp_u8x3(src, matrix, dst, p)
        assert a.tobytes() == b.tobytes()


@pytest.mark.skipif(not ol.have_ref(), reason="reference CPU backend not built (needs the reference tree)")
@pytest.mark.parametrize("dtype,cn", [(np.uint8, 4), (np.uint16, 3), (np.uint8, 1)])
def test_warp_of_other_pixel_types_matches_reference_backend(dtype, cn):
    import math
    rng = np.random.RandomState(9)
    shape = (50, 71, cn) if cn > 1 else (50, 71)
    src = rng.randint(0, 1000 if dtype == np.uint16 else 256, shape).astype(dtype)
    th = math.radians(-11)
    affine = [[0.8 * math.cos(th), -0.8 * math.sin(th), -6.5], [0.8 * math.sin(th), 0.8 * math.cos(th), 9.25]]
    persp = [[1.1, 0.05, -3.0], [0.02, 0.9, 4.0], [0.0008, -0.0005, 1.0]]
    for matrix, p, dst in ((affine, False, (90, 60)), (persp, True, (80, 64)), ([[1, 0, 40], [0, 1, 0]], False, (71, 50))):
        a = ol.oracle_warp(src, cn, matrix, dst, p)
        b = ol.ref_warp(src, matrix, dst, p)
        assert a.tobytes() == b.tobytes()


def test_warp_closed_forms():
    """Identity warp returns float(source); an integer shift returns the shifted source and zeros outside."""
    rng = np.random.RandomState(8)
    src = rng.randint(0, 256, (20, 30, 3)).astype(np.uint8)
    out = ol.oracle_warp(src, 3, [[1, 0, 0], [0, 1, 0]], (30, 20), False)
    assert (out == src.astype(np.float32)).all()
    out = ol.oracle_warp(src, 3, [[1, 0, 4], [0, 1, -2]], (30, 20), False)   # dst (x,y) reads src (x+4, y-2)
    assert (out[2:, :26] == src[:18, 4:].astype(np.float32)).all()
    assert (out[:2] == 0).all() and (out[:, 26:] == 0).all()


@pytest.mark.skipif(not ol.have_ref(), reason="reference CPU backend not built (needs the reference tree)")
def test_deinterlace_matches_reference_backend():
    rng = np.random.RandomState(5)
    for shape in ((12, 17, 3), (11, 9, 3), (1, 4, 3), (2, 3, 3)):
        src = rng.randint(0, 256, shape).astype(np.uint8)
        for mode in (ol.DEINTERLACE_BLEND, ol.DEINTERLACE_LINEAR_EVEN, ol.DEINTERLACE_LINEAR_ODD):
            if mode == ol.DEINTERLACE_LINEAR_ODD and shape[0] % 2:
                continue   # outside the reference's domain: its last line would read past the image
            assert ol.oracle_deinterlace(src, 3, mode).tobytes() == ol.ref_deinterlace_u8x3(src, mode).tobytes()


def test_deinterlace_closed_forms():
    """Rows r*10: BLEND gives ((r + r-1)*10 + 1)/2; INTER_LINEAR keeps one field and averages the neighbours of the other."""
    src = np.repeat((np.arange(6, dtype=np.uint8) * 10)[:, None], 4, axis=1)
    b = ol.oracle_deinterlace(src, 1, ol.DEINTERLACE_BLEND)
    assert (b[0] == 0).all() and all((b[r] == ((2 * r - 1) * 10 + 1) * 0.5).all() for r in range(1, 6))
    e = ol.oracle_deinterlace(src, 1, ol.DEINTERLACE_LINEAR_EVEN)
    assert all((e[r] == r * 10).all() for r in (0, 2, 4, 5)) and all((e[r] == (2 * r * 10 + 1) * 0.5).all() for r in (1, 3))
    o = ol.oracle_deinterlace(src, 1, ol.DEINTERLACE_LINEAR_ODD)
    assert all((o[r] == r * 10).all() for r in (0, 1, 3, 5)) and all((o[r] == (2 * r * 10 + 1) * 0.5).all() for r in (2, 4))
