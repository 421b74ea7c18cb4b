"""Pixel-format readers and writers (NV12, NV21, P010, P210, Y210, UYVY), YCbCr<->RGB for the depths, ranges and
primaries of the reference (color_conversion.h:150-201, itu_color.h:185-265), ColorConversion codes, NormalizePixel:
bit for bit against the CPU oracle, which test_oracle_color.py pins to the reference's unit-test vectors and to the
reference's CPU backend running the very same chain text (tests/cases/color_chains.h)."""
import numpy as np
import pytest

import oracle_lib as ol
import fkl_cases as cases

pytestmark = pytest.mark.gpu


def to_dev(a, device):
    import torch
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).to(device)
    return torch.from_numpy(a).to(device)


def to_host(t, dtype):
    a = t.cpu().numpy()
    return a.view(np.uint16) if np.dtype(dtype) == np.uint16 else a


def frame(pf, w, h, seed, pad=0):
    rows, cols = ol.frame_shape(pf, w, h)
    r = np.random.default_rng(seed)
    if ol.PF_WIDE[pf]:
        return r.integers(0, 1024, (rows, cols + pad), dtype=np.uint16)
    return r.integers(0, 256, (rows, cols + pad), dtype=np.uint8)


Y2R = [(ol.PF_NV12, 0, 0), (ol.PF_NV12, 1, 0), (ol.PF_NV12, 0, 1), (ol.PF_NV12, 0, 2), (ol.PF_NV12, 1, 2), (ol.PF_NV21, 1, 1),
       (ol.PF_NV21, 0, 0), (ol.PF_P010, 0, 2), (ol.PF_P210, 1, 1), (ol.PF_Y210, 0, 1), (ol.PF_UYVY, 0, 0), (ol.PF_UYVY, 1, 1)]
R2Y = [(ol.PF_NV12, 0, 1), (ol.PF_NV21, 1, 0), (ol.PF_P010, 0, 2), (ol.PF_P210, 1, 1), (ol.PF_Y210, 0, 0), (ol.PF_UYVY, 1, 2)]
DEPTHS = [(0, 0, 2), (2, 0, 0), (2, 1, 1), (3, 0, 1), (4, 1, 0), (5, 0, 2)]


@pytest.mark.parametrize("pf,cr,cp", Y2R)
def test_yuv_to_rgb(device, pf, cr, cp):
    import torch
    for (w, h, pad) in ((38, 12, 5), (640, 360, 0), (6, 2, 1)):
        buf = frame(pf, w, h, 900 + pf * 7 + cr * 3 + cp, pad)
        out = torch.full((h, w, 3), -7.0, dtype=torch.float32, device=device)
        cases.yuv_to_rgb(pf, cr, cp, to_dev(buf, device), w, h, out)
        torch.cuda.synchronize()
        assert out.cpu().numpy().tobytes() == ol.oracle_yuv_to_rgb(pf, cr, cp, buf, w, h).tobytes(), (w, h)


@pytest.mark.parametrize("pf,cr,cp", R2Y)
def test_rgb_to_yuv(device, pf, cr, cp):
    """Even and odd sizes: odd ones leave the last chroma block to a single column / row."""
    import torch
    dt = np.uint16 if ol.PF_WIDE[pf] else np.uint8
    for (w, h) in ((36, 10), (640, 360), (13, 7), (2, 2)):
        rgb = np.random.default_rng(950 + pf).integers(0, 1024 if ol.PF_WIDE[pf] else 256, (h, w, 3)).astype(dt)
        rows, cols = ol.frame_shape(pf, w + (w & 1), h + (h & 1))
        if pf in (ol.PF_NV12, ol.PF_NV21, ol.PF_P010, ol.PF_P210):
            rows = h + (h + 1) // 2 if pf != ol.PF_P210 else 2 * h     # chroma rows start right after `height` luma rows
        start = np.full((rows, cols + 4), 9, dt)
        dev = to_dev(start.copy(), device)
        cases.rgb_to_yuv(pf, cr, cp, to_dev(rgb, device), dev)
        torch.cuda.synchronize()
        want = ol.oracle_rgb_to_yuv(pf, cr, cp, rgb, start.copy())
        assert np.array_equal(to_host(dev, dt), want), (w, h)


@pytest.mark.parametrize("pf", [ol.PF_NV21, ol.PF_UYVY, ol.PF_P010])
def test_yuv_resize(device, pf):
    """NV21 feeds the bilinear gather kernel; the other formats take their taps one element at a time."""
    import torch
    w, h = 320, 180
    buf = frame(pf, w, h, 980 + pf)
    src = to_dev(buf, device)
    for dst in ((128, 64), (17, 9), (400, 231)):
        out = torch.zeros((dst[1], dst[0], 3), dtype=torch.float32, device=device)
        cases.yuv_resize(pf, src, w, h, dst, 0.5, out)
        torch.cuda.synchronize()
        assert out.cpu().numpy().tobytes() == ol.oracle_yuv_resize(pf, buf, w, h, dst, 0.5).tobytes(), dst


def test_yuv_resize_to_a_large_image_runs_in_bands(device):
    """A bilinear read that takes its taps one element at a time runs on the rows kernel, one element per thread; from 4 096
    workgroups per plane up its launch takes the one-dimensional grid whose workgroups are renumbered into one band per XCD."""
    import torch
    from fusedkernellibrary_amd import last_launch
    pf, w, h, dst = ol.PF_UYVY, 320, 180, (1030, 1021)
    buf = frame(pf, w, h, 1234)
    out = torch.zeros((dst[1], dst[0], 3), dtype=torch.float32, device=device)
    cases.yuv_resize(pf, to_dev(buf, device), w, h, dst, 0.5, out)
    torch.cuda.synchronize()
    ll = last_launch()
    blocks = ((dst[0] + 63) // 64) * ((dst[1] + 3) // 4)
    assert blocks >= 4096 and ll["kernel"].startswith("rows") and ll["grid"] == [(blocks + 7) // 8 * 8, 1, 1], ll
    assert out.cpu().numpy().tobytes() == ol.oracle_yuv_resize(pf, buf, w, h, dst, 0.5).tobytes()


RESIZED = [ol.PF_NV21, ol.PF_UYVY, ol.PF_P010]


def test_sweep_of_random_sizes(device):
    """900 seeded cases of the three chain kinds above (tests/random_cases.py) at random sizes and pitches."""
    import torch
    import random_cases as rc
    for i in range(900):
        family, c = rc.color_sweep_case(i, Y2R, R2Y, RESIZED)
        pf = c["pf"]
        if family == 0:
            out = torch.full((c["h"], c["w"], 3), -7.0, dtype=torch.float32, device=device)
            cases.yuv_to_rgb(pf, c["cr"], c["cp"], to_dev(c["frame"], device), c["w"], c["h"], out)
            torch.cuda.synchronize()
            same = out.cpu().numpy().tobytes() == ol.oracle_yuv_to_rgb(pf, c["cr"], c["cp"], c["frame"], c["w"], c["h"]).tobytes()
        elif family == 1:
            dev = to_dev(c["start"].copy(), device)
            cases.rgb_to_yuv(pf, c["cr"], c["cp"], to_dev(c["rgb"], device), dev)
            torch.cuda.synchronize()
            same = np.array_equal(to_host(dev, c["rgb"].dtype), ol.oracle_rgb_to_yuv(pf, c["cr"], c["cp"], c["rgb"], c["start"].copy()))
        else:
            dst = c["dst"]
            out = torch.zeros((dst[1], dst[0], 3), dtype=torch.float32, device=device)
            cases.yuv_resize(pf, to_dev(c["frame"], device), c["w"], c["h"], dst, 0.5, out)
            torch.cuda.synchronize()
            same = out.cpu().numpy().tobytes() == ol.oracle_yuv_resize(pf, c["frame"], c["w"], c["h"], dst, 0.5).tobytes()
        assert same, f"case {i} (family {family}): " + str({k: v for k, v in c.items() if not isinstance(v, np.ndarray)})


@pytest.mark.parametrize("cd,cr,cp", DEPTHS)
def test_depth_conversions(device, cd, cr, cp):
    import torch
    r = np.random.default_rng(1000 + cd)
    h, w = 45, 131
    if cd >= 3:
        src = (r.random((h, w, 3), dtype=np.float32) * np.float32(1.2) - np.float32(0.1)).astype(np.float32)
    elif cd == 0:
        src = r.integers(0, 256, (h, w, 3), dtype=np.uint8)
    else:
        src = r.integers(0, 4096, (h, w, 3)).astype(np.uint16)
    for to_rgb in (True, False):
        out = torch.zeros((h, w, 3), dtype=torch.float32, device=device)
        cases.convert_depth(cd, cr, cp, to_rgb, to_dev(src, device), out)
        torch.cuda.synchronize()
        assert out.cpu().numpy().tobytes() == ol.oracle_convert_depth(cd, cr, cp, to_rgb, src).tobytes(), to_rgb


@pytest.mark.parametrize("which", sorted(ol.COLOR_CODES))
def test_color_codes(device, which):
    import torch
    idt, cin, odt, cout, _ = ol.COLOR_CODES[which]
    r = np.random.default_rng(1100 + which)
    h, w = 33, 257
    if idt == np.float32:
        src = (r.random((h, w, cin), dtype=np.float32) * np.float32(255.0)).astype(np.float32)
    else:
        src = r.integers(0, 256 if idt == np.uint8 else 1024, (h, w, cin)).astype(idt)
    out = to_dev(np.zeros((h, w, cout) if cout > 1 else (h, w), odt), device)
    cases.convert_code(which, to_dev(src, device), out)
    torch.cuda.synchronize()
    assert to_host(out, odt).tobytes() == ol.oracle_convert_code(which, src).tobytes()


def test_gray_ties_round_to_even(device):
    """Luminances that land exactly on .5: R = G = B = v gives v * (0.299f + 0.587f + 0.114f) ~ v; build ties from floats."""
    import torch
    v = np.array([[0.5, 0.5, 0.5], [1.5, 1.5, 1.5], [2.5, 2.5, 2.5], [127.5, 127.5, 127.5]], np.float32).reshape(1, 4, 3)
    out = torch.zeros((1, 4), dtype=torch.float32, device=device)
    cases.convert_code(9, torch.from_numpy(v).to(device), out)
    torch.cuda.synchronize()
    assert out.cpu().numpy().tobytes() == ol.oracle_convert_code(9, v).tobytes()


@pytest.mark.parametrize("which", [0, 1])
def test_normalize(device, which):
    import torch
    dt, mx = ol.NORMALIZE[which]
    h, w = 21, 300
    src = np.random.default_rng(1200 + which).integers(0, int(mx) + 1, (h, w, 3)).astype(dt)
    out = torch.zeros((h, w, 3), dtype=torch.float32, device=device)
    cases.normalize(which, to_dev(src, device), out)
    torch.cuda.synchronize()
    assert out.cpu().numpy().tobytes() == ol.oracle_normalize(which, src).tobytes()


def test_sweep_of_random_sizes_of_the_per_pixel_conversions(device):
    """400 seeded cases at random sizes (1 x 1 to 600 x 12): the depth conversions in both directions, every ColorConversion
    code, NormalizePixel.  Inputs as in the tests above."""
    import torch
    codes = sorted(ol.COLOR_CODES)
    for i in range(400):
        r = np.random.default_rng(150000 + i)
        h, w = int(r.integers(1, 13)), int(r.integers(1, 601))
        kind = i % 3
        if kind == 0:
            cd, cr, cp = DEPTHS[int(r.integers(0, len(DEPTHS)))]
            to_rgb = bool(r.integers(0, 2))
            if cd >= 3:
                src = (r.random((h, w, 3), dtype=np.float32) * np.float32(1.2) - np.float32(0.1)).astype(np.float32)
            elif cd == 0:
                src = r.integers(0, 256, (h, w, 3), dtype=np.uint8)
            else:
                src = r.integers(0, 4096, (h, w, 3)).astype(np.uint16)
            out = torch.zeros((h, w, 3), dtype=torch.float32, device=device)
            cases.convert_depth(cd, cr, cp, to_rgb, to_dev(src, device), out)
            torch.cuda.synchronize()
            same = out.cpu().numpy().tobytes() == ol.oracle_convert_depth(cd, cr, cp, to_rgb, src).tobytes()
            what = ("depth", cd, cr, cp, to_rgb)
        elif kind == 1:
            which = codes[int(r.integers(0, len(codes)))]
            idt, cin, odt, cout, _ = ol.COLOR_CODES[which]
            if idt == np.float32:
                src = (r.random((h, w, cin), dtype=np.float32) * np.float32(255.0)).astype(np.float32)
            else:
                src = r.integers(0, 256 if idt == np.uint8 else 1024, (h, w, cin)).astype(idt)
            out = to_dev(np.zeros((h, w, cout) if cout > 1 else (h, w), odt), device)
            cases.convert_code(which, to_dev(src, device), out)
            torch.cuda.synchronize()
            same = to_host(out, odt).tobytes() == ol.oracle_convert_code(which, src).tobytes()
            what = ("code", which)
        else:
            which = int(r.integers(0, 2))
            dt, mx = ol.NORMALIZE[which]
            src = r.integers(0, int(mx) + 1, (h, w, 3)).astype(dt)
            out = torch.zeros((h, w, 3), dtype=torch.float32, device=device)
            cases.normalize(which, to_dev(src, device), out)
            torch.cuda.synchronize()
            same = out.cpu().numpy().tobytes() == ol.oracle_normalize(which, src).tobytes()
            what = ("normalize", which)
        assert same, (i, what, w, h)
