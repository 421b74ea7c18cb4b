"""GPU edge cases of the two kernels: row tails, unaligned pitches, crops touching the image border (where the
gather kernel must not read past the last row), one-pixel crops, strong up- and down-scaling, letterboxing in both
orientations, repeated launches."""
import numpy as np
import pytest

import oracle_lib as ol
from fusedkernellibrary_amd import last_launch
import fkl_cases as cases
import workloads as wl

pytestmark = pytest.mark.gpu


def _c3(src_np, rects, dst, sub, div, device):
    import torch
    src = torch.from_numpy(src_np).to(device)
    out = torch.zeros((len(rects), 3, dst[1], dst[0]), dtype=torch.float32, device=device)
    cases.crop_resize_norm_split(src, rects, dst, sub, div, out)
    torch.cuda.synchronize()
    return out.cpu().numpy()


def test_crops_touching_borders_and_tiny_crops(device):
    rng = np.random.RandomState(41)
    w, h = 333, 217
    src = rng.randint(0, 256, (h, w, 3)).astype(np.uint8)
    rects = np.array([[0, 0, w, h], [w - 1, h - 1, 1, 1], [0, h - 2, w, 2], [w - 3, 0, 3, h],
                      [5, 7, 1, 50], [9, 3, 50, 1], [100, 100, 2, 2], [17, 19, 200, 150]], np.int32)
    sub, div = wl.C3_MEAN, wl.C3_STD
    for dst in ((224, 224), (97, 33), (1, 1), (130, 5)):
        got = _c3(src, rects, dst, sub, div, device)
        want = ol.oracle_crop_resize_norm_split(src, rects, dst, sub, div)
        assert got.tobytes() == want.tobytes(), dst


def test_strong_down_and_upscale_stay_exact(device):
    rng = np.random.RandomState(42)
    w, h = 1900, 1000
    src = rng.randint(0, 256, (h, w, 3)).astype(np.uint8)
    rects = np.array([[0, 0, w, h]] * 8, np.int32)
    rects[1] = [10, 10, 1800, 900]
    got = _c3(src, rects, (16, 16), wl.C3_MEAN, wl.C3_STD, device)   # factor ~119x62 per output pixel
    assert last_launch()["kernel"] == "strip"       # narrow planar output: a workgroup owns 8 whole rows
    assert got.tobytes() == ol.oracle_crop_resize_norm_split(src, rects, (16, 16), wl.C3_MEAN, wl.C3_STD).tobytes()
    got = _c3(src, rects, (640, 360), wl.C3_MEAN, wl.C3_STD, device)  # ~3x
    assert last_launch()["kernel"] == "gather"
    assert got.tobytes() == ol.oracle_crop_resize_norm_split(src, rects, (640, 360), wl.C3_MEAN, wl.C3_STD).tobytes()
    small = np.array([[w - 8, h - 6, 8, 6], [0, 0, 3, 2], [700, 400, 5, 9], [w - 2, 0, 2, h], [0, h - 1, w, 1],
                      [w - 1, h - 1, 1, 1], [33, 44, 17, 2], [5, h - 3, 9, 3]], np.int32)   # up to ~300x upscale, some at the last row
    got = _c3(src, small, (640, 360), wl.C3_MEAN, wl.C3_STD, device)
    assert got.tobytes() == ol.oracle_crop_resize_norm_split(src, small, (640, 360), wl.C3_MEAN, wl.C3_STD).tobytes()


def test_letterbox_both_orientations(device):
    import torch
    rng = np.random.RandomState(43)
    src_np = rng.randint(0, 256, (300, 400, 3)).astype(np.uint8)
    src = torch.from_numpy(src_np).to(device)
    rects = np.array([[0, 0, 400, 300], [10, 10, 30, 200], [10, 10, 300, 20], [50, 60, 7, 290 - 60], [0, 0, 1, 1]], np.int32)
    bg, mul, sub = np.array([3, 200, 77], np.float32), np.array([1.5, 0.5, 2.0], np.float32), np.array([10, -5, 128], np.float32)
    for dst in ((128, 64), (64, 128), (33, 33)):
        out = torch.zeros((5, dst[1], dst[0], 3), dtype=torch.uint8, device=device)
        cases.crop_resize_par_u8(src, rects, dst, bg, mul, sub, out)
        torch.cuda.synchronize()
        want = ol.oracle_crop_resize_par_u8(src_np, rects, dst, bg, mul, sub)
        assert np.array_equal(out.cpu().numpy(), want), dst


def test_letterbox_in_the_even_and_left_aligned_modes(device):
    # PRESERVE_AR_RN_EVEN and PRESERVE_AR_LEFT (and PRESERVE_AR through the same driver): the geometry is made on the host,
    # the kernel is the letterboxing one; band pixels are the background exactly, the picture is the oracle's bit for bit
    import torch
    rng = np.random.RandomState(143)
    src_np = rng.randint(0, 256, (300, 400, 3)).astype(np.uint8)
    src = torch.from_numpy(src_np).to(device)
    bg = np.array([3, 200, 77], np.float32)
    for rect in ([0, 0, 400, 300], [10, 10, 31, 200], [10, 10, 301, 21], [50, 60, 7, 230], [5, 5, 111, 67]):
        for dst in ((128, 64), (64, 128), (33, 33), (97, 35)):
            for ar in (ol.PRESERVE_AR, ol.PRESERVE_AR_RN_EVEN, ol.PRESERVE_AR_LEFT):
                out = torch.zeros((dst[1], dst[0], 3), dtype=torch.float32, device=device)
                cases.letterbox_ar(ar, src, rect, bg, out)
                torch.cuda.synchronize()
                want = ol.oracle_letterbox_ar(ar, src_np, np.array(rect, np.int32), dst, bg)
                assert out.cpu().numpy().tobytes() == want.tobytes(), (rect, dst, ar)
                if ar == ol.PRESERVE_AR_LEFT and rect[2] * dst[1] < rect[3] * dst[0]:      # narrower than the frame: band on the right only
                    assert not np.array_equal(want[dst[1] // 2, 0], bg) and np.array_equal(want[dst[1] // 2, -1], bg)


def test_unaligned_pitch_and_odd_width_rows(device):
    import torch
    rng = np.random.RandomState(44)
    for w, h, pad in ((1, 1, 0), (3, 5, 0), (5, 3, 1), (250, 9, 3), (256, 4, 0), (1023, 2, 2)):
        pitch_elems = w + pad
        buf = rng.uniform(-1, 1, (h, pitch_elems)).astype(np.float32)
        src = torch.from_numpy(buf).to(device)
        out = torch.full((h, pitch_elems), 7.0, dtype=torch.float32, device=device)
        cases.add_mul_chain(src[:, :w], 3, 0.5, 1.0001, out[:, :w])
        torch.cuda.synchronize()
        want = ol.oracle_add_mul_chain(np.ascontiguousarray(buf[:, :w]), 3, np.float32(0.5), np.float32(1.0001))
        got = out.cpu().numpy()
        assert got[:, :w].tobytes() == want.tobytes(), (w, h, pad)
        assert np.all(got[:, w:] == 7.0), "padding columns must not be written"


def test_uchar3_rows_with_unaligned_pitch(device):
    import torch
    rng = np.random.RandomState(45)
    for w, h in ((322, 11), (5, 2), (64, 64)):
        srcs_np = [rng.randint(0, 256, (h, w, 3)).astype(np.uint8) for _ in range(4)]
        mul = rng.uniform(0.5, 2, (4, 3)).astype(np.float32)
        add = rng.uniform(-64, 64, (4, 3)).astype(np.float32)
        srcs = [torch.from_numpy(s).to(device) for s in srcs_np]
        outs = [torch.zeros_like(s) for s in srcs]
        cases.batch_muladd_sat(srcs, mul, add, outs)
        torch.cuda.synchronize()
        want = ol.oracle_batch_muladd_sat(srcs_np, mul, add)
        for i in range(4):
            assert np.array_equal(outs[i].cpu().numpy(), want[i]), (w, h, i)
        expect = "rows" if (w * 3) % 4 == 0 else "rows_unaligned"
        assert last_launch()["kernel"] == expect


def test_repeated_launches_are_idempotent(device):
    import torch
    c = wl.config3(batch=8, width=640, height=360, dst=96, seed=51, rect_seed=52, min_side=24, span=300)
    src = torch.from_numpy(c["src"]).to(device)
    out = torch.zeros((8, 3, 96, 96), dtype=torch.float32, device=device)
    cases.set_reps(5)
    cases.crop_resize_norm_split(src, c["rects"], c["dst"], c["sub"], c["div"], out)
    torch.cuda.synchronize()
    first = out.cpu().numpy().copy()
    cases.crop_resize_norm_split(src, c["rects"], c["dst"], c["sub"], c["div"], out)
    torch.cuda.synchronize()
    assert out.cpu().numpy().tobytes() == first.tobytes()
    assert first.tobytes() == ol.oracle_crop_resize_norm_split(c["src"], c["rects"], c["dst"], c["sub"], c["div"]).tobytes()


def test_nv12_odd_targets(device):
    import torch
    rng = np.random.RandomState(46)
    for (w, h), dst in (((64, 32), (64, 32)), ((64, 32), (17, 9)), ((130, 66), (200, 100)), ((2, 2), (1, 1))):
        nv12 = rng.randint(0, 256, (h * 3 // 2, w)).astype(np.uint8)
        src = torch.from_numpy(nv12).to(device)
        out = torch.zeros((3, dst[1], dst[0]), dtype=torch.float32, device=device)
        cases.nv12_rgb_resize_split(src, w, h, dst, np.float32(1 / 255), out)
        torch.cuda.synchronize()
        want = ol.oracle_nv12_rgb_resize_split(nv12, w, h, dst, np.float32(1 / 255))
        assert out.cpu().numpy().tobytes() == want.tobytes(), ((w, h), dst)
