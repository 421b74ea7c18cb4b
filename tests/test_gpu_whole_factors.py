"""Resizes whose scale factors are whole numbers (4K -> 1080p and the like).  Every source point is then a pixel, three of
the four bilinear weights are zero, and the kernel takes only the first tap; the results must stay bit for bit those
of the four-tap blend (reference interpolation.h:70-104), which the CPU oracle computes in full.  Planes with whole
and with fractional factors share a launch, so both tap modes run side by side."""
import numpy as np
import pytest

import oracle_lib as ol
from fusedkernellibrary_amd import last_launch
import fkl_cases as cases

pytestmark = pytest.mark.gpu


def _dev(a, device):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def test_normalise_batch_with_whole_and_fractional_planes(device):
    import torch
    rng = np.random.RandomState(11)
    src = rng.randint(0, 256, (300, 400, 3)).astype(np.uint8)
    dw, dh = 32, 24
    rects = []
    for i in range(64):
        kind = i % 4
        if kind == 0:      # whole in both directions: 1x .. 4x
            w, h = dw * (1 + i // 4 % 4), dh * (1 + i // 16 % 4)
        elif kind == 1:    # whole in x only
            w, h = dw * (1 + i // 4 % 4), dh + 5 + i
        elif kind == 2:    # whole in y only
            w, h = dw + 3 + i, dh * (1 + i // 4 % 4)
        else:              # neither
            w, h = 37 + i, 29 + i // 2
        x = int(rng.randint(0, 400 - w + 1))
        y = int(rng.randint(0, 300 - h + 1))
        rects.append((x, y, w, h))
    rects[0] = (400 - 4 * dw, 300 - 4 * dh, 4 * dw, 4 * dh)     # reaches the image's last row and column
    rects[8] = (123, 45, dw, dh)                                # 1x: the crop itself
    rects = np.array(rects, np.int32)
    sub = np.array([10.5, 20.25, 30.125], np.float32)
    div = np.array([3.0, 57.375, 0.7], np.float32)
    want = ol.oracle_crop_resize_norm_split(src, rects, (dw, dh), sub, div)
    # a 32-pixel-wide planar output goes to the strip form of the kernel (which always blends four taps); with that form
    # switched off the tile form runs, whose waves pick the one-tap path plane by plane
    from fusedkernellibrary_amd import lib
    for form, kernel in ((1, "strip"), (0, "gather")):
        old = lib().fklhip_strip_form(form)
        try:
            out = torch.zeros((64, 3, dh, dw), dtype=torch.float32, device=device)
            cases.crop_resize_norm_split(_dev(src, device), rects, (dw, dh), sub, div, out)
            torch.cuda.synchronize()
        finally:
            lib().fklhip_strip_form(old)
        assert last_launch()["kernel"] == kernel
        assert out.cpu().numpy().tobytes() == want.tobytes()
    # a 1x plane is the crop itself, channels swapped, normalised
    plane = 8
    x, y, w, h = rects[plane]
    crop = src[y:y + h, x:x + w, ::-1].astype(np.float32)
    direct = ((crop - sub) / div).transpose(2, 0, 1)
    assert out[plane].cpu().numpy().tobytes() == direct.astype(np.float32).tobytes()


def test_letterboxed_batch_with_whole_factors(device):
    import torch
    rng = np.random.RandomState(12)
    src = rng.randint(0, 256, (400, 600, 3)).astype(np.uint8)
    dw, dh = 128, 64
    # 2x without bars; 2x with side bars; 1x with side bars; fractional; 3x
    rects = np.array([(10, 20, 256, 128), (300, 100, 128, 128), (0, 0, 64, 64), (77, 33, 100, 77), (216, 208, 384, 192)], np.int32)
    bg = np.array([1.0, 2.0, 3.0], np.float32)
    mul = np.array([2.0, 2.0, 2.0], np.float32)
    sub = np.array([128.0, 128.0, 128.0], np.float32)
    out = torch.zeros((5, dh, dw, 3), dtype=torch.uint8, device=device)
    cases.crop_resize_par_u8(_dev(src, device), rects, (dw, dh), bg, mul, sub, out)
    torch.cuda.synchronize()
    want = ol.oracle_crop_resize_par_u8(src, rects, (dw, dh), bg, mul, sub)
    assert out.cpu().numpy().tobytes() == want.tobytes()


@pytest.mark.parametrize("size,dst", [((64, 48), (32, 24)), ((64, 48), (64, 48)), ((128, 96), (32, 24)), ((66, 50), (33, 25)),
                                      ((64, 48), (32, 48)), ((64, 48), (40, 24))])
def test_nv12_whole_factors(device, size, dst):
    import torch
    w, h = size
    rng = np.random.RandomState(13)
    nv12 = rng.randint(0, 256, (h + h // 2, w)).astype(np.uint8)
    out = torch.zeros((3, dst[1], dst[0]), dtype=torch.float32, device=device)
    scale = np.float32(1.0 / 255.0)
    cases.nv12_rgb_resize_split(_dev(nv12, device), w, h, dst, scale, out)
    torch.cuda.synchronize()
    want = ol.oracle_nv12_rgb_resize_split(nv12, w, h, dst, scale)
    assert out.cpu().numpy().tobytes() == want.tobytes()
