"""Warping<Affine|Perspective> (reference warping.h:42-96): destination pixels mapped through a matrix, bilinear read,
zero outside the source.  Bit for bit against the CPU oracle, which test_oracle.py pins to the reference backend."""
import math

import numpy as np
import pytest

import oracle_lib as ol
import fkl_cases as cases

pytestmark = pytest.mark.gpu

TH = math.radians(17)
AFFINE = [[1.3 * math.cos(TH), -1.3 * math.sin(TH), 20.5], [1.3 * math.sin(TH), 1.3 * math.cos(TH), -7.25]]
IDENTITY = [[1, 0, 0], [0, 1, 0]]
SHIFT_OUT = [[1, 0, 500], [0, 1, 0]]
PERSPECTIVE = [[1.1, 0.05, -3.0], [0.02, 0.9, 4.0], [0.0008, -0.0005, 1.0]]


@pytest.mark.parametrize("name,matrix,persp", [("affine", AFFINE, False), ("identity", IDENTITY, False), ("outside", SHIFT_OUT, False),
                                               ("perspective", PERSPECTIVE, True)])
@pytest.mark.parametrize("dst", [(100, 70), (131, 90), (7, 3)])
def test_warp_uchar3(device, name, matrix, persp, dst):
    import torch
    rng = np.random.RandomState(5)
    img = rng.randint(0, 256, (90, 131, 3)).astype(np.uint8)
    src = torch.from_numpy(img).to(device)
    out = torch.full((dst[1], dst[0], 3), -1.0, dtype=torch.float32, device=device)
    cases.warp(src, matrix, persp, dst, out)
    torch.cuda.synchronize()
    want = ol.oracle_warp(img, 3, matrix, dst, persp)
    assert out.cpu().numpy().tobytes() == want.tobytes()


@pytest.mark.parametrize("matrix,persp", [(AFFINE, False), (PERSPECTIVE, True)])
def test_warp_float(device, matrix, persp):
    import torch
    rng = np.random.RandomState(6)
    img = (rng.rand(64, 80).astype(np.float32) * 10 - 5)
    src = torch.from_numpy(img).to(device)
    out = torch.zeros((50, 60), dtype=torch.float32, device=device)
    cases.warp(src, matrix, persp, (60, 50), out)
    torch.cuda.synchronize()
    want = ol.oracle_warp(img, 1, matrix, (60, 50), persp)
    assert out.cpu().numpy().tobytes() == want.tobytes()
