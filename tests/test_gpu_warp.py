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


@pytest.mark.parametrize("dtype,cn", [(np.uint8, 4), (np.uint16, 3), (np.uint8, 1)])
@pytest.mark.parametrize("matrix,persp", [(AFFINE, False), (SHIFT_OUT, False), (PERSPECTIVE, True)])
def test_warp_other_pixel_types(device, matrix, persp, dtype, cn):
    """Pixels of 4, 6 and 1 bytes (chains compiled on first use): the tap windows, the duplicate of the edge tap and the
    zero weights of lanes outside are per element size."""
    import torch
    rng = np.random.RandomState(25)
    shape = (90, 131, cn) if cn > 1 else (90, 131)
    img = rng.randint(0, 1000 if dtype == np.uint16 else 256, shape).astype(dtype)
    src = torch.from_numpy(img.view(np.int16) if dtype == np.uint16 else img).to(device)
    for dst in ((100, 70), (131, 90), (9, 5)):
        out = torch.full((dst[1], dst[0], cn) if cn > 1 else (dst[1], dst[0]), -1.0, dtype=torch.float32, device=device)
        cases.warp(src, matrix, persp, dst, out, kind=ol.warp_kind(dtype, cn))
        torch.cuda.synchronize()
        want = ol.oracle_warp(img, cn, matrix, dst, persp)
        assert out.cpu().numpy().tobytes() == want.tobytes(), dst


def test_lanes_outside_the_source_ignore_what_their_stand_in_pixel_holds(device):
    """A lane whose source point lies outside fetches pixel (0, 0) instead and drops it.  A float image may hold anything
    there: the result is +0 all the same (integer images get there through weights of zero, float images must not)."""
    import torch
    img = (np.random.RandomState(16).rand(40, 48).astype(np.float32) * 10 - 5)
    img[0, 0] = np.nan
    img[0, 1] = np.inf
    matrix = [[1, 0, 5], [0, 1, -3]]                       # rows 0-2 and the last five columns map outside; column 0 and 1 are never read
    src = torch.from_numpy(img).to(device)
    out = torch.full((40, 48), -1.0, dtype=torch.float32, device=device)
    cases.warp(src, matrix, False, (48, 40), out)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    want = ol.oracle_warp(img, 1, matrix, (48, 40), False)
    assert np.isfinite(want).all() and (want[:3] == 0).all() and (want[:, 43:] == 0).all()
    assert got.tobytes() == want.tobytes()


@pytest.mark.parametrize("persp,dst", [(False, (2048, 2052)), (True, (2051, 2049)), (False, (1024, 3000))])
def test_large_warps_run_their_workgroups_in_one_band_per_xcd(device, persp, dst):
    """Launches of 4 096 workgroups per plane or more take a one-dimensional grid whose workgroups the kernel renumbers
    (one contiguous band of the output per XCD); smaller ones keep the two-dimensional grid.  Same bits either way: the
    affine chain is compiled ahead of time, the perspective one at run time, and the odd sizes leave partial blocks
    at the right and bottom edges and idle workgroups at the end of the grid."""
    import torch
    from fusedkernellibrary_amd import last_launch
    rng = np.random.RandomState(15)
    img = rng.randint(0, 256, (300, 417, 3)).astype(np.uint8)
    s = 0.19
    matrix = ([[s * math.cos(TH), -s * math.sin(TH), 60.0], [s * math.sin(TH), s * math.cos(TH), -40.0], [0.00001, -0.00002, 1.0]] if persp
              else [[s * math.cos(TH), -s * math.sin(TH), 60.0], [s * math.sin(TH), s * math.cos(TH), -40.0]])
    src = torch.from_numpy(img).to(device)
    out = torch.full((dst[1], dst[0], 3), -1.0, dtype=torch.float32, device=device)
    cases.warp(src, matrix, persp, dst, out)
    torch.cuda.synchronize()
    ll = last_launch()
    blocks = ((dst[0] + 255) // 256) * ((dst[1] + 3) // 4)
    if blocks >= 4096:
        assert ll["grid"] == [(blocks + 7) // 8 * 8, 1, 1], ll
    else:
        assert ll["grid"] == [(dst[0] + 255) // 256, (dst[1] + 3) // 4, 1], ll
    want = ol.oracle_warp(img, 3, matrix, dst, persp)
    assert out.cpu().numpy().tobytes() == want.tobytes()
