"""Seeded random cases of the three resizing chains (tests/random_cases.py), GPU against the C oracle and against the
digests the reference CPU backend gave for the same cases (tests/golden/random_batches_reference_digests.json), bit for
bit: source pitches that are and are not a multiple of four, crops from one pixel to the whole image (planes up to 256
wide whose source rows share their alignment and whose crops have two columns take the strip form of the kernel, all
others the tile form), enlarging and reducing in the same batch, divisors that take each of the three division
sequences, letterboxed planes, NV12 frames from 2 x 2 up.
Reference path: FK/algorithms/image_processing/resize.h:86-123, interpolation.h:70-104, crop.h,
color_conversion.h (ReadYUV, ConvertYUVToRGB), memory_operations.h:181-212."""
import json
import os

import numpy as np
import pytest

import fkl_cases as cases
import oracle_lib as ol
import random_cases as rc
from fusedkernellibrary_amd import last_launch

pytestmark = pytest.mark.gpu

with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "random_batches_reference_digests.json")) as f:
    REFERENCE = json.load(f)


@pytest.fixture(scope="module")
def device():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


def _image_on(device, backing, w):
    import torch
    h, pitch = backing.shape
    return torch.as_strided(torch.from_numpy(backing).to(device), (h, w, 3), (pitch, 3, 1))


def _same_bits(got, want, key):
    assert got.shape == want.shape
    a, b = got.view(np.uint8).reshape(-1), want.view(np.uint8).reshape(-1)
    assert a.tobytes() == b.tobytes(), f"{(a != b).sum()} of {a.size} bytes differ from the oracle; first at byte {np.argwhere(a != b)[0][0]}"
    assert rc.digest(got) == REFERENCE[key], "differs from what the reference CPU backend gave"


@pytest.mark.parametrize("seed,batch,size,pad,least,dst", rc.NORMALISE)
def test_random_batch_equals_the_oracle(device, seed, batch, size, pad, least, dst):
    import torch
    backing, rects, sub, div = rc.normalise_inputs(seed, batch, size, pad, least)
    w, pitch = size[0], backing.shape[1]
    out = torch.full((batch, 3, dst[1], dst[0]), float("nan"), dtype=torch.float32, device=device)
    print(f"seed {seed} batch {batch} source {size[0]}x{size[1]} pitch {pitch} target {dst[0]}x{dst[1]}", flush=True)
    cases.crop_resize_norm_split(_image_on(device, backing, w), rects, dst, sub, div, out)
    torch.cuda.synchronize()
    strip = dst[0] <= 256 and pitch % 4 == 0 and int(rects[:, 2].min()) >= 2
    assert last_launch()["kernel"] == ("strip" if strip else "gather")
    want = ol.oracle_crop_resize_norm_split(np.ascontiguousarray(rc.image_of(backing, w)), rects, dst, sub, div)
    _same_bits(out.cpu().numpy(), want, f"normalise:{seed}")


@pytest.mark.parametrize("seed,size,pad,dst", rc.LETTERBOX)
def test_random_letterboxed_batch_equals_the_oracle(device, seed, size, pad, dst):
    import torch
    backing, rects, bg, mul, sub = rc.letterbox_inputs(seed, size, pad)
    w = size[0]
    out = torch.full((5, dst[1], dst[0], 3), 7, dtype=torch.uint8, device=device)
    print(f"seed {seed} source {size[0]}x{size[1]} pitch {backing.shape[1]} target {dst[0]}x{dst[1]}", flush=True)
    cases.crop_resize_par_u8(_image_on(device, backing, w), rects, dst, bg, mul, sub, out)
    torch.cuda.synchronize()
    want = ol.oracle_crop_resize_par_u8(np.ascontiguousarray(rc.image_of(backing, w)), rects, dst, bg, mul, sub)
    _same_bits(out.cpu().numpy(), want, f"letterbox:{seed}")


@pytest.mark.parametrize("seed,size,pad,dst", rc.FRAMES)
def test_random_nv12_frame_equals_the_oracle(device, seed, size, pad, dst):
    import torch
    backing, scale = rc.frame_inputs(seed, size, pad)
    w, h = size
    frame = torch.from_numpy(backing).to(device)[:, :w]
    out = torch.full((3, dst[1], dst[0]), float("nan"), dtype=torch.float32, device=device)
    print(f"seed {seed} frame {w}x{h} pitch {backing.shape[1]} target {dst[0]}x{dst[1]} scale {scale}", flush=True)
    cases.nv12_rgb_resize_split(frame, w, h, dst, scale, out)
    torch.cuda.synchronize()
    want = ol.oracle_nv12_rgb_resize_split(np.ascontiguousarray(backing[:, :w]), w, h, dst, scale)
    _same_bits(out.cpu().numpy(), want, f"frame:{seed}")


def test_sweep_of_random_cases_equals_the_oracle(device):
    # 1 500 cases of random_cases.sweep_case, a few seconds; the first differing case is named
    import torch
    kernels = set()
    for i in range(1500):
        family, c = rc.sweep_case(i)
        backing, w, dst = c["backing"], c["w"], c["dst"]
        if family == 0:
            out = torch.full((8, 3, dst[1], dst[0]), float("nan"), dtype=torch.float32, device=device)
            cases.crop_resize_norm_split(_image_on(device, backing, w), c["rects"], dst, c["sub"], c["div"], out)
            want = ol.oracle_crop_resize_norm_split(np.ascontiguousarray(rc.image_of(backing, w)), c["rects"], dst, c["sub"], c["div"])
        elif family == 1:
            out = torch.full((5, dst[1], dst[0], 3), 7, dtype=torch.uint8, device=device)
            cases.crop_resize_par_u8(_image_on(device, backing, w), c["rects"], dst, c["bg"], c["mul"], c["sub"], out)
            want = ol.oracle_crop_resize_par_u8(np.ascontiguousarray(rc.image_of(backing, w)), c["rects"], dst, c["bg"], c["mul"], c["sub"])
        else:
            out = torch.full((3, dst[1], dst[0]), float("nan"), dtype=torch.float32, device=device)
            cases.nv12_rgb_resize_split(torch.from_numpy(backing).to(device)[:, :w], w, c["h"], dst, c["scale"], out)
            want = ol.oracle_nv12_rgb_resize_split(np.ascontiguousarray(backing[:, :w]), w, c["h"], dst, c["scale"])
        torch.cuda.synchronize()
        kernels.add((family, last_launch()["kernel"]))
        got = out.cpu().numpy()
        assert got.shape == want.shape and got.tobytes() == want.tobytes(), \
            f"case {i} (family {family}, source {backing.shape}, target {dst}, kernel {last_launch()['kernel']}) differs from the oracle"
    assert {(0, "strip"), (0, "gather"), (1, "gather"), (2, "gather")} <= kernels


BORDERS = [ol.BORDER_CONSTANT, ol.BORDER_REPLICATE, ol.BORDER_REFLECT, ol.BORDER_WRAP, ol.BORDER_REFLECT_101]


def test_sweep_of_random_reader_cases_equals_the_oracle(device):
    # 1 000 cases of random_cases.reader_sweep_case: Warping, Deinterlace, BorderReader (reference warping.h:42-96,
    # deinterlace.h, border_reader.h:177-327)
    import torch
    for i in range(1000):
        family, c = rc.reader_sweep_case(i)
        img = c["img"]
        src = torch.from_numpy(img).to(device)
        if family < 2:
            dst = c["dst"]
            out = torch.full((dst[1], dst[0], 3) if family == 0 else (dst[1], dst[0]), -1.0, dtype=torch.float32, device=device)
            cases.warp(src, c["matrix"], c["perspective"], dst, out)
            want = ol.oracle_warp(img, 3 if family == 0 else 1, c["matrix"], dst, c["perspective"])
        elif family == 2:
            out = torch.full(img.shape, -1.0, dtype=torch.float32, device=device)
            cases.deinterlace(src, c["mode"], out)
            want = ol.oracle_deinterlace(img, 3, c["mode"])
        else:
            shape = (c["out_h"], c["out_w"], 3) if img.ndim == 3 else (c["out_h"], c["out_w"])
            out = torch.zeros(shape, dtype=torch.uint8 if img.dtype == np.uint8 else torch.float32, device=device)
            cases.pad(src, BORDERS[c["border"]], c["left"], c["top"], out, value=c["value"])
            want = ol.oracle_pad(img, BORDERS[c["border"]], c["left"], c["top"], c["out_w"], c["out_h"], value=c["value"])
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        assert got.shape == want.shape and got.tobytes() == want.tobytes(), \
            f"case {i} (family {family}, source {img.shape}) differs from the oracle: " + str({k: v for k, v in c.items() if k != "img"})


def test_sweep_of_random_chain_cases_equals_the_oracle(device):
    # 1 200 cases of random_cases.chain_sweep_case: the float chain, the horizontal batch, the two conditional batches
    import torch
    for i in range(1200):
        family, c = rc.chain_sweep_case(i)
        if family == 0:
            w, src = c["w"], c["src"]
            o = torch.full((src.shape[0], w + c["out_pad"]), 5.0, dtype=torch.float32, device=device)
            cases.add_mul_chain(torch.from_numpy(src).to(device)[:, :w], c["n"], 0.5, 1.0001, o[:, :w], tf=c["tf"])
            torch.cuda.synchronize()
            got = o.cpu().numpy()
            want = ol.oracle_add_mul_chain(np.ascontiguousarray(src[:, :w]), c["n"], 0.5, 1.0001)
            same = got[:, :w].tobytes() == want.tobytes() and bool((got[:, w:] == 5.0).all())
        elif family == 1:
            w, h = c["w"], c["backings"][0].shape[0]
            srcs = [_image_on(device, b, w) for b in c["backings"]]
            outs = [torch.zeros((h, w, 3), dtype=torch.uint8, device=device) for _ in range(4)]
            cases.batch_muladd_sat(srcs, c["mul"], c["add"], outs)
            torch.cuda.synchronize()
            want = ol.oracle_batch_muladd_sat([np.ascontiguousarray(rc.image_of(b, w)) for b in c["backings"]], c["mul"], c["add"])
            same = np.stack([o.cpu().numpy() for o in outs]).tobytes() == np.stack(want).tobytes()
        elif family == 2:
            dst = c["dst"]
            out = torch.full((8, 3, dst[1], dst[0]), 7.0, dtype=torch.float32, device=device)
            cases.crop_resize_default_norm_split(torch.from_numpy(c["img"]).to(device), c["rects"], dst, c["used"], c["default"],
                                                 c["sub"], c["div"], out)
            torch.cuda.synchronize()
            want = ol.oracle_crop_resize_default_norm_split(c["img"], c["rects"], dst, c["used"], c["default"], c["sub"], c["div"])
            same = out.cpu().numpy().tobytes() == want.tobytes()
        else:
            h, w = c["imgs"][0].shape[:2]
            out = torch.zeros((4, h, w, 3), dtype=torch.float32, device=device)
            cases.batch_default_cast_mul([torch.from_numpy(s).to(device) for s in c["imgs"]], c["active"], (7, 200, 33), (0.5, 2.0, 1.25), out)
            torch.cuda.synchronize()
            same = out.cpu().numpy().tobytes() == ol.oracle_batch_default_cast_mul(c["imgs"], c["active"], (7, 200, 33), (0.5, 2.0, 1.25)).tobytes()
        assert same, f"case {i} (family {family}) differs from the oracle: " + str({k: v for k, v in c.items() if not isinstance(v, (np.ndarray, list))})
