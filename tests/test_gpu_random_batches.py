"""Seeded random batches of crop -> bilinear resize -> channel swap -> (x - mean) / std -> planar float, GPU against the C
oracle, bit for bit: source pitches that are and are not a multiple of four, crops from one pixel to the whole image
(planes up to 256 wide whose source rows share their alignment and whose crops have two columns take the strip form of
the kernel, all others the tile form), enlarging and reducing in the same batch, divisors that take each of the three
division sequences.
Reference path: FK/algorithms/image_processing/resize.h:86-123, interpolation.h:70-104, crop.h, memory_operations.h:181-212."""
import numpy as np
import pytest

import fkl_cases as cases
import oracle_lib as ol
from fusedkernellibrary_amd import last_launch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def device():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


def _rects(rng, n, w, h, least):
    out = []
    for i in range(n):
        kind = i % 8
        if kind == 0:
            cw, ch = min(w, least + rng.randint(0, 3)), 1 + rng.randint(0, 3)  # a few pixels
        elif kind == 1:
            cw, ch = w, h                                                   # the whole image
        elif kind == 2:
            cw, ch = w, 1 + rng.randint(0, h)                               # full width
        elif kind == 3:
            cw, ch = rng.randint(least, w + 1), h                           # full height
        else:
            cw, ch = rng.randint(least, w + 1), 1 + rng.randint(0, h)
        x = rng.randint(0, w - cw + 1)
        y = rng.randint(0, h - ch + 1)
        if kind == 4:
            x, y = w - cw, h - ch                                           # ends in the image's last pixel
        out.append((x, y, cw, ch))
    return np.array(out, np.int32)


# (seed, batch, source w x h, pitch padding in bytes, narrowest crop, target w x h)
CASES = [
    (1, 8, (97, 61), 1, 2, (32, 5)),        # pitch 292
    (2, 8, (97, 61), 0, 1, (64, 9)),        # pitch 291: rows of every alignment
    (3, 64, (131, 77), 3, 2, (96, 7)),      # pitch 396
    (4, 8, (40, 33), 0, 2, (224, 3)),
    (5, 8, (97, 61), 1, 2, (17, 11)),
    (6, 64, (131, 77), 1, 1, (50, 6)),
    (7, 8, (300, 9), 0, 2, (130, 13)),
    (8, 8, (9, 200), 1, 2, (33, 31)),
    (9, 8, (64, 64), 0, 2, (1, 1)),
    (10, 64, (257, 129), 1, 2, (160, 10)),  # pitch 772
    (11, 8, (5, 4), 1, 1, (64, 8)),
    (12, 8, (512, 300), 0, 2, (256, 4)),
    (13, 8, (512, 300), 0, 2, (260, 4)),    # wider than the strip form takes
]


@pytest.mark.parametrize("seed,batch,size,pad,least,dst", CASES)
def test_random_batch_equals_the_oracle(device, seed, batch, size, pad, least, dst):
    import torch
    rng = np.random.RandomState(1000 + seed)
    w, h = size
    pitch = w * 3 + pad
    backing = torch.from_numpy(rng.randint(0, 256, (h, pitch)).astype(np.uint8)).to(device)
    src = backing[:, :w * 3].view(h, w, 3) if pad == 0 else torch.as_strided(backing, (h, w, 3), (pitch, 3, 1))
    host = backing.cpu().numpy()[:, :w * 3].reshape(h, w, 3)
    rects = _rects(rng, batch, w, h, least)
    sub = rng.uniform(-20, 140, 3).astype(np.float32)
    # 58.395 takes the two-instruction division, 0.7 the five-instruction one, a denormal-range divisor the generic one
    div = np.array([[58.395, 57.12, 57.375], [0.7, 3.0, 1e-39], [1.0, 255.0, 0.1]][seed % 3], np.float32)
    out = torch.full((batch, 3, dst[1], dst[0]), float("nan"), dtype=torch.float32, device=device)
    print(f"seed {seed} batch {batch} source {w}x{h} pitch {pitch} target {dst[0]}x{dst[1]}", flush=True)
    cases.crop_resize_norm_split(src, rects, dst, sub, div, out)
    torch.cuda.synchronize()
    strip = dst[0] <= 256 and pitch % 4 == 0 and int(rects[:, 2].min()) >= 2
    assert last_launch()["kernel"] == ("strip" if strip else "gather")
    want = ol.oracle_crop_resize_norm_split(np.ascontiguousarray(host), rects, dst, sub, div)
    got = out.cpu().numpy()
    assert got.shape == want.shape
    same = got.view(np.uint32) == want.view(np.uint32)
    assert same.all(), f"{(~same).sum()} of {same.size} values differ; first at {np.argwhere(~same)[0]}"


# (seed, source w x h, pitch padding, target w x h): crop -> bilinear resize that keeps the aspect ratio (bands of the
# background colour) -> Mul -> Sub -> SaturateCast -> packed uchar3 tensor, five planes.
LETTERBOX = [
    (1, (97, 61), 0, (128, 64)),
    (2, (97, 61), 1, (31, 17)),
    (3, (200, 40), 0, (40, 200)),
    (4, (33, 150), 3, (64, 9)),
    (5, (64, 64), 0, (1, 1)),
    (6, (300, 200), 0, (260, 70)),
    (7, (12, 7), 0, (50, 50)),
]


@pytest.mark.parametrize("seed,size,pad,dst", LETTERBOX)
def test_random_letterboxed_batch_equals_the_oracle(device, seed, size, pad, dst):
    import torch
    rng = np.random.RandomState(2000 + seed)
    w, h = size
    pitch = w * 3 + pad
    backing = torch.from_numpy(rng.randint(0, 256, (h, pitch)).astype(np.uint8)).to(device)
    src = backing.view(h, w, 3) if pad == 0 else torch.as_strided(backing, (h, w, 3), (pitch, 3, 1))
    host = np.ascontiguousarray(backing.cpu().numpy()[:, :w * 3].reshape(h, w, 3))
    rects = _rects(rng, 8, w, h, 1)[[0, 1, 4, 5, 6]]
    bg = rng.uniform(0, 255, 3).astype(np.float32)
    mul = rng.uniform(0.25, 3.0, 3).astype(np.float32)
    sub = rng.uniform(-50, 200, 3).astype(np.float32)
    out = torch.full((5, dst[1], dst[0], 3), 7, dtype=torch.uint8, device=device)
    print(f"seed {seed} source {w}x{h} pitch {pitch} target {dst[0]}x{dst[1]}", flush=True)
    cases.crop_resize_par_u8(src, rects, dst, bg, mul, sub, out)
    torch.cuda.synchronize()
    want = ol.oracle_crop_resize_par_u8(host, rects, dst, bg, mul, sub)
    got = out.cpu().numpy()
    assert got.shape == want.shape
    assert got.tobytes() == want.tobytes(), f"{(got != want).sum()} of {got.size} bytes differ; first at {np.argwhere(got != want)[0]}"


# (seed, frame w x h, pitch padding, target w x h): NV12 -> RGB -> bilinear resize -> Mul -> three float planes.
FRAMES = [
    (1, (64, 48), 0, (37, 19)),
    (2, (66, 50), 2, (66, 50)),
    (3, (130, 34), 0, (65, 17)),
    (4, (34, 130), 6, (300, 5)),
    (5, (2, 2), 0, (9, 9)),
    (6, (256, 128), 0, (255, 127)),
    (7, (40, 30), 0, (1, 1)),
]


@pytest.mark.parametrize("seed,size,pad,dst", FRAMES)
def test_random_nv12_frame_equals_the_oracle(device, seed, size, pad, dst):
    import torch
    rng = np.random.RandomState(3000 + seed)
    w, h = size
    backing = torch.from_numpy(rng.randint(0, 256, (h * 3 // 2, w + pad)).astype(np.uint8)).to(device)
    frame = backing[:, :w]
    scale = float(np.float32(rng.uniform(0.001, 2.0)))
    out = torch.full((3, dst[1], dst[0]), float("nan"), dtype=torch.float32, device=device)
    print(f"seed {seed} frame {w}x{h} pitch {w + pad} target {dst[0]}x{dst[1]} scale {scale}", flush=True)
    cases.nv12_rgb_resize_split(frame, w, h, dst, scale, out)
    torch.cuda.synchronize()
    want = ol.oracle_nv12_rgb_resize_split(np.ascontiguousarray(frame.cpu().numpy()), w, h, dst, scale)
    got = out.cpu().numpy()
    assert got.shape == want.shape
    same = got.view(np.uint32) == want.view(np.uint32)
    assert same.all(), f"{(~same).sum()} of {same.size} values differ; first at {np.argwhere(~same)[0]}"
