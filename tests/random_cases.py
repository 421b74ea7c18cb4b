"""Seeded random cases of the three resizing chains, shared by the GPU tests (tests/test_gpu_random_batches.py), the CPU
test that pins the oracle on them (tests/test_oracle_random_batches.py) and the script that writes the reference's
digests of them (tests/golden/make_random_batches_golden.py).  Every function returns host arrays only."""
import hashlib

import numpy as np


def digest(a) -> str:
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def rects(rng, n, w, h, least):
    out = []
    for i in range(n):
        kind = i % 8
        if kind == 0:
            cw, ch = min(w, least + rng.randint(0, 3)), min(h, 1 + rng.randint(0, 3))  # a few pixels
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


# crop -> bilinear resize -> channel swap -> (x - mean) / std -> three float planes per crop
# (seed, batch, source w x h, pitch padding in bytes, narrowest crop, target w x h)
NORMALISE = [
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
    (13, 8, (512, 300), 0, 2, (260, 4)),    # wider than the strip form of the kernel takes
]


def normalise_inputs(seed, batch, size, pad, least):
    """backing (h, pitch) u8, rects (batch, 4), sub (3), div (3); the image is backing[:, :w*3] seen as (h, w, 3)."""
    rng = np.random.RandomState(1000 + seed)
    w, h = size
    backing = rng.randint(0, 256, (h, w * 3 + pad)).astype(np.uint8)
    r = rects(rng, batch, w, h, least)
    sub = rng.uniform(-20, 140, 3).astype(np.float32)
    # 58.395 takes the two-instruction division, 0.7 the five-instruction one, a denormal-range divisor the generic one
    div = np.array([[58.395, 57.12, 57.375], [0.7, 3.0, 1e-39], [1.0, 255.0, 0.1]][seed % 3], np.float32)
    return backing, r, sub, div


# crop -> bilinear resize that keeps the aspect ratio (bands of the background colour) -> Mul -> Sub -> SaturateCast ->
# packed uchar3 tensor, five planes.  (seed, source w x h, pitch padding, target w x h)
LETTERBOX = [
    (1, (97, 61), 0, (128, 64)),
    (2, (97, 61), 1, (31, 17)),
    (3, (200, 40), 0, (40, 200)),
    (4, (33, 150), 3, (64, 9)),
    (5, (64, 64), 0, (1, 1)),
    (6, (300, 200), 0, (260, 70)),
    (7, (12, 7), 0, (50, 50)),
]


def letterbox_inputs(seed, size, pad):
    rng = np.random.RandomState(2000 + seed)
    w, h = size
    backing = rng.randint(0, 256, (h, w * 3 + pad)).astype(np.uint8)
    r = rects(rng, 8, w, h, 1)[[0, 1, 4, 5, 6]]
    bg = rng.uniform(0, 255, 3).astype(np.float32)
    mul = rng.uniform(0.25, 3.0, 3).astype(np.float32)
    sub = rng.uniform(-50, 200, 3).astype(np.float32)
    return backing, r, bg, mul, sub


# NV12 -> RGB -> bilinear resize -> Mul -> three float planes.  (seed, frame w x h, pitch padding, target w x h)
FRAMES = [
    (1, (64, 48), 0, (37, 19)),
    (2, (66, 50), 2, (66, 50)),
    (3, (130, 34), 0, (65, 17)),
    (4, (34, 130), 6, (300, 5)),
    (5, (2, 2), 0, (9, 9)),
    (6, (256, 128), 0, (255, 127)),
    (7, (40, 30), 0, (1, 1)),
]


def frame_inputs(seed, size, pad):
    rng = np.random.RandomState(3000 + seed)
    w, h = size
    backing = rng.randint(0, 256, (h * 3 // 2, w + pad)).astype(np.uint8)
    scale = float(np.float32(rng.uniform(0.001, 2.0)))
    return backing, scale


def image_of(backing, w):
    """The (h, w, 3) image at the start of every row of `backing`, as a view with the backing's pitch."""
    h, pitch = backing.shape
    return np.lib.stride_tricks.as_strided(backing, (h, w, 3), (pitch, 3, 1), writeable=False)


def sweep_case(i):
    """Case i of an open-ended seeded sweep over the three chains: (family, arguments) with family 0 normalise (batch 8),
    1 letterbox, 2 NV12 frame; sizes from one or two pixels to a few hundred, pitches of every alignment, target sizes
    that take either form of the bilinear kernel, whole and fractional factors, divisors of every division sequence."""
    rng = np.random.RandomState(50000 + i)
    w, h = int(rng.randint(2, 400)), int(rng.randint(1, 300))
    pad = int(rng.choice([0, 0, 1, 2, 3, 4]))
    family = i % 3
    if family == 0:
        dst = (int(rng.choice([rng.randint(1, 300), 32 * rng.randint(1, 9), 224])), int(rng.randint(1, 40)))
        backing = rng.randint(0, 256, (h, w * 3 + pad)).astype(np.uint8)
        r = rects(rng, 8, w, h, min(int(rng.choice([1, 2])), w))
        sub = rng.uniform(-20, 140, 3).astype(np.float32)
        div = rng.choice([58.395, 57.12, 57.375, 0.7, 3.0, 1.0, 255.0, 0.1, 1e-39, 7.0, 1.5e10], 3).astype(np.float32)
        return family, dict(backing=backing, w=w, rects=r, dst=dst, sub=sub, div=div)
    if family == 1:
        dst = (int(rng.randint(1, 300)), int(rng.randint(1, 80)))
        backing = rng.randint(0, 256, (h, w * 3 + pad)).astype(np.uint8)
        r = rects(rng, 8, w, h, 1)[[0, 1, 4, 5, 6]]
        bg = rng.uniform(0, 255, 3).astype(np.float32)
        mul = rng.uniform(0.25, 3.0, 3).astype(np.float32)
        sub = rng.uniform(-50, 200, 3).astype(np.float32)
        return family, dict(backing=backing, w=w, rects=r, dst=dst, bg=bg, mul=mul, sub=sub)
    w, h = 2 * int(rng.randint(1, 200)), 2 * int(rng.randint(1, 120))
    pad = 2 * int(rng.randint(0, 4))
    k = int(rng.choice([0, 1, 2, 3]))
    dst = (w // k, h // k) if k in (1, 2) else (int(rng.randint(1, 300)), int(rng.randint(1, 100)))
    backing = rng.randint(0, 256, (h * 3 // 2, w + pad)).astype(np.uint8)
    scale = float(np.float32(rng.uniform(0.001, 2.0)))
    return family, dict(backing=backing, w=w, h=h, dst=dst, scale=scale)


def reader_sweep_case(i):
    """Case i of a seeded sweep over the read-back operations either side of the path: family 0 Warping of a uchar3 image,
    1 Warping of a float image (affine or perspective, rotation by any angle, scale 0.3 to 3, shifts that move part of the
    target outside the source), 2 Deinterlace of a uchar3 image (all three modes), 3 BorderReader under a Crop that leaves
    the image by up to three image sizes (all five border types, uchar3 or float)."""
    import math
    rng = np.random.RandomState(70000 + i)
    family = i % 4
    w, h = int(rng.randint(2, 300)), int(rng.randint(2, 200))
    if family < 2:
        perspective = bool(rng.randint(0, 2))
        angle, s = rng.uniform(-math.pi, math.pi), rng.uniform(0.3, 3.0)
        m = [[s * math.cos(angle), -s * math.sin(angle), rng.uniform(-50, 50)], [s * math.sin(angle), s * math.cos(angle), rng.uniform(-50, 50)]]
        if perspective:
            m.append([rng.uniform(-1e-3, 1e-3), rng.uniform(-1e-3, 1e-3), 1.0])
        dst = (int(rng.randint(1, 300)), int(rng.randint(1, 120)))
        if family == 0:
            img = rng.randint(0, 256, (h, w, 3)).astype(np.uint8)
        else:
            img = (rng.random_sample((h, w)) * 200 - 100).astype(np.float32)
        return family, dict(img=img, matrix=m, perspective=perspective, dst=dst)
    if family == 2:
        mode = int(rng.randint(1, 4))
        return family, dict(img=rng.randint(0, 256, (h, w, 3)).astype(np.uint8), mode=mode)
    border = int(rng.randint(0, 5))
    left, top = int(rng.randint(-w // 2, 3 * w)), int(rng.randint(-h // 2, 3 * h))
    out_w, out_h = int(rng.randint(1, 400)), int(rng.randint(1, 150))
    if rng.randint(0, 2):
        img, value = rng.randint(0, 256, (h, w, 3)).astype(np.uint8), (9, 8, 7)
    else:
        img, value = (rng.random_sample((h, w)) * 100 - 50).astype(np.float32), (-1.5,)
    return family, dict(img=img, border=border, left=left, top=top, out_w=out_w, out_h=out_h, value=value)


def color_sweep_case(i, y2r, r2y, resize_formats):
    """Case i of a seeded sweep over the pixel-format chains: family 0 ReadYUV -> ConvertYUVToRGB, 1 ConvertRGBToYUV ->
    WriteYUV (odd sizes leave the last chroma block to one column or row), 2 ReadYUV under a bilinear resize.  `y2r`, `r2y`:
    the (pixel format, range, primaries) combinations the case driver has chains for; `resize_formats`: pixel formats."""
    import oracle_lib as ol
    rng = np.random.RandomState(90000 + i)
    family = i % 3

    def frame(pf, w, h, pad):
        rows, cols = ol.frame_shape(pf, w, h)
        if ol.PF_WIDE[pf]:
            return rng.randint(0, 1024, (rows, cols + pad)).astype(np.uint16)
        return rng.randint(0, 256, (rows, cols + pad)).astype(np.uint8)

    if family == 0:
        pf, cr, cp = y2r[int(rng.randint(0, len(y2r)))]
        w, h = 2 * int(rng.randint(1, 400)), 2 * int(rng.randint(1, 100))
        return family, dict(pf=pf, cr=cr, cp=cp, w=w, h=h, frame=frame(pf, w, h, int(rng.randint(0, 6))))
    if family == 1:
        pf, cr, cp = r2y[int(rng.randint(0, len(r2y)))]
        wide = ol.PF_WIDE[pf]
        w, h = int(rng.randint(1, 500)), int(rng.randint(1, 120))
        if pf in (ol.PF_Y210, ol.PF_UYVY):
            w += w & 1
        rgb = rng.randint(0, 1024 if wide else 256, (h, w, 3)).astype(np.uint16 if wide else np.uint8)
        rows, cols = ol.frame_shape(pf, w + (w & 1), h + (h & 1))
        if pf in (ol.PF_NV12, ol.PF_NV21, ol.PF_P010, ol.PF_P210):
            rows = h + (h + 1) // 2 if pf != ol.PF_P210 else 2 * h     # chroma rows start right after `height` luma rows
        return family, dict(pf=pf, cr=cr, cp=cp, rgb=rgb, start=np.full((rows, cols + 4), 9, rgb.dtype))
    pf = resize_formats[int(rng.randint(0, len(resize_formats)))]
    w, h = 2 * int(rng.randint(1, 200)), 2 * int(rng.randint(1, 100))
    dst = (int(rng.randint(1, 300)), int(rng.randint(1, 100)))
    return family, dict(pf=pf, w=w, h=h, dst=dst, frame=frame(pf, w, h, 0))


def chain_sweep_case(i):
    """Case i of a seeded sweep over the rest of the benchmark chains: family 0 the float chain of N alternating Add / Mul
    (N in 1, 2, 3, 10, 50, 100; with and without the thread-fusion spelling), 1 four uchar3 images with their own Mul and Add
    in one launch, 2 the normalising chain on eight crops of which only the first `used` are read, 3 an array of four images
    of which only the first `active` are read.  Sizes from 1 x 1 to 700 x 40, padded pitches."""
    rng = np.random.RandomState(130000 + i)
    family = i % 4
    w, h = int(rng.randint(1, 700)), int(rng.randint(1, 40))
    if family == 0:
        n = int(rng.choice([1, 2, 3, 10, 50, 100]))
        pads = (int(rng.randint(0, 4)), int(rng.randint(0, 4)))
        src = (rng.random_sample((h, w + pads[0])) * 2 - 1).astype(np.float32)
        return family, dict(n=n, w=w, src=src, out_pad=pads[1], tf=int(rng.randint(0, 2)))
    if family == 1:
        pad = int(rng.randint(0, 4))
        backings = [rng.randint(0, 256, (h, w * 3 + pad)).astype(np.uint8) for _ in range(4)]
        return family, dict(w=w, backings=backings, mul=rng.uniform(0.5, 2, (4, 3)).astype(np.float32),
                            add=rng.uniform(-64, 64, (4, 3)).astype(np.float32))
    if family == 2:
        w = max(w, 2)
        used = int(rng.randint(0, 9))
        dst = (int(rng.randint(1, 200)), int(rng.randint(1, 30)))
        img = rng.randint(0, 256, (h, w, 3)).astype(np.uint8)
        r = rects(rng, 8, w, h, 1)
        default = rng.uniform(-5, 300, 3).astype(np.float32)
        sub = rng.uniform(0, 130, 3).astype(np.float32)
        div = rng.choice([58.395, 57.12, 0.7, 3.0, 255.0], 3).astype(np.float32)
        return family, dict(img=img, rects=r, dst=dst, used=used, default=default, sub=sub, div=div)
    active = int(rng.randint(0, 5))
    return family, dict(active=active, imgs=[rng.randint(0, 256, (h, w, 3)).astype(np.uint8) for _ in range(4)])
