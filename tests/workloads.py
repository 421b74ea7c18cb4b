"""Deterministic synthetic inputs for the five benchmark configurations.

Every value is a raw output of the 32-bit Mersenne Twister (the generator C++ calls
``std::mt19937``), seeded with a small integer, consumed in row-major order (y, x, channel):

* byte            = gen() & 0xFF
* float in [-1,1) = (gen() >> 8) * 2**-23 - 1
* float in [a,b)  = a + ((gen() >> 8) * 2**-24) * (b - a)        (all in binary32)

``numpy.random.RandomState(seed)`` seeds the same generator the same way (init_genrand) and
``randint(0, 2**32, dtype=uint32)`` hands out its raw outputs one per element, so these arrays can be
reproduced from C++ with ``std::mt19937 gen(seed)``.
"""
from __future__ import annotations

import numpy as np

# README crop rectangles (x, y, w, h) of configuration 1.
C1_RECTS = np.array(
    [[300, 125, 60, 40], [400, 125, 60, 40], [530, 270, 130, 140], [560, 115, 100, 35], [572, 196, 40, 15]],
    dtype=np.int32,
)
C3_MEAN = (np.array([0.485, 0.456, 0.406], dtype=np.float32) * np.float32(255.0)).astype(np.float32)
C3_STD = (np.array([0.229, 0.224, 0.225], dtype=np.float32) * np.float32(255.0)).astype(np.float32)


class RawMT:
    """Raw std::mt19937 stream."""

    def __init__(self, seed: int):
        self._rs = np.random.RandomState(int(seed))

    def u32(self, n: int) -> np.ndarray:
        return self._rs.randint(0, 2**32, size=int(n), dtype=np.uint32)

    def bytes(self, n: int) -> np.ndarray:
        out = np.empty(int(n), dtype=np.uint8)
        step = 1 << 24
        for i in range(0, int(n), step):
            m = min(step, int(n) - i)
            out[i : i + m] = (self.u32(m) & np.uint32(0xFF)).astype(np.uint8)
        return out

    def unit_floats(self, n: int) -> np.ndarray:
        u = (self.u32(n) >> np.uint32(8)).astype(np.float32)
        return u * np.float32(2.0**-23) - np.float32(1.0)

    def range_floats(self, n: int, a: float, b: float) -> np.ndarray:
        u = (self.u32(n) >> np.uint32(8)).astype(np.float32)
        return np.float32(a) + (u * np.float32(2.0**-24)) * (np.float32(b) - np.float32(a))


def config1(width: int = 3840, height: int = 2160, seed: int = 1):
    """README chain: uchar3 source + 5 crops -> 128x64x5 uchar3 (PRESERVE_AR)."""
    src = RawMT(seed).bytes(width * height * 3).reshape(height, width, 3)
    return {
        "src": src,
        "rects": C1_RECTS.copy(),
        "dst": (128, 64),
        "bg": np.zeros(3, np.float32),
        "mul": np.full(3, 2.0, np.float32),
        "sub": np.full(3, 128.0, np.float32),
    }


def config2(width: int = 3840, height: int = 2160, seed: int = 2):
    """Pure vertical fusion: float image, N alternating Add(0.5f)/Mul(1.0001f)."""
    src = RawMT(seed).unit_floats(width * height).reshape(height, width)
    return {"src": src, "add": np.float32(0.5), "mul": np.float32(1.0001), "n_ops": (1, 10, 50, 100),
            "n_ops_sweep": (1, 10, 20, 30, 40, 50, 100)}       # the benchmark's sweep for the instruction-vs-bandwidth crossover


def config3_rects(batch: int = 64, width: int = 1920, height: int = 1080, seed: int = 33,
                  min_side: int = 64, span: int = 449) -> np.ndarray:
    g = RawMT(seed)
    rects = np.zeros((batch, 4), dtype=np.int32)
    for i in range(batch):
        r = g.u32(4).astype(np.int64)
        x = int(r[0] % (width - min_side + 1))
        y = int(r[1] % (height - min_side + 1))
        w = min(min_side + int(r[2] % span), width - x)
        h = min(min_side + int(r[3] % span), height - y)
        rects[i] = (x, y, w, h)
    return rects


def config3(batch: int = 64, width: int = 1920, height: int = 1080, dst: int = 224, seed: int = 3,
            rect_seed: int = 33, min_side: int = 64, span: int = 449):
    """DNN preprocessing: BGR uchar3 source, `batch` crops -> dst x dst, BGR->RGB, (x-mean)/std, planar float."""
    src = RawMT(seed).bytes(width * height * 3).reshape(height, width, 3)
    rects = config3_rects(batch, width, height, rect_seed, min_side, span)
    return {"src": src, "rects": rects, "dst": (dst, dst), "sub": C3_MEAN.copy(), "div": C3_STD.copy()}


def config3_union_pixels(rects: np.ndarray, width: int, height: int) -> int:
    """Distinct source pixels covered by the union of the crop rectangles."""
    mask = np.zeros((height, width), dtype=bool)
    for x, y, w, h in rects:
        mask[y : y + h, x : x + w] = True
    return int(mask.sum())


def config4(batch: int = 100, width: int = 1920, height: int = 1080, seed: int = 4, param_seed: int = 44):
    """Horizontal fusion: `batch` independent uchar3 images with per-image Mul in [0.5,2) and Add in [-64,64)."""
    g = RawMT(seed)
    srcs = [g.bytes(width * height * 3).reshape(height, width, 3) for _ in range(batch)]
    p = RawMT(param_seed)
    mul = np.zeros((batch, 3), np.float32)
    add = np.zeros((batch, 3), np.float32)
    for i in range(batch):
        mul[i] = p.range_floats(3, 0.5, 2.0)
        add[i] = p.range_floats(3, -64.0, 64.0)
    return {"srcs": srcs, "mul": mul, "add": add}


def config5(width: int = 3840, height: int = 2160, dst=(1920, 1080), seed: int = 5):
    """Video frame: NV12 (Y plane, then interleaved UV plane, one buffer of height*3/2 rows)."""
    g = RawMT(seed)
    y = g.bytes(width * height).reshape(height, width)
    uv = g.bytes(width * (height // 2)).reshape(height // 2, width)
    return {"nv12": np.ascontiguousarray(np.concatenate([y, uv], axis=0)), "width": width, "height": height,
            "dst": tuple(dst), "scale": np.float32(1.0) / np.float32(255.0)}
