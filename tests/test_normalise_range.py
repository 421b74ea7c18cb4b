"""(x - mean) / std after a read that can only deliver bounded values: the host proves that every element reaching the
division is zero or lies in the range the short division sequences need, and the device then skips its per-element
range test (fkd::Chain::finalize).  Here: when the proof is granted and when not (CPU), and that results stay bit for bit
those of IEEE division in all those cases, zeros included (GPU, against the CPU oracle)."""
import numpy as np
import pytest

import oracle_lib as ol
import fkl_cases as cases
import workloads as wl

PROVEN = 4


def test_proof_is_granted_for_the_benchmark_constants():
    mode = cases.normalise_mode(0, wl.C3_MEAN, wl.C3_STD)
    assert mode & PROVEN and (mode & 3) in (1, 2)


@pytest.mark.parametrize("kind,sub,div,want", [
    (0, (100.0, 100.0, 100.0), (2.0, 3.0, 5.0), True),
    (0, (100.0, 1e-9, 100.0), (2.0, 3.0, 5.0), False),        # a mean below 2^-20: differences could be tiny
    (0, (100.0, 0.0, 100.0), (2.0, 3.0, 5.0), False),
    (0, (100.0, 1e20, 100.0), (2.0, 3.0, 5.0), False),        # above 2^59
    (0, (100.0, 100.0, 100.0), (2.0, -3.0, 5.0), False),      # a zero difference over a negative divisor is -0
    (0, (100.0, 100.0, 100.0), (2.0, 1e-30, 5.0), False),     # divisor outside the short sequences' range
    (0, (-100.0, 100.0, -0.5), (2.0, 3.0, 5.0), True),
    (1, (100.0, 100.0, 100.0), (2.0, 3.0, 5.0), False),       # float pixels: infinities and NaNs may arrive
    (2, (100.0, 100.0, 100.0), (2.0, 3.0, 5.0), False),       # letterbox colour is a run-time value
])
def test_when_the_proof_is_granted(kind, sub, div, want):
    assert bool(cases.normalise_mode(kind, sub, div) & PROVEN) == want


def _run(device, src, rects, dst, sub, div):
    import torch
    out = torch.full((len(rects), 3, dst[1], dst[0]), 7.0, dtype=torch.float32, device=device)
    cases.crop_resize_norm_split(torch.from_numpy(src).to(device), rects, dst, np.array(sub, np.float32), np.array(div, np.float32), out)
    torch.cuda.synchronize()
    return out.cpu().numpy()


@pytest.mark.gpu
@pytest.mark.parametrize("sub,div", [
    ((100.0, 100.0, 100.0), (2.0, 3.0, 5.0)),           # proven; the constant image gives zeros everywhere
    ((100.0, 100.0, 100.0), (2.0, -3.0, 5.0)),          # refused: -0 in channel 1
    ((100.0, 1e-9, 100.0), (2.0, 3.0, 5.0)),            # refused
    ((37.0, 200.0, 0.5), (0.229 * 255, 0.224 * 255, 0.225 * 255)),
])
def test_zero_differences_and_refused_constants(device, sub, div):
    rng = np.random.RandomState(5)
    src = np.full((120, 160, 3), 100, np.uint8)
    src[60:, :, :] = rng.randint(0, 256, (60, 160, 3))            # lower half random, upper half constant
    src[60:, ::3, 0] = 37                                            # exact hits of a mean in the random half
    rects = [(int(rng.randint(0, 100)), int(rng.randint(0, 70)), 32 + int(rng.randint(0, 28)), 24 + int(rng.randint(0, 26))) for _ in range(64)]
    rects[0] = (5, 3, 32, 24)          # factor 1 inside the constant half: every difference is exactly zero
    rects[1] = (0, 60, 64, 48)         # factor 2 in the random half
    rects[2] = (3, 66, 32, 24)         # factor 1 in the random half: the pixels themselves, some equal to a mean
    rects = np.array(rects, np.int32)
    got = _run(device, src, rects, (32, 24), sub, div)
    want = ol.oracle_crop_resize_norm_split(src, rects, (32, 24), np.array(sub, np.float32), np.array(div, np.float32))
    assert got.tobytes() == want.tobytes()
    if sub[0] == 100.0:
        zeros = got[0, 2]              # channel order is swapped: output channel 2 is source channel 0
        assert (zeros.view(np.uint32) == 0).all()
