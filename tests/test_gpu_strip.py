"""The strip form of the bilinear kernel (narrow planar outputs: a workgroup owns 8 whole rows of a plane, half a wave
one row) against the oracle and against the tile form on the same inputs.  fklhip_strip_form(0) switches the strip form
off for the launches that follow, so one process runs both."""
import numpy as np
import pytest

import fkl_cases as cases
import oracle_lib as ol
import workloads as wl
from fusedkernellibrary_amd import last_launch, lib

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def device():
    import torch
    return torch.device("cuda:0")


class strip_switched:
    def __init__(self, on):
        self.value = 1 if on else 0

    def __enter__(self):
        self.old = lib().fklhip_strip_form(self.value)

    def __exit__(self, *exc):
        lib().fklhip_strip_form(self.old)


def _c3(src, rects, dst, sub, div, device):
    import torch
    out = torch.full((len(rects), 3, dst[1], dst[0]), -7.0, dtype=torch.float32, device=device)
    cases.crop_resize_norm_split(src, rects, dst, sub, div, out)
    torch.cuda.synchronize()
    return out.cpu().numpy()


def _rects(rng, n, w, h, lo, hi):
    out = []
    for _ in range(n):
        rw, rh = int(rng.randint(lo, hi + 1)), int(rng.randint(lo, hi + 1))
        rw, rh = min(rw, w), min(rh, h)
        out.append((int(rng.randint(0, w - rw + 1)), int(rng.randint(0, h - rh + 1)), rw, rh))
    return np.array(out, np.int32)


@pytest.mark.parametrize("dst", [(224, 224), (1, 1), (31, 9), (32, 8), (33, 7), (100, 50), (250, 3), (256, 17), (2, 300)])
def test_both_forms_agree_with_the_oracle(device, dst):
    import torch
    rng = np.random.RandomState(1000 + dst[0])
    w, h = 640, 360                                   # pitch 1920: rows share their alignment
    img = rng.randint(0, 256, (h, w, 3)).astype(np.uint8)
    rects = _rects(rng, 8, w, h, 2, 330)              # up- and downscaling planes in one launch
    rects[0] = (0, 0, w, h)
    rects[1] = (w - 5, h - 3, 5, 3)                   # the image's last rows and columns, strongly upscaled
    rects[2] = (0, h - 2, 300, 2)
    rects[3] = (w - 2, 0, 2, 200)
    src = torch.from_numpy(img).to(device)
    want = ol.oracle_crop_resize_norm_split(img, rects, dst, wl.C3_MEAN, wl.C3_STD)
    with strip_switched(True):
        strip = _c3(src, rects, dst, wl.C3_MEAN, wl.C3_STD, device)
        ll = last_launch()
        assert ll["kernel"] == "strip" and ll["grid"] == [(dst[1] + 7) // 8, 1, 8]
    with strip_switched(False):
        tiles = _c3(src, rects, dst, wl.C3_MEAN, wl.C3_STD, device)
        assert last_launch()["kernel"] == "gather"
    assert strip.tobytes() == want.tobytes()
    assert tiles.tobytes() == want.tobytes()


def test_wider_outputs_keep_the_tile_form(device):
    import torch
    rng = np.random.RandomState(5)
    img = rng.randint(0, 256, (120, 400, 3)).astype(np.uint8)
    rects = _rects(rng, 8, 400, 120, 20, 110)
    src = torch.from_numpy(img).to(device)
    got = _c3(src, rects, (257, 16), wl.C3_MEAN, wl.C3_STD, device)
    assert last_launch()["kernel"] == "gather"
    assert got.tobytes() == ol.oracle_crop_resize_norm_split(img, rects, (257, 16), wl.C3_MEAN, wl.C3_STD).tobytes()


def test_planes_the_strip_form_cannot_take_are_declined_on_the_host(device):
    import torch
    rng = np.random.RandomState(6)
    # rows that do not share their alignment (pitch 999), and a one-column crop among aligned rows
    for w, rects in ((333, np.array([[0, 0, 333, 100]] * 8, np.int32)),
                     (332, np.array([[0, 0, 332, 100]] * 7 + [[5, 7, 1, 50]], np.int32))):
        img = rng.randint(0, 256, (100, w, 3)).astype(np.uint8)
        src = torch.from_numpy(img).to(device)
        got = _c3(src, rects, (64, 40), wl.C3_MEAN, wl.C3_STD, device)
        assert last_launch()["kernel"] == "gather"
        assert got.tobytes() == ol.oracle_crop_resize_norm_split(img, rects, (64, 40), wl.C3_MEAN, wl.C3_STD).tobytes()


def test_source_that_ends_with_its_allocation(device):
    """Windows of the last rows reach past the image; the strip form's buffer resource ends with the image, so those
    bytes read as zero and are never used.  The image is the tail of its allocation here (a view that ends where the
    tensor ends), and the rows in front of it hold other values than the image."""
    import torch
    rng = np.random.RandomState(7)
    w, h = 128, 40
    whole = torch.from_numpy(rng.randint(0, 256, (h + 3, w, 3)).astype(np.uint8)).to(device)
    src = whole[3:]                                    # ends with the allocation's last byte
    img = src.cpu().numpy()
    rects = np.array([[0, h - 1, w, 1], [w - 2, h - 2, 2, 2], [0, 0, w, h], [3, h - 5, 100, 5],
                      [w - 3, h - 1, 3, 1], [0, h - 3, 7, 3], [60, 20, 68, 20], [1, 1, 126, 38]], np.int32)
    for dst in ((224, 224), (37, 11)):
        got = _c3(src, rects, dst, wl.C3_MEAN, wl.C3_STD, device)
        assert last_launch()["kernel"] == "strip"
        assert got.tobytes() == ol.oracle_crop_resize_norm_split(img, rects, dst, wl.C3_MEAN, wl.C3_STD).tobytes()


@pytest.mark.parametrize("dst", [(96, 64), (200, 30), (45, 100)])
def test_letterboxed_chain_compiled_on_first_use(device, dst):
    """PRESERVE_AR (bands of the background colour left/right or above/below) -> Mul -> planar float, three planes;
    not in the ahead-of-time list, so the strip form comes from the run-time compiler."""
    import torch
    rng = np.random.RandomState(8)
    w, h = 320, 200
    img = rng.randint(0, 256, (h, w, 3)).astype(np.uint8)
    rects = np.array([[10, 20, 300, 60], [40, 0, 50, 200], [100, 50, 120, 120]], np.int32)   # wide, tall, square
    bg = np.array([0.25, 128.5, 255.0], np.float32)
    mul = np.array([0.5, 2.0, 1.0 / 255.0], np.float32)
    src = torch.from_numpy(img).to(device)
    want = np.zeros((3, 3, dst[1], dst[0]), np.float32)
    reads = [ol.read_2d(img, 3, crop=rects[i], resize=dst, ar=ol.PRESERVE_AR, bg=tuple(bg) + (0.0,)) for i in range(3)]
    ol.execute(reads, [ol.op(ol.MUL, tuple(mul) + (0.0,))], [ol.write(ol.TENSOR_SPLIT, want, 3, dst[0], dst[1], 3, 3)])
    results = {}
    for on in (True, False):
        with strip_switched(on):
            out = torch.full((3, 3, dst[1], dst[0]), -7.0, dtype=torch.float32, device=device)
            cases.uncompiled_letterbox_split_b3(src, rects, dst, bg, mul, out)
            torch.cuda.synchronize()
            assert last_launch()["kernel"] == ("strip_jit" if on else "gather_jit")
            results[on] = out.cpu().numpy()
    assert results[True].tobytes() == want.tobytes()
    assert results[False].tobytes() == want.tobytes()


@pytest.mark.parametrize("kind,cn,dtype", [(0, 2, np.uint8), (1, 4, np.uint8), (2, 3, np.uint16)])
@pytest.mark.parametrize("dst,rect", [((200, 40), (10, 5, 60, 90)),       # enlarging: the last columns repeat the crop's last pixel
                                      ((64, 64), (0, 0, 160, 120)),       # reducing, the whole image
                                      ((33, 9), (158, 117, 2, 3))])        # the image's last rows and columns
def test_other_pixel_types_compiled_on_first_use(device, kind, cn, dtype, dst, rect):
    """2-, 4- and 6-byte pixels: the tap pair of a clamped column is handled per element size (dword select for 4 bytes, on
    the unpacked values otherwise)."""
    import torch
    rng = np.random.RandomState(90 + kind)
    w, h = 160, 120
    img = rng.randint(0, 1024 if dtype == np.uint16 else 256, (h, w, cn)).astype(dtype)
    src = torch.from_numpy(img.view(np.int16) if dtype == np.uint16 else img).to(device)
    want = np.zeros((cn, dst[1], dst[0]), np.float32)
    ol.execute([ol.read_2d(img, cn, crop=rect, resize=dst, ar=ol.IGNORE_AR)], [ol.op(ol.MUL, (0.5, 0.5, 0.5, 0.5))],
               [ol.write(ol.TENSOR_SPLIT, want, cn, dst[0], dst[1], 1, cn)])
    for on in (True, False):
        with strip_switched(on):
            out = torch.full((cn, dst[1], dst[0]), -7.0, dtype=torch.float32, device=device)
            cases.uncompiled_resize_split(kind, src, rect, dst, 0.5, out)
            torch.cuda.synchronize()
            assert last_launch()["kernel"] == ("strip_jit" if on else "gather_jit")
            assert out.cpu().numpy().tobytes() == want.tobytes(), (kind, dst, rect, on)


def test_configuration_3_takes_the_strip_form(device):
    import torch
    c = wl.config3()
    src = torch.from_numpy(c["src"]).to(device)
    got = _c3(src, c["rects"], c["dst"], c["sub"], c["div"], device)
    ll = last_launch()
    assert ll["kernel"] == "strip" and ll["grid"] == [28, 1, 64] and ll["block"] == [64, 4, 1]
    with strip_switched(False):
        tiles = _c3(src, c["rects"], c["dst"], c["sub"], c["div"], device)
        assert last_launch()["kernel"] == "gather"
    assert got.tobytes() == tiles.tobytes()


@pytest.mark.parametrize("rows", [256, 257, 448])
def test_wave_priorities_follow_the_size_of_the_launch(device, rows):
    """A strip launch of up to 2 048 workgroups (64 planes of 256 rows) runs its waves at priorities that fall as they
    advance, with workgroups from number 1 024 on one step behind; a larger one (257 rows: 2 112 workgroups, 448 rows:
    two full rounds) leaves the priorities alone.  Either way the result is the tile form's and the oracle's."""
    import torch
    c = wl.config3()
    dst = (224, rows)
    src = torch.from_numpy(c["src"]).to(device)
    got = _c3(src, c["rects"], dst, c["sub"], c["div"], device)
    ll = last_launch()
    assert ll["kernel"] == "strip" and ll["grid"] == [(rows + 7) // 8, 1, 64]
    with strip_switched(False):
        tiles = _c3(src, c["rects"], dst, c["sub"], c["div"], device)
        assert last_launch()["kernel"] == "gather"
    assert got.tobytes() == tiles.tobytes()
    assert got.tobytes() == ol.oracle_crop_resize_norm_split(c["src"], c["rects"], dst, c["sub"], c["div"]).tobytes()


@pytest.mark.parametrize("rows", [16384, 16392])
def test_wave_priorities_in_a_kernel_compiled_on_first_use(device, rows):
    """One tall plane through the run-time compiled strip form: 2 048 workgroups (priorities on, the second half of the
    workgroups counted as started late) and 2 049 (priorities off)."""
    import torch
    rng = np.random.RandomState(77)
    w, h, cn = 160, 120, 4
    img = rng.randint(0, 256, (h, w, cn)).astype(np.uint8)
    src = torch.from_numpy(img).to(device)
    dst, rect = (40, rows), (3, 2, 150, 117)
    want = np.zeros((cn, dst[1], dst[0]), np.float32)
    ol.execute([ol.read_2d(img, cn, crop=rect, resize=dst, ar=ol.IGNORE_AR)], [ol.op(ol.MUL, (0.5, 0.5, 0.5, 0.5))],
               [ol.write(ol.TENSOR_SPLIT, want, cn, dst[0], dst[1], 1, cn)])
    out = torch.full((cn, dst[1], dst[0]), -7.0, dtype=torch.float32, device=device)
    cases.uncompiled_resize_split(1, src, rect, dst, 0.5, out)
    torch.cuda.synchronize()
    ll = last_launch()
    assert ll["kernel"] == "strip_jit" and ll["grid"] == [(rows + 7) // 8, 1, 1]
    assert out.cpu().numpy().tobytes() == want.tobytes()

