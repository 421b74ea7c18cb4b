"""BorderReader<CONSTANT|REPLICATE|REFLECT|WRAP|REFLECT_101> under a Crop that leaves the image (reference
border_reader.h:177-327), bit for bit against the CPU oracle, which test_oracle_border.py pins to numpy.pad and to the
reference's CPU backend."""
import numpy as np
import pytest

import oracle_lib as ol
import fkl_cases as cases

pytestmark = pytest.mark.gpu
TYPES = [ol.BORDER_CONSTANT, ol.BORDER_REPLICATE, ol.BORDER_REFLECT, ol.BORDER_WRAP, ol.BORDER_REFLECT_101]


@pytest.mark.parametrize("bt", TYPES)
def test_pad_uchar3(device, bt):
    import torch
    img = np.random.default_rng(21).integers(0, 256, (90, 161, 3), dtype=np.uint8)
    src = torch.from_numpy(img).to(device)
    h, w = img.shape[:2]
    for (left, top, ow, oh) in ((8, 8, w + 16, h + 16), (2 * w + 3, 3 * h + 1, 5 * w + 2, 7 * h), (-5, -3, 64, 40), (0, 0, w, h), (1, 0, 3, 1)):
        out = torch.zeros((oh, ow, 3), dtype=torch.uint8, device=device)
        cases.pad(src, bt, left, top, out, value=(9, 8, 7))
        torch.cuda.synchronize()
        assert out.cpu().numpy().tobytes() == ol.oracle_pad(img, bt, left, top, ow, oh, value=(9, 8, 7)).tobytes(), (left, top, ow, oh)


@pytest.mark.parametrize("bt", TYPES)
def test_pad_float(device, bt):
    import torch
    img = (np.random.default_rng(22).random((37, 53), dtype=np.float32) * 100 - 50).astype(np.float32)
    src = torch.from_numpy(img).to(device)
    for (left, top, ow, oh) in ((5, 9, 70, 60), (60, 40, 200, 130)):
        out = torch.zeros((oh, ow), dtype=torch.float32, device=device)
        cases.pad(src, bt, left, top, out, value=(-1.5,))
        torch.cuda.synchronize()
        assert out.cpu().numpy().tobytes() == ol.oracle_pad(img, bt, left, top, ow, oh, value=(-1.5,)).tobytes(), (left, top, ow, oh)



@pytest.mark.parametrize("dtype,cn", [(np.uint8, 4), (np.uint16, 3), (np.uint8, 1), (np.float32, 3)])
@pytest.mark.parametrize("bt", [ol.BORDER_CONSTANT, ol.BORDER_REPLICATE, ol.BORDER_WRAP, ol.BORDER_REFLECT_101])
def test_pad_other_pixel_types(device, bt, dtype, cn):
    """Pixels of 4, 6, 1 and 12 bytes: a lane on the left or right edge fetches each pixel as one access of whole dwords where
    the bytes behind the pixel are still inside the image (6-byte pixels: two bytes behind), element by element on the
    image's last rows; the second pad reaches further out than an image size, where indices are folded with divisions."""
    import torch
    rng = np.random.default_rng(23)
    shape = (45, 67, cn) if cn > 1 else (45, 67)
    img = (rng.random(shape, dtype=np.float32) * 100 - 50) if dtype == np.float32 else rng.integers(0, 1000 if dtype == np.uint16 else 256, shape).astype(dtype)
    src = torch.from_numpy(img.view(np.int16) if dtype == np.uint16 else img).to(device)
    h, w = img.shape[:2]
    value = (9, 8, 7, 6)[:cn]
    for (left, top, ow, oh) in ((6, 5, w + 13, h + 9), (3 * w + 2, 2 * h + 1, 5 * w, 4 * h)):
        out = torch.zeros((oh, ow, cn) if cn > 1 else (oh, ow), dtype=src.dtype, device=device)
        cases.pad(src, bt, left, top, out, value=value, kind=ol.pad_kind(dtype, cn))
        torch.cuda.synchronize()
        want = ol.oracle_pad(img, bt, left, top, ow, oh, value=value)
        assert out.cpu().numpy().tobytes() == want.tobytes(), (left, top, ow, oh)
