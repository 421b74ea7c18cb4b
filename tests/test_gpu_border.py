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
