"""Deinterlace<BLEND|INTER_LINEAR> (reference deinterlace.h:44-103), bit for bit against the CPU oracle, which
test_oracle.py pins to the reference backend."""
import numpy as np
import pytest

import oracle_lib as ol
import fkl_cases as cases

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("mode", [ol.DEINTERLACE_BLEND, ol.DEINTERLACE_LINEAR_EVEN, ol.DEINTERLACE_LINEAR_ODD])
@pytest.mark.parametrize("shape", [(12, 17), (1080, 1920), (1, 5), (2, 64), (35, 259)])
def test_deinterlace_uchar3(device, mode, shape):
    import torch
    rng = np.random.RandomState(31)
    img = rng.randint(0, 256, shape + (3,)).astype(np.uint8)
    src = torch.from_numpy(img).to(device)
    out = torch.full(shape + (3,), -1.0, dtype=torch.float32, device=device)
    cases.deinterlace(src, mode, out)
    torch.cuda.synchronize()
    assert out.cpu().numpy().tobytes() == ol.oracle_deinterlace(img, 3, mode).tobytes()


@pytest.mark.parametrize("mode", [ol.DEINTERLACE_BLEND, ol.DEINTERLACE_LINEAR_EVEN, ol.DEINTERLACE_LINEAR_ODD])
def test_deinterlace_float(device, mode):
    import torch
    rng = np.random.RandomState(32)
    img = (rng.rand(40, 131).astype(np.float32) * 100 - 50)
    src = torch.from_numpy(img).to(device)
    out = torch.zeros((40, 131), dtype=torch.float32, device=device)
    cases.deinterlace(src, mode, out)
    torch.cuda.synchronize()
    assert out.cpu().numpy().tobytes() == ol.oracle_deinterlace(img, 1, mode).tobytes()
