"""BatchRead<CONDITIONAL_WITH_DEFAULT>: horizontal fusion compiled for B planes, run with fewer live ones; the
other planes take the default value through the chain.  Reference: batch_operations.h:221-281 and the executor
overloads with activeBatch/defaultValue (executors.h:80-100).  Checked bit for bit against the CPU oracle (itself
identical to the reference's CPU backend on these chains, test_oracle.py)."""
import numpy as np
import pytest

import oracle_lib as ol
from fusedkernellibrary_amd import last_launch
import fkl_cases as cases
import workloads as wl

pytestmark = pytest.mark.gpu

RECTS = np.array([[0, 0, 50, 40], [10, 10, 100, 80], [150, 80, 50, 40], [5, 5, 20, 100], [0, 0, 200, 120], [100, 60, 3, 2],
                  [20, 30, 64, 64], [1, 2, 77, 33]], np.int32)


@pytest.mark.parametrize("used", [0, 1, 3, 8])
@pytest.mark.parametrize("dst", [(32, 24), (224, 224), (131, 7)])
def test_crop_resize_with_default_planes(device, used, dst):
    import torch
    rng = np.random.RandomState(3)
    src_np = rng.randint(0, 256, (120, 200, 3)).astype(np.uint8)
    default = (1.5, -2.0, 300.0)
    src = torch.from_numpy(src_np).to(device)
    out = torch.full((8, 3, dst[1], dst[0]), 7.0, dtype=torch.float32, device=device)
    cases.crop_resize_default_norm_split(src, RECTS, dst, used, default, wl.C3_MEAN, wl.C3_STD, out)
    torch.cuda.synchronize()
    assert last_launch()["kernel"] == "gather"
    want = ol.oracle_crop_resize_default_norm_split(src_np, RECTS, dst, used, default, wl.C3_MEAN, wl.C3_STD)
    assert out.cpu().numpy().tobytes() == want.tobytes()


@pytest.mark.parametrize("active", [0, 2, 4])
def test_image_array_with_active_batch_and_default(device, active):
    import torch
    rng = np.random.RandomState(9)
    srcs_np = [rng.randint(0, 256, (30, 41, 3)).astype(np.uint8) for _ in range(4)]
    srcs = [torch.from_numpy(s).to(device) for s in srcs_np]
    out = torch.zeros((4, 30, 41, 3), dtype=torch.float32, device=device)
    cases.batch_default_cast_mul(srcs, active, (7, 200, 33), (0.5, 2.0, 1.25), out)
    torch.cuda.synchronize()
    want = ol.oracle_batch_default_cast_mul(srcs_np, active, (7, 200, 33), (0.5, 2.0, 1.25))
    assert out.cpu().numpy().tobytes() == want.tobytes()
