"""SaturateDepth, DenormalizePixel, SaturateDenormalizePixel, Saturate, SaturateFloat (reference
color_conversion.h:96-148, saturate.h:38-64) and the transposed tensor forms TensorTSplit / TensorTPack /
CircularTensor<..., ColorPlanes::Transposed> (memory_operations.h:214-241, 292-327, circular_tensor.h:84-168) on the GPU,
bit for bit against the CPU oracle, which test_oracle_depth_and_transposed.py pins to the reference's CPU backend
running the same chain text (tests/cases/color_chains.h, circular_chains.h)."""
import numpy as np
import pytest

import oracle_lib as ol
import fkl_cases as cases
from test_oracle_depth_and_transposed import float_image, images

pytestmark = pytest.mark.gpu


def dev_out(which, src, device):
    import torch
    cn, dt, _ = ol.DEPTH_OPS[which]
    tdt = {np.uint8: torch.uint8, np.uint16: torch.int16, np.float32: torch.float32}[dt]
    return torch.zeros(src.shape[:2] + ((cn,) if cn > 1 else ()), dtype=tdt, device=device)


@pytest.mark.parametrize("which", sorted(ol.DEPTH_OPS))
def test_depth_operations(device, which):
    import torch
    for seed, (h, w) in enumerate([(5, 9), (37, 301)]):        # odd widths: every row-tail path of the rows kernel
        src = float_image(which, h, w, 400 + 10 * which + seed)
        out = dev_out(which, src, device)
        cases.depth_ops(which, torch.from_numpy(src).to(device), out, -2.5, 9.25)
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        want = ol.oracle_depth_ops(which, src, -2.5, 9.25)
        assert got.tobytes() == want.tobytes(), (which, h, w)


def test_saturate_denormalize_values_of_the_reference_unit_test(device):
    """utests/algorithm/image_processing/utest_color_conversion.h:282-297 on the GPU; 0.5 -> 127 as on the reference's
    CPU backend (a C cast of 127.5), where that file's literal says 128."""
    import torch
    src = np.array([[[-0.5, 0.5, 1.5], [0.25, 0.75, 0.9]]], np.float32)
    out = dev_out(4, src, device)
    cases.depth_ops(4, torch.from_numpy(src).to(device), out)
    torch.cuda.synchronize()
    assert out.cpu().numpy().tolist() == [[[0, 127, 255], [63, 191, 229]]]


@pytest.mark.parametrize("planes,w,h", [(1, 8, 4), (3, 10, 6), (4, 333, 25), (2, 1920, 64)])
def test_transposed_tensor_round_trip(device, planes, w, h):
    import torch
    imgs = images(planes, w, h, 500 + planes)
    tensor_t = torch.full((3, planes, h, w), -7.0, dtype=torch.float32, device=device)
    packed = torch.zeros((planes, h, w, 3), dtype=torch.float32, device=device)
    cases.transposed_round_trip([torch.from_numpy(i).to(device) for i in imgs], 1.25, tensor_t, 0.75, packed)
    torch.cuda.synchronize()
    want_t, want_p = ol.oracle_transposed_round_trip(imgs, 1.25, 0.75)
    assert tensor_t.cpu().numpy().tobytes() == want_t.tobytes()
    assert packed.cpu().numpy().tobytes() == want_p.tobytes()


@pytest.mark.parametrize("batch", [2, 3, 5])
@pytest.mark.parametrize("oldest_first", [False, True])
def test_transposed_circular_window(device, batch, oldest_first):
    import torch
    h, w = 36, 52
    imgs = images(batch + 4, w, h, 520 + batch)
    got = cases.circular_transposed(batch, oldest_first, [torch.from_numpy(i).to(device) for i in imgs], 10.0)
    want = ol.oracle_circular(batch, oldest_first, imgs, 10.0)
    defined = ~np.isnan(want)
    assert defined[batch - 1:].all()
    assert np.array_equal(got[defined], want[defined])
