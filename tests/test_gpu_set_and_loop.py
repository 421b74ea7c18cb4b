"""setTo (ReadSet -> PerThreadWrite on library-owned Ptr1D / Ptr2D / Tensor) and StaticLoop<Add<float>, N>, spelled as
the reference's instruction-count benchmark spells them (benchmark_numinstructions_x_operation.h:40-75).  Expected
values are closed forms: N float additions of `add` starting from `init`, each rounded once."""
import numpy as np
import pytest

import fkl_cases as cases

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("iterations", [1, 6, 50])
@pytest.mark.parametrize("n", [1, 255, 3840 * 8 + 3])
def test_set_to_then_static_loop(device, iterations, n):
    init, add = np.float32(1.0), np.float32(0.1)
    got = cases.set_and_loop_f32(n, init, add, iterations)
    want = init
    for _ in range(iterations):
        want = np.float32(want + add)
    assert got.shape == (n,) and (got.view(np.uint32) == np.float32(want).view(np.uint32)).all()


def test_set_to_pitched_image_and_tensor(device):
    w, h, planes = 37, 11, 3
    img, pitch, ten = cases.set_to_shapes(w, h, planes, (7, 200, 33), -2.5)
    assert pitch >= w * 3
    px = img[:, : w * 3].reshape(h, w, 3)
    assert (px == np.array([7, 200, 33], np.uint8)).all()
    assert (ten == np.float32(-2.5)).all() and ten.shape == (planes, h, w)


def test_set_to_fills_every_colour_plane_of_a_transposed_tensor(device):
    """Documented difference: the reference's setTo on an ND::T3D Ptr goes through PerThreadWrite<T3D>, which addresses
    colour plane 0 only and leaves the other colour planes as they were (FK/core/data/ptr_utils.h:24-45,
    FK/core/data/rawptr.h:228-240); here every element of the Ptr takes the value, as for the other dimensionalities."""
    got = cases.set_to_transposed(21, 5, 4, 3, sentinel=-99.0, value=6.25)
    assert got.shape == (12, 5, 21) and (got == np.float32(6.25)).all()
