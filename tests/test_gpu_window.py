"""DivergentBatchTransformDPP launches and CircularTensor::update (reference data_parallel_patterns.h:286-381,
executors.h:360-411, circular_tensor.h:111-161) on the GPU, bit for bit against the restatement that
test_oracle_window.py pins to the reference's CPU backend.  Planes of the window that the reference fills from
memory nothing was stored in yet (fewer updates than planes) are left out of the comparison."""
import numpy as np
import pytest

import oracle_lib as ol
import fkl_cases as cases

pytestmark = pytest.mark.gpu


def test_divergent_two_sequences(device):
    """The reference's own divergent-batch test (tests/data_parallel_patterns/test_divergent_batch.h) on random data."""
    import torch
    r = np.random.default_rng(61)
    for (h, w) in ((32, 32), (45, 301)):
        a = r.integers(0, 2**32, (h, w), dtype=np.uint32)
        b = r.integers(0, 2**32, (h, w), dtype=np.uint32)
        da, db = torch.from_numpy(a.view(np.int32)).to(device), torch.from_numpy(b.view(np.int32)).to(device)
        out = torch.zeros((2, h, w), dtype=torch.int32, device=device)
        cases.divergent_two(da, db, 3, out)
        torch.cuda.synchronize()
        got = out.cpu().numpy().view(np.uint32)
        assert np.array_equal(got[0], a + np.uint32(3)) and np.array_equal(got[1], b)


def test_divergent_sequences_of_different_shapes_and_kernels(device):
    """A pointwise tensor sequence (four elements per thread) and a bilinear sequence (one per thread) share a launch."""
    import torch
    r = np.random.default_rng(62)
    for (h, w, ih, iw) in ((12, 20, 7, 9), (270, 480, 333, 517)):
        t = (r.random((4, h, w, 3), dtype=np.float32) * 10 - 5).astype(np.float32)
        img = r.integers(0, 256, (ih, iw, 3), dtype=np.uint8)
        out = torch.full((4, h, w, 3), -1.0, dtype=torch.float32, device=device)
        cases.divergent_mixed(torch.from_numpy(t).to(device), 1.5, torch.from_numpy(img).to(device), out)
        torch.cuda.synchronize()
        assert out.cpu().numpy().tobytes() == ol.oracle_divergent_mixed(t, 1.5, img).tobytes()


@pytest.mark.parametrize("batch", [2, 3, 4, 15])
@pytest.mark.parametrize("oldest_first", [False, True])
def test_circular_tensor_window(device, batch, oldest_first):
    import torch
    r = np.random.default_rng(70 + batch)
    h, w = 36, 52
    imgs = [r.integers(0, 256, (h, w, 3), dtype=np.uint8) for _ in range(batch + 4)]
    got = cases.circular(batch, oldest_first, [torch.from_numpy(i).to(device) for i in imgs], 10.0)
    want = ol.oracle_circular(batch, oldest_first, imgs, 10.0)
    defined = ~np.isnan(want)
    assert defined[batch - 1:].all()
    assert np.array_equal(got[defined], want[defined])


def test_circular_tensor_reference_scenario(device):
    """tests/data/test_circular_tensor.h: constant images 1..ITERS; afterwards plane z holds ITERS - z."""
    import torch
    iters, batch, h, w = 20, 4, 128, 128
    imgs = [torch.full((h, w, 3), i + 1, dtype=torch.uint8, device=device) for i in range(iters)]
    got = cases.circular(batch, False, imgs, 10.0)
    for z in range(batch):
        assert (got[-1, z] == float(iters - z)).all()


def test_sweep_of_random_sizes(device):
    """150 seeded cases at random sizes: the two divergent launches above, and the window for every batch size and
    order the case driver has (2, 3, 4, 15; newest or oldest first) with a random number of updates."""
    import torch
    for i in range(150):
        r = np.random.default_rng(170000 + i)
        h, w = int(r.integers(1, 60)), int(r.integers(1, 400))
        kind = i % 3
        if kind == 0:
            a = r.integers(0, 2**32, (h, w), dtype=np.uint32)
            b = r.integers(0, 2**32, (h, w), dtype=np.uint32)
            add = int(r.integers(0, 1000))
            out = torch.zeros((2, h, w), dtype=torch.int32, device=device)
            cases.divergent_two(torch.from_numpy(a.view(np.int32)).to(device), torch.from_numpy(b.view(np.int32)).to(device), add, out)
            torch.cuda.synchronize()
            got = out.cpu().numpy().view(np.uint32)
            same = np.array_equal(got[0], a + np.uint32(add)) and np.array_equal(got[1], b)
        elif kind == 1:
            ih, iw = int(r.integers(1, 200)), int(r.integers(2, 300))
            t = (r.random((4, h, w, 3), dtype=np.float32) * 10 - 5).astype(np.float32)
            img = r.integers(0, 256, (ih, iw, 3), dtype=np.uint8)
            mul = float(np.float32(r.uniform(0.1, 4.0)))
            out = torch.full((4, h, w, 3), -1.0, dtype=torch.float32, device=device)
            cases.divergent_mixed(torch.from_numpy(t).to(device), mul, torch.from_numpy(img).to(device), out)
            torch.cuda.synchronize()
            same = out.cpu().numpy().tobytes() == ol.oracle_divergent_mixed(t, mul, img).tobytes()
        else:
            batch = int(r.choice([2, 3, 4, 15]))
            oldest_first = bool(r.integers(0, 2))
            imgs = [r.integers(0, 256, (h, w, 3), dtype=np.uint8) for _ in range(batch + int(r.integers(0, 6)))]
            got = cases.circular(batch, oldest_first, [torch.from_numpy(x).to(device) for x in imgs], 10.0)
            want = ol.oracle_circular(batch, oldest_first, imgs, 10.0)
            defined = ~np.isnan(want)
            same = np.array_equal(got[defined], want[defined])
        assert same, (i, kind, w, h)
