"""Four host threads, each with a stream of its own, launch different chains through the host API at the same time and
check every result against the oracle: the library's registry of compiled chains, its per-thread state (last launch,
remembered divisors, error text) and the run-time compiler must not depend on who else is calling.
Reference behaviour: executeOperations is a free function on a caller-owned Stream (FK/fused_kernel.h), callable from
any thread."""
import threading

import numpy as np
import pytest

import fkl_cases as cases
import oracle_lib as ol
import random_cases as rc

pytestmark = pytest.mark.gpu

ROUNDS = 25


@pytest.fixture(scope="module")
def device():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


def _image_on(device, backing, w):
    import torch
    h, pitch = backing.shape
    return torch.as_strided(torch.from_numpy(backing).to(device), (h, w, 3), (pitch, 3, 1))


def test_four_threads_launch_different_chains(device):
    import torch
    po = ol.pointwise_oracle()
    import pointwise_cases as pc

    # every worker: (launch, output tensor, expected bytes); inputs are uploaded before the threads start
    seed, batch, size, pad, least, dst = rc.NORMALISE[2]
    backing, rects, sub, div = rc.normalise_inputs(seed, batch, size, pad, least)
    n_img = _image_on(device, backing, size[0])
    n_out = torch.zeros((batch, 3, dst[1], dst[0]), dtype=torch.float32, device=device)
    n_want = ol.oracle_crop_resize_norm_split(np.ascontiguousarray(rc.image_of(backing, size[0])), rects, dst, sub, div)
    n_dst = dst

    seed, size, pad, dst = rc.LETTERBOX[0]
    lb, l_rects, bg, mul, lsub = rc.letterbox_inputs(seed, size, pad)
    l_img = _image_on(device, lb, size[0])
    l_out = torch.zeros((5, dst[1], dst[0], 3), dtype=torch.uint8, device=device)
    l_want = ol.oracle_crop_resize_par_u8(np.ascontiguousarray(rc.image_of(lb, size[0])), l_rects, dst, bg, mul, lsub)
    l_dst = dst

    seed, size, pad, dst = rc.FRAMES[5]
    fb, scale = rc.frame_inputs(seed, size, pad)
    f_in = torch.from_numpy(fb).to(device)[:, :size[0]]
    f_out = torch.zeros((3, dst[1], dst[0]), dtype=torch.float32, device=device)
    f_want = ol.oracle_nv12_rgb_resize_split(np.ascontiguousarray(fb[:, :size[0]]), size[0], size[1], dst, scale)
    f_size, f_dst = size, dst

    which, h, w = 9, 37, 300                                   # AbsDiff<float3>, compiled at run time on first use
    p_src = pc.inputs(which, po.CASES, h, w, 3)
    p_in = torch.from_numpy(np.ascontiguousarray(p_src).view(np.uint8).reshape(h, -1)).to(device)
    p_out = torch.zeros_like(p_in)
    p_want = po.run(which, p_src, pc.constants(which), pc.MATRIX)

    def bits(want):
        return lambda got: got.tobytes() == np.ascontiguousarray(want).tobytes()

    def values(got):    # produced NaNs compare as NaN, everything else bit for bit
        return pc.same(which, np.ascontiguousarray(got).view(np.float32).reshape(p_want.shape), p_want, po.INEXACT)

    jobs = [
        (lambda: cases.crop_resize_norm_split(n_img, rects, n_dst, sub, div, n_out), n_out, bits(n_want)),
        (lambda: cases.crop_resize_par_u8(l_img, l_rects, l_dst, bg, mul, lsub, l_out), l_out, bits(l_want)),
        (lambda: cases.nv12_rgb_resize_split(f_in, f_size[0], f_size[1], f_dst, scale, f_out), f_out, bits(f_want)),
        (lambda: cases.pointwise(which, p_in, w, h, p_out, pc.constants(which), pc.MATRIX), p_out, values),
    ]
    torch.cuda.synchronize()
    start = threading.Barrier(len(jobs))
    failures = []

    def worker(index, launch, out, equal):
        try:
            stream = torch.cuda.Stream(device=device)
            with torch.cuda.stream(stream):
                start.wait(timeout=60)
                for r in range(ROUNDS):
                    out.zero_()
                    launch()
                    stream.synchronize()
                    if not equal(out.cpu().numpy()):
                        failures.append(f"thread {index}, round {r}: result differs from the oracle")
                        return
        except Exception as e:   # noqa: BLE001 - reported to the main thread
            failures.append(f"thread {index}: {type(e).__name__}: {e}")

    threads = [threading.Thread(target=worker, args=(i, *job)) for i, job in enumerate(jobs)]
    print(f"{len(threads)} threads x {ROUNDS} launches", flush=True)
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not any(t.is_alive() for t in threads), "a worker did not finish"
    assert not failures, failures
