"""Chains that are not in csrc/aot_signatures.txt: the library compiles them with hiprtc when it first sees their
signature (same device headers, same flags as the ahead-of-time build) and must give the oracle's bits."""
import numpy as np
import pytest

import oracle_lib as ol
from fusedkernellibrary_amd import cases, last_launch, signatures

pytestmark = pytest.mark.gpu


def test_pointwise_chain_compiled_on_first_use(device):
    import torch
    rng = np.random.RandomState(21)
    x = (rng.rand(37, 1001).astype(np.float32) * 200 - 100)
    src = torch.from_numpy(x).to(device)
    out = torch.zeros_like(src)
    before = set(signatures())
    cases.uncompiled_pointwise_f32(src, out)
    torch.cuda.synchronize()
    assert last_launch()["kernel"] == "rows_jit"
    new = set(signatures()) - before
    assert len(new) <= 1 and all("Div<f32,f32,f32>" in s[0] for s in new)
    want = np.float32(np.float32(np.float32(x * np.float32(1.5)) - np.float32(0.25)) / np.float32(3.0)) + np.float32(7.0)
    assert out.cpu().numpy().tobytes() == want.astype(np.float32).tobytes()
    # second call: served from the registry, same result
    out.zero_()
    cases.uncompiled_pointwise_f32(src, out)
    torch.cuda.synchronize()
    assert out.cpu().numpy().tobytes() == want.astype(np.float32).tobytes()


@pytest.mark.parametrize("dst", [(64, 48), (9, 200), (301, 7)])
def test_one_channel_resize_compiled_on_first_use(device, dst):
    import torch
    rng = np.random.RandomState(22)
    img = rng.randint(0, 256, (90, 131)).astype(np.uint8)
    rect = (3, 5, 120, 85)
    src = torch.from_numpy(img).to(device)
    out = torch.zeros((dst[1], dst[0]), dtype=torch.float32, device=device)
    cases.uncompiled_gray_resize(src, rect, dst, 0.5, out)
    torch.cuda.synchronize()
    assert last_launch()["kernel"] == "gather_jit"
    want = np.zeros((dst[1], dst[0]), np.float32)
    ol.execute([ol.read_2d(img, 1, crop=rect, resize=dst, ar=ol.IGNORE_AR)], [ol.op(ol.MUL, (0.5, 0, 0, 0))],
               [ol.write(ol.WRITE_2D, want, 1, dst[0], dst[1])])
    assert out.cpu().numpy().tobytes() == want.tobytes()


def test_float4_resize_compiled_on_first_use(device):
    import torch
    rng = np.random.RandomState(23)
    img = rng.rand(40, 55, 4).astype(np.float32)
    dst = (77, 23)
    src = torch.from_numpy(img).to(device)
    out = torch.zeros((dst[1], dst[0], 4), dtype=torch.float32, device=device)
    cases.uncompiled_float4_resize(src, dst, out)
    torch.cuda.synchronize()
    assert last_launch()["kernel"] == "gather_jit"
    want = np.zeros((dst[1], dst[0], 4), np.float32)
    ol.execute([ol.read_2d(img, 4, resize=dst, ar=ol.IGNORE_AR)], [], [ol.write(ol.WRITE_2D, want, 4, dst[0], dst[1])])
    assert out.cpu().numpy().tobytes() == want.tobytes()
