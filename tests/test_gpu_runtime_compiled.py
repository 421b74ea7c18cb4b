"""Chains that are not in csrc/aot_signatures.txt: the library compiles them with hiprtc when it first sees their
signature (same device headers, same flags as the ahead-of-time build) and must give the oracle's bits."""
import numpy as np
import pytest

import oracle_lib as ol
from fusedkernellibrary_amd import last_launch, signatures
import fkl_cases as cases

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


_CACHE_SCRIPT = r"""
import ctypes, os, sys, time
sys.path.insert(0, sys.argv[1]); sys.path.insert(0, os.path.join(sys.argv[1], "tests"))
import numpy as np, torch
from fusedkernellibrary_amd import lib
import fkl_cases as cases
dev = torch.device("cuda:0")
x = np.random.RandomState(5).rand(33, 70).astype(np.float32)
src = torch.from_numpy(x).to(dev); out = torch.zeros_like(src)
t0 = time.time(); cases.uncompiled_pointwise_f32(src, out); torch.cuda.synchronize(); dt = time.time() - t0
log = ctypes.c_char_p(); lib().fklhip_jit_log(ctypes.byref(log))
np.save(sys.argv[2], out.cpu().numpy())
print("LOG:" + (log.value or b"").decode()); print("SECONDS:%.3f" % dt)
"""


def test_code_objects_are_reused_from_the_cache_directory(device, tmp_path):
    """FKLHIP_JIT_CACHE: the first process compiles and leaves a file, the second loads it; both give the same result."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cache = tmp_path / "cache"
    cache.mkdir()
    env = dict(os.environ, FKLHIP_JIT_CACHE=str(cache))
    outs = []
    for run in range(2):
        res = tmp_path / f"out{run}.npy"
        r = subprocess.run([sys.executable, "-c", _CACHE_SCRIPT, root, str(res)], env=env, capture_output=True, text=True, timeout=240)
        assert r.returncode == 0, r.stderr[-2000:]
        outs.append((np.load(res), r.stdout))
        files = [f for f in os.listdir(cache) if f.endswith(".co")]
        assert len(files) == 1 and not any(f.endswith(".tmp") for f in os.listdir(cache)), os.listdir(cache)
    assert "loaded from" not in outs[0][1] and "loaded from" in outs[1][1], (outs[0][1], outs[1][1])
    assert outs[0][0].tobytes() == outs[1][0].tobytes()
    # a damaged file is replaced, not trusted
    path = os.path.join(cache, files[0])
    with open(path, "wb") as f:
        f.write(b"not a code object")
    res = tmp_path / "out2.npy"
    r = subprocess.run([sys.executable, "-c", _CACHE_SCRIPT, root, str(res)], env=env, capture_output=True, text=True, timeout=240)
    assert r.returncode == 0, r.stderr[-2000:]
    assert np.load(res).tobytes() == outs[0][0].tobytes() and os.path.getsize(path) > 1000


def test_a_chain_that_would_need_scratch_memory_is_compiled_again_or_refused(device, tmp_path):
    """A per-thread array that cannot stay in registers (forced here through the kernel's test hook): by default the chain is
    compiled a second time with the array in LDS, runs, and the log says so; with FKLHIP_JIT_STRICT=1 it is refused."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    hook = "-DFKD_TEST_UNRESOLVED_INDEX=1"
    res = tmp_path / "out.npy"
    env = dict(os.environ, FKLHIP_JIT_DEFINES=hook, FKLHIP_JIT_STRICT="0")
    r = subprocess.run([sys.executable, "-c", _CACHE_SCRIPT, root, str(res)], env=env, capture_output=True, text=True, timeout=240)
    assert r.returncode == 0, r.stderr[-2000:]
    assert "bytes of scratch memory per lane; compiled again with per-thread arrays in LDS" in r.stdout, r.stdout
    ref = tmp_path / "ref.npy"
    r = subprocess.run([sys.executable, "-c", _CACHE_SCRIPT, root, str(ref)], env=dict(os.environ), capture_output=True, text=True, timeout=240)
    assert r.returncode == 0, r.stderr[-2000:]
    assert np.load(res).tobytes() == np.load(ref).tobytes()
    env["FKLHIP_JIT_STRICT"] = "1"
    r = subprocess.run([sys.executable, "-c", _CACHE_SCRIPT, root, str(res)], env=env, capture_output=True, text=True, timeout=240)
    assert r.returncode != 0 and "could not be compiled at run time" in r.stderr, r.stderr[-2000:]


def test_a_chain_whose_parameters_exceed_the_kernel_argument_limit_is_refused_with_a_sentence(device):
    """45 000 planes of 24-byte pointers on either side are 2 MB of by-value kernel arguments: the run-time compiler
    refuses the chain (FKLHIP_EBLOB_SIZE) and its log names the limit, instead of the launch call failing later."""
    import ctypes as C
    from fusedkernellibrary_amd import lib
    sig = b"Chain<BatchRead<45000,Read2D<Vec<u8,3>>>,OpList<>,BatchWrite<45000,Write2D<Vec<u8,3>>>>"
    h = C.c_void_p()
    assert lib().fklhip_lookup(sig, C.byref(h)) == 10002
    log = C.c_char_p()
    lib().fklhip_jit_log(C.byref(log))
    assert b"FKLHIP_MAX_BLOB_BYTES" in log.value and b"smaller batch" in log.value
    assert sig.decode() not in [s for s, _ in signatures()]
