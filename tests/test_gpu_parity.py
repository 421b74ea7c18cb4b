"""GPU parity tests: every benchmark chain, spelled with the C++ host API (tests/cases/fkl_cases.cpp), launched
through the C ABI on the MI355X and compared with the CPU oracle / golden fixtures.

Bars (written here as the north star states them): integer-only chains bit-exact; uchar outputs after float
bilinear + SaturateCast within +-1 LSB; float outputs within 1e-5 relative.  The kernels are built without FMA
contraction and with IEEE division, so in practice every comparison below is bit-exact; the asserts check the
stated bar and report bit-exactness separately so a regression to "merely within tolerance" is visible.
"""
import hashlib
import json
import os

import numpy as np
import pytest

import oracle_lib as ol
from fusedkernellibrary_amd import last_launch
import fkl_cases as cases
import workloads as wl

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
GOLD = np.load(os.path.join(HERE, "golden", "golden_outputs.npz"))
META = json.load(open(os.path.join(HERE, "golden", "golden_digests.json")))
DIG = META["digests"]
CASES = META["cases"]

FLOAT_RTOL = 1e-5   # relative, on float outputs
U8_ATOL = 1         # LSB, on uchar outputs after float arithmetic


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def check_float(got, want, what):
    assert got.shape == want.shape and got.dtype == np.float32, what
    exact = got.tobytes() == want.tobytes()
    if not exact:
        denom = np.maximum(np.abs(want), np.float32(1e-30))
        rel = float(np.max(np.abs(got - want) / denom))
        assert rel <= FLOAT_RTOL, f"{what}: max relative error {rel:.3e} exceeds {FLOAT_RTOL}"
    return exact


def check_u8(got, want, what, atol=U8_ATOL):
    assert got.shape == want.shape and got.dtype == np.uint8, what
    exact = got.tobytes() == want.tobytes()
    if not exact:
        d = int(np.max(np.abs(got.astype(np.int16) - want.astype(np.int16))))
        assert d <= atol, f"{what}: max difference {d} LSB exceeds {atol}"
    return exact


def dev_u8(a, device):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def run_c1(c, rects, device):
    import torch
    src = dev_u8(c["src"], device)
    out = torch.zeros((5, c["dst"][1], c["dst"][0], 3), dtype=torch.uint8, device=device)
    cases.crop_resize_par_u8(src, rects, c["dst"], c["bg"], c["mul"], c["sub"], out)
    torch.cuda.synchronize()
    return out.cpu().numpy()


def run_c3(c, device):
    import torch
    src = dev_u8(c["src"], device)
    out = torch.zeros((len(c["rects"]), 3, c["dst"][1], c["dst"][0]), dtype=torch.float32, device=device)
    cases.crop_resize_norm_split(src, c["rects"], c["dst"], c["sub"], c["div"], out)
    torch.cuda.synchronize()
    return out.cpu().numpy()


def run_c5(c, device):
    import torch
    src = dev_u8(c["nv12"], device)
    out = torch.zeros((3, c["dst"][1], c["dst"][0]), dtype=torch.float32, device=device)
    cases.nv12_rgb_resize_split(src, c["width"], c["height"], c["dst"], c["scale"], out)
    torch.cuda.synchronize()
    return out.cpu().numpy()


def run_c2(c, n, device, tf=0):
    import torch
    src = torch.from_numpy(c["src"]).to(device)
    out = torch.zeros_like(src)
    cases.add_mul_chain(src, n, c["add"], c["mul"], out, tf=tf)
    torch.cuda.synchronize()
    return out.cpu().numpy()


def run_c4(c, device):
    import torch
    srcs = [dev_u8(s, device) for s in c["srcs"]]
    outs = [torch.zeros_like(s) for s in srcs]
    cases.batch_muladd_sat(srcs, c["mul"], c["add"], outs)
    torch.cuda.synchronize()
    return srcs, outs


# ---- configuration 1: README chain ----------------------------------------------------------------------------

def test_config1_full_size(device):
    c = wl.config1()
    got = run_c1(c, c["rects"], device)
    assert last_launch()["kernel"] == "gather"
    assert check_u8(got, GOLD["c1_full"], "config 1 vs reference golden"), "config 1 is expected to be bit-exact"
    assert sha(got) == DIG["c1_full"]


def test_config1_reduced(device):
    c = wl.config1(**CASES["c1_small"])
    rects = np.array(META["c1_small_rects"], np.int32)
    got = run_c1(c, rects, device)
    assert check_u8(got, GOLD["c1_small"], "config 1 small vs golden")
    assert check_u8(got, ol.oracle_crop_resize_par_u8(c["src"], rects, c["dst"], c["bg"], c["mul"], c["sub"]), "vs oracle")


# ---- configuration 2: pure vertical fusion ----------------------------------------------------------------------

@pytest.mark.parametrize("n", [1, 10, 20, 30, 40, 50, 100])
def test_config2_full_size(device, n):
    c = wl.config2()
    got = run_c2(c, n, device)
    assert last_launch()["kernel"] == "rows"
    assert sha(got) == DIG[f"c2_full_n{n}"], f"config 2 N={n}: not bit-identical to the reference CPU backend"
    if n == 10:
        assert check_float(got, ol.oracle_add_mul_chain(c["src"], n, c["add"], c["mul"]), "config 2 vs oracle")
        assert np.array_equal(got, run_c2(c, n, device, tf=1)), "TF::ENABLED spelling must give identical results"


@pytest.mark.parametrize("n", [1, 2, 3, 10, 50, 100])
def test_config2_reduced_odd_width(device, n):
    c = wl.config2(**CASES["c2_small"])   # 250 x 64: exercises the row tail (250 % 4 != 0)
    assert check_float(run_c2(c, n, device), GOLD[f"c2_small_n{n}"], f"config 2 small N={n}")


# ---- configuration 3: DNN preprocessing batch -----------------------------------------------------------------------

def test_config3_full_size(device):
    c = wl.config3()
    got = run_c3(c, device)
    assert last_launch()["kernel"] == "strip"
    want = ol.oracle_crop_resize_norm_split(c["src"], c["rects"], c["dst"], c["sub"], c["div"])
    exact = check_float(got, want, "config 3 vs oracle")
    assert exact and sha(got) == DIG["c3_full"], "config 3 is expected to be bit-identical to the reference CPU backend"


def test_config3_reduced(device):
    c = wl.config3(**CASES["c3_small"])
    assert check_float(run_c3(c, device), GOLD["c3_small"], "config 3 small vs golden")


# ---- configuration 4: horizontal fusion of independent images -----------------------------------------------------

def test_config4_reduced(device):
    c = wl.config4(**CASES["c4_small"])   # width 322: not a multiple of 4, rows 966 bytes: unaligned kernel variant
    _, outs = run_c4(c, device)
    got = np.stack([o.cpu().numpy() for o in outs])
    assert check_u8(got, GOLD["c4_small"], "config 4 small vs golden")


def test_config4_full_size(device):
    import torch
    c = wl.config4()
    srcs, outs = run_c4(c, device)
    ll = last_launch()
    assert ll["kernel"] == "rows" and ll["grid"][2] == 100
    # planes 0 and 99 against the reference's digests, 3 planes against the oracle
    assert sha(outs[0].cpu().numpy()) == DIG["c4_full_plane0"]
    assert sha(outs[99].cpu().numpy()) == DIG["c4_full_plane99"]
    for i in (1, 50, 98):
        want = ol.oracle_batch_muladd_sat(c["srcs"][i:i + 1], c["mul"][i:i + 1], c["add"][i:i + 1])[0]
        assert check_u8(outs[i].cpu().numpy(), want, f"config 4 plane {i} vs oracle")
    # every plane against the same arithmetic done by torch on the GPU (mul, add, round-half-even, clamp)
    for i in range(100):
        m = torch.from_numpy(c["mul"][i]).to(device)
        a = torch.from_numpy(c["add"][i]).to(device)
        want = torch.clamp(torch.round(srcs[i].to(torch.float32) * m + a), 0, 255).to(torch.uint8)
        assert torch.equal(outs[i], want), f"plane {i}"
    h = hashlib.sha256()
    for o in outs:
        h.update(o.cpu().numpy().tobytes())
    assert h.hexdigest() == DIG["c4_full"]


# ---- configuration 5: video frame ------------------------------------------------------------------------------------

def test_config5_full_size(device):
    c = wl.config5()
    got = run_c5(c, device)
    assert last_launch()["kernel"] == "gather"
    want = ol.oracle_nv12_rgb_resize_split(c["nv12"], c["width"], c["height"], c["dst"], c["scale"])
    assert check_float(got, want, "config 5 vs oracle") and sha(got) == DIG["c5_full"]
    # exact 2x: every output equals the colour-converted even source pixel (times 1/255)
    y = c["nv12"][:c["height"]:2, ::2].astype(np.float32)
    assert got.shape == (3, 1080, 1920) and np.isfinite(got).all()
    v = c["nv12"][c["height"]:, 1::2][:, ::1].astype(np.float32)[:, :1920] - np.float32(128)
    r = (y + (v * np.float32(1.5748))).astype(np.float32) * c["scale"]
    assert np.allclose(got[0], r, rtol=1e-5, atol=1e-6)


def test_config5_reduced(device):
    for name in ("c5_small", "c5_odd"):
        c = wl.config5(**CASES[name])
        assert check_float(run_c5(c, device), GOLD[name], name)


# ---- integer-only chain ------------------------------------------------------------------------------------------------

def test_integer_only_chain_is_bit_exact(device):
    import torch
    c = wl.config1(width=640, height=360, seed=31)
    for rects in ([[3, 5, 77, 41], [100, 50, 77, 41], [201, 17, 77, 41], [563, 319, 77, 41]],      # odd origin: unaligned rows
                  [[0, 0, 64, 32], [4, 8, 64, 32], [128, 100, 64, 32], [576, 328, 64, 32]]):      # x origin % 4 == 0: wide rows
        rects = np.array(rects, np.int32)
        src = dev_u8(c["src"], device)
        out = torch.zeros((4, rects[0][3], rects[0][2], 3), dtype=torch.uint8, device=device)
        cases.crop_swap_u8(src, rects, out)
        torch.cuda.synchronize()
        want = ol.oracle_crop_swap_u8(c["src"], rects)
        assert np.array_equal(out.cpu().numpy(), want)
        for z, (x, y, w, h) in enumerate(rects):
            assert np.array_equal(want[z], c["src"][y:y + h, x:x + w, ::-1])
