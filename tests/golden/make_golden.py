"""Regenerates the golden fixtures from the REFERENCE library's own CPU backend (oracle/_ref/libfkl_ref.so, built
by oracle/Makefile from the reference headers).  Run in the build container:  python tests/golden/make_golden.py

Fixtures are data only: reduced-size outputs of the five benchmark chains (same operation chains, same seeds
scheme, smaller images) and SHA-256 digests of the full-size outputs.  The tests compare the plain-C oracle and
the HIP kernels against them, so they keep working where the reference tree is not present.
"""
from __future__ import annotations

import hashlib
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import oracle_lib as ol  # noqa: E402
import workloads as wl  # noqa: E402


def sha(a) -> str:
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def reduced_cases():
    """(name, kwargs for the workload generator).  Shared with the tests through golden_cases.json."""
    return {
        "c1_small": dict(width=640, height=360, seed=11),
        "c2_small": dict(width=250, height=64, seed=12),
        "c3_small": dict(batch=8, width=640, height=360, dst=96, seed=13, rect_seed=133, min_side=24, span=300),
        "c4_small": dict(batch=4, width=322, height=120, seed=14, param_seed=144),
        "c5_small": dict(width=256, height=144, dst=(128, 72), seed=15),
        "c5_odd": dict(width=256, height=144, dst=(100, 50), seed=16),
    }


C1_SMALL_RECTS = np.array([[30, 12, 60, 40], [400, 125, 60, 40], [330, 170, 130, 140], [500, 115, 100, 35], [572, 196, 40, 15]], np.int32)


def main():
    assert ol.have_ref(), "build oracle/_ref first (make -C oracle ref)"
    out = {}
    digests = {}
    cases = reduced_cases()

    c = wl.config1(**cases["c1_small"])
    out["c1_small"] = ol.ref_crop_resize_par_u8(c["src"], C1_SMALL_RECTS, c["dst"], c["bg"], c["mul"], c["sub"])
    c = wl.config2(**cases["c2_small"])
    for n in (1, 2, 3, 10, 50, 100):
        out[f"c2_small_n{n}"] = ol.ref_add_mul_chain(c["src"], n, c["add"], c["mul"])
    c = wl.config3(**cases["c3_small"])
    out["c3_small"] = ol.ref_crop_resize_norm_split(c["src"], c["rects"], c["dst"], c["sub"], c["div"])
    c = wl.config4(**cases["c4_small"])
    out["c4_small"] = np.stack(ol.ref_batch_muladd_sat(c["srcs"], c["mul"], c["add"]))
    for name in ("c5_small", "c5_odd"):
        c = wl.config5(**cases[name])
        out[name] = ol.ref_nv12_rgb_resize_split(c["nv12"], c["width"], c["height"], c["dst"], c["scale"])

    # full-size digests (and the oracle must agree bit for bit, or the fixtures are not written)
    c = wl.config1()
    r = ol.ref_crop_resize_par_u8(c["src"], c["rects"], c["dst"], c["bg"], c["mul"], c["sub"])
    assert sha(r) == sha(ol.oracle_crop_resize_par_u8(c["src"], c["rects"], c["dst"], c["bg"], c["mul"], c["sub"]))
    out["c1_full"] = r   # 122 880 bytes: small enough to keep whole
    digests["c1_full"] = sha(r)
    c = wl.config2()
    for n in c["n_ops_sweep"]:
        r = ol.ref_add_mul_chain(c["src"], n, c["add"], c["mul"])
        assert sha(r) == sha(ol.oracle_add_mul_chain(c["src"], n, c["add"], c["mul"]))
        digests[f"c2_full_n{n}"] = sha(r)
    c = wl.config3()
    r = ol.ref_crop_resize_norm_split(c["src"], c["rects"], c["dst"], c["sub"], c["div"])
    assert sha(r) == sha(ol.oracle_crop_resize_norm_split(c["src"], c["rects"], c["dst"], c["sub"], c["div"]))
    digests["c3_full"] = sha(r)
    digests["c3_rects"] = sha(c["rects"])
    c = wl.config5()
    r = ol.ref_nv12_rgb_resize_split(c["nv12"], c["width"], c["height"], c["dst"], c["scale"])
    assert sha(r) == sha(ol.oracle_nv12_rgb_resize_split(c["nv12"], c["width"], c["height"], c["dst"], c["scale"]))
    digests["c5_full"] = sha(r)
    c = wl.config4()
    r = ol.ref_batch_muladd_sat(c["srcs"], c["mul"], c["add"])
    digests["c4_full"] = sha(np.stack(r))
    digests["c4_full_plane0"] = sha(r[0])
    digests["c4_full_plane99"] = sha(r[99])
    assert sha(r[0]) == sha(ol.oracle_batch_muladd_sat(c["srcs"][:1], c["mul"][:1], c["add"][:1])[0])

    # small known-answer tables straight from the reference
    import ctypes as C
    m = (C.c_float * 9)()
    ol.ref().fklref_yuv2rgb_709_full_matrix(m)
    digests["bt709_full_matrix"] = [float(np.float32(v)) for v in m]
    vals = np.array([0.5, 1.5, 2.5, 3.5, 254.5, 255.5, -0.5, -3.0, np.nan, np.inf, -np.inf, 1e9, 127.49999, 0.49999997], np.float32)
    o = np.zeros(len(vals), np.uint8)
    ol.ref().fklref_saturate_cast_u8(vals.ctypes.data_as(C.c_void_p), len(vals), o.ctypes.data_as(C.c_void_p))
    digests["saturate_inputs"] = [repr(float(v)) for v in vals]
    digests["saturate_outputs"] = [int(v) for v in o]
    geo = {}
    for sw, sh in ((60, 40), (130, 140), (100, 35), (40, 15), (1920, 1080), (7, 300), (300, 7)):
        o4 = (C.c_int32 * 4)()
        f2 = (C.c_float * 2)()
        ol.ref().fklref_resize_params_par(sw, sh, 128, 64, o4, f2)
        geo[f"{sw}x{sh}->128x64"] = {"rect": list(o4), "fx": float(np.float32(f2[0])), "fy": float(np.float32(f2[1]))}
    digests["letterbox"] = geo

    np.savez_compressed(os.path.join(HERE, "golden_outputs.npz"), **out)
    with open(os.path.join(HERE, "golden_digests.json"), "w") as f:
        json.dump({"cases": cases, "c1_small_rects": C1_SMALL_RECTS.tolist(), "digests": digests}, f, indent=1, sort_keys=True)
    print("wrote", len(out), "arrays and", len(digests), "digests")


if __name__ == "__main__":
    main()
