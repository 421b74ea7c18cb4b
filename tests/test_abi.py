"""CPU tests of the drop-in boundary: libfklhip.so loads, exports every symbol include/fklhip.h declares, knows the
benchmark chains, and rejects bad requests without touching a GPU."""
import ctypes as C
import os
import re
import subprocess

import pytest

import fusedkernellibrary_amd as fkl

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "fklhip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fklhip_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = fkl.lib()
    names = declared_symbols()
    assert len(names) >= 25
    for name in names:
        assert hasattr(lib, name), f"{name} is declared in include/fklhip.h but not exported"
    assert set(names) == set(fkl.ABI_SYMBOLS)
    assert lib.fklhip_abi_version() == 1


def test_benchmark_chains_are_compiled_in():
    sigs = dict(fkl.signatures())
    assert len(sigs) >= 13
    want = [
        "Chain<BatchRead<5,ResizeLinear<0,Crop<Read2D<Vec<u8,3>>>>>,OpList<Mul<",          # configuration 1
        "Chain<Read2D<f32>,OpList<Add<f32,f32,f32>>,Write2D<f32>>",                          # configuration 2, N = 1
        "Chain<BatchRead<64,ResizeLinear<1,Crop<Read2D<Vec<u8,3>>>>>,OpList<Reorder<",      # configuration 3
        "Chain<BatchRead<100,FusedRead<Read2D<Vec<u8,3>>,Mul<",                              # configuration 4
        "Chain<ResizeLinear<1,FusedRead<ReadNV12,YUV2RGB<0,1,1>>>,OpList<Mul<Vec<f32,3>,f32,Vec<f32,3>>>,TensorSplit<",  # 5
    ]
    for prefix in want:
        assert any(s.startswith(prefix) for s in sigs), prefix
    # parameter block of configuration 3: 16-byte header + 64 planes + (empty reorder, sub, div) + tensor
    c3 = [b for s, b in sigs.items() if s.startswith("Chain<BatchRead<64,")][0]
    assert 64 * 64 <= c3 <= 8192


def test_unknown_signature_and_bad_blob_are_reported_without_a_gpu():
    lib = fkl.lib()
    blob = (C.c_char * 64)()
    rc = lib.fklhip_launch(b"Chain<NoSuchRead,OpList<>,NoSuchWrite>", blob, 64, None)
    assert rc == 10001
    assert b"signature" in lib.fklhip_error_string(rc)
    sig = [s for s, _ in fkl.signatures() if s.startswith("Chain<Read2D<f32>,OpList<Add<f32,f32,f32>>,")][0]
    assert lib.fklhip_launch(sig.encode(), blob, 7, None) == 10002
    assert lib.fklhip_launch(sig.encode(), None, 72, None) == 10003
    h = C.c_void_p()
    assert lib.fklhip_lookup(None, C.byref(h)) == 10003
    assert lib.fklhip_launch_handle(None, blob, 64, None) == 10003


def test_host_api_translation_unit_compiles_and_resolves_signatures():
    """The case drivers are written against include/fused_kernel/ exactly like user code of the reference library;
    compiling them with plain g++ (no HIP headers on the include path) is the source-compatibility check."""
    src = os.path.join(ROOT, "tests", "cases", "api_compat.cpp")
    r = subprocess.run(["g++", "-std=c++20", "-fsyntax-only", "-I", os.path.join(ROOT, "include"), src],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]


def test_launching_a_user_defined_operation_without_a_lowering_is_a_compile_time_message():
    """A reference-style user Operation (Parent + DECLARE_*_PARENT + exec) compiles and fuses; asking the GPU executor to
    launch it stops the build with the sentence that says what is missing, not with a template error."""
    src = os.path.join(ROOT, "tests", "cases", "api_compat.cpp")
    r = subprocess.run(["g++", "-std=c++20", "-fsyntax-only", "-DFK_API_COMPAT_LAUNCH_USER_OP", "-I", os.path.join(ROOT, "include"), src],
                       capture_output=True, text=True)
    assert r.returncode != 0
    assert "this Operation has no MI355X lowering: specialise fk::amd::Lower<Operation>" in r.stderr
