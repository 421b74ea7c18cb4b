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


def test_a_batch_whose_parameters_exceed_the_kernel_argument_limit_is_a_compile_time_message():
    """The host executor bounds sizeof(Chain::Params), a compile-time constant, by FKLHIP_MAX_BLOB_BYTES: 45 000 planes of
    24-byte pointers twice over are 2 MB of by-value kernel arguments, which stops the build with a sentence."""
    src = os.path.join(ROOT, "tests", "cases", "api_compat.cpp")
    r = subprocess.run(["g++", "-std=c++20", "-fsyntax-only", "-DFK_API_COMPAT_HUGE_BATCH", "-I", os.path.join(ROOT, "include"), src],
                       capture_output=True, text=True)
    assert r.returncode != 0
    assert "exceed FKLHIP_MAX_BLOB_BYTES" in r.stderr and "smaller BATCH per launch" in r.stderr


def max_blob_bytes():
    text = open(os.path.join(ROOT, "include", "fklhip.h")).read()
    return int(re.search(r"#define\s+FKLHIP_MAX_BLOB_BYTES\s+(\d+)", text).group(1))


def test_a_parameter_block_above_the_limit_is_refused_before_it_reaches_the_runtime():
    lib = fkl.lib()
    limit = max_blob_bytes()
    assert 64 * 1024 <= limit <= 1024 * 1024
    sig = [s for s, _ in fkl.signatures() if s.startswith("Chain<Read2D<f32>,OpList<Add<f32,f32,f32>>,")][0]
    h = C.c_void_p()
    assert lib.fklhip_lookup(sig.encode(), C.byref(h)) == 0
    blob = (C.c_char * (limit + 1))()
    assert lib.fklhip_launch_handle(h, blob, limit + 1, None) == 10002
    assert b"FKLHIP_MAX_BLOB_BYTES" in lib.fklhip_error_string(10002)
    # every chain compiled into the library is far below it
    assert max(b for _, b in fkl.signatures()) <= limit


def test_strip_form_switch_round_trip():
    lib = fkl.lib()
    first = lib.fklhip_strip_form(-1)
    assert first in (0, 1)
    assert lib.fklhip_strip_form(0) == first and lib.fklhip_strip_form(-1) == 0
    assert lib.fklhip_strip_form(1) == 0 and lib.fklhip_strip_form(-1) == 1
    lib.fklhip_strip_form(first)


def test_an_output_without_columns_launches_nothing_in_either_form():
    """Configuration 3's chain with an active extent of 0 x 8 x 1: the strip form's grid (rows / 8 workgroups) would not be
    empty, so the launcher must not take it; the tile form's grid has no workgroup and nothing is launched (no GPU call is
    made, so this runs without one)."""
    lib = fkl.lib()
    sig, size = [(s, b) for s, b in fkl.signatures() if s.startswith("Chain<BatchRead<64,ResizeLinear<1,Crop<Read2D<Vec<u8,3>>>>>,OpList<Reorder<")][0]
    blob = (C.c_uint32 * (size // 4))()
    for w, h in ((0, 8), (0, 224), (8, 0)):
        blob[0], blob[1], blob[2], blob[3] = w, h, 1, 1      # active_w, active_h, active_z, strip form allowed
        for form in (1, 0):
            old = lib.fklhip_strip_form(form)
            try:
                assert lib.fklhip_launch(sig.encode(), blob, size, None) == 0
            finally:
                lib.fklhip_strip_form(old)
            ll = fkl.last_launch()
            assert ll["grid"][0] * ll["grid"][1] * ll["grid"][2] == 0, ll
