"""Host-side use of the API the way the reference's unit tests use it: Operation::exec on one value on the calling thread,
the ArrayVector / toArray / transformArray helpers, the colour constants (tests/cases/host_values.cpp, compiled here with
plain g++ and run).  Its checks are closed forms and the constants the ITU recommendations print.  No GPU."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_operations_and_array_helpers_on_the_host(tmp_path):
    exe = str(tmp_path / "host_values")
    lib = os.path.join(ROOT, "fusedkernellibrary_amd")
    r = subprocess.run(["g++", "-std=c++20", "-O1", "-ffp-contract=off", "-I", os.path.join(ROOT, "include"),
                        os.path.join(ROOT, "tests", "cases", "host_values.cpp"), "-o", exe,
                        "-L", lib, "-lfklhip", "-Wl,-rpath," + lib], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]
    r = subprocess.run([exe], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0 and "all checks passed" in r.stdout, r.stdout + r.stderr
