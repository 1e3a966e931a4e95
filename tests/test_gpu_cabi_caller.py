"""The C ABI used without Python or torch: tests/cabi/c_caller.cpp (built by
__graft_entry__.build()) allocates with the HIP runtime, calls libminf_hip.so through
include/minf_hip.h only, and checks dense and vertical-slash attention, the index builder's
mask, the estimation's forced entries and an error status against host loops (tolerance
max-abs 2e-2 / mean-abs 1e-3 for the 16-bit outputs, stated in the program)."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

EXE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cabi", "c_caller")


def test_c_program_calls_the_library_directly(gpu):
    if not os.path.exists(EXE):
        pytest.fail("tests/cabi/c_caller has not been built (run __graft_entry__.build())")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for dep in (os.path.join(root, "include", "minf_hip.h"), os.path.join(root, "tests", "cabi", "c_caller.cpp")):
        # a program compiled against an older header would hand the library a struct of the wrong size
        if os.path.getmtime(dep) > os.path.getmtime(EXE):
            pytest.fail(f"tests/cabi/c_caller is older than {os.path.relpath(dep, root)}: run __graft_entry__.build()")
    r = subprocess.run([EXE], capture_output=True, text=True, timeout=120)
    print(r.stdout)
    print(r.stderr)
    assert r.returncode == 0, r.stderr
    assert "c_caller ok" in r.stdout
