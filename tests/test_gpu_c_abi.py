"""The C ABI called from plain C (tests/c_abi/decode_step.c, built by `python -m inference_lib_amd.build`): no Python,
no torch and no C++ between the caller and the library.  The program checks the fused and the paged step against closed
forms (uniform attention) itself; this test runs it."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "c_abi", "decode_step")


@pytest.mark.gpu
def test_plain_c_caller():
    assert os.path.exists(EXE), "tests/c_abi/decode_step is not built (python -m inference_lib_amd.build)"
    r = subprocess.run([EXE], capture_output=True, text=True, timeout=120)
    print(r.stdout, r.stderr, flush=True)
    assert r.returncode == 0, (r.returncode, r.stdout, r.stderr)
    assert "c_abi ok" in r.stdout


def test_plain_c_caller_links_against_the_library_only():
    """No GPU needed: the program's dynamic dependencies are the library, the HIP runtime and libc/libm."""
    if not os.path.exists(EXE):
        pytest.skip("not built")
    out = subprocess.run(["readelf", "-d", EXE], capture_output=True, text=True).stdout
    needed = [l.split("[")[1].split("]")[0] for l in out.splitlines() if "(NEEDED)" in l]
    assert "libhogwild_hip.so" in needed
    assert not any("torch" in n or "c10" in n or "stdc++" in n for n in needed), needed
