"""The host-only part of the library (validation, split planning: inference_lib_amd/csrc/hogwild_plan.cpp) built with plain g++
under AddressSanitizer + UndefinedBehaviorSanitizer and fuzzed with random problems (tests/host_fuzz/plan_fuzz.cpp).  CPU only."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("seed", [1, 2])
def test_planner_and_validators_under_sanitizers(tmp_path, seed):
    if shutil.which("g++") is None:
        pytest.skip("no g++")
    exe = str(tmp_path / "plan_fuzz")
    cmd = ["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-static-libasan",
           "-I", os.path.join(ROOT, "include"), os.path.join(ROOT, "tests", "host_fuzz", "plan_fuzz.cpp"),
           os.path.join(ROOT, "inference_lib_amd", "csrc", "hogwild_plan.cpp"), "-o", exe]
    subprocess.run(cmd, check=True)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    r = subprocess.run([exe, "1500", str(seed)], capture_output=True, text=True, env=env, timeout=300)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]
    assert "0 failures" in r.stdout
