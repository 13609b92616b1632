"""The two measurement aids that stay in the kernel sources behind compile-time switches (-DHW_CLOCKS: phase timestamps
into a device buffer; -DHW_NO_COMPUTE: tiles are consumed but nothing is computed) are exercised by no GPU test, so at
least they have to keep compiling: device-only compile of the kernel translation units for gfx950, no GPU needed."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


@pytest.mark.parametrize("unit,flags", [
    ("hogwild_kernels.hip", ["-DHW_CLOCKS"]),
    ("hogwild_kernels.hip", ["-DHW_NO_COMPUTE"]),
    ("hogwild_wide.hip", ["-DHW_NO_COMPUTE"]),
])
def test_tuning_switches_still_compile(tmp_path, unit, flags):
    if shutil.which(HIPCC) is None and not os.path.exists(HIPCC):
        pytest.skip("no hipcc")
    from inference_lib_amd import build
    cmd = [HIPCC, f"--offload-arch={build.ARCH}", "-O1", "-std=c++17", "-fno-gpu-rdc", "--cuda-device-only", *build.DEVICE_FLAGS,
           "-I", os.path.join(ROOT, "include"), *flags, "-c", os.path.join(build.CSRC, unit), "-o", str(tmp_path / "unit.o")]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-3000:]
