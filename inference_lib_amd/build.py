"""In-tree build of the native pieces for gfx950.

  libhogwild_hip.so ... HIP kernels + the C ABI declared in include/hogwild_hip.h
  hogatt.abi3.so ...... torch operator binding (namespace libhogatt) on top of the C ABI
  libhogwild_bench.so . calibration kernels of the measurement harness (include/hogwild_bench.h), not part of the product

Run as `python -m inference_lib_amd.build`.  hipcc cross-compiles for gfx950 without a GPU present.
"""
from __future__ import annotations

import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libhogwild_hip.so")
TORCH_EXT = os.path.join(HERE, "hogatt.abi3.so")
BENCH_LIB = os.path.join(HERE, "libhogwild_bench.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
# packed fp32 VALU ops are switched off for every device compile of this library; MFMA accumulators are kept in
# architectural VGPRs (the attention kernel touches them with VALU ops, and shuttling them to and from the
# accumulation registers cost more instructions than the arithmetic)
DEVICE_FLAGS = ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-mllvm", "-amdgpu-mfma-vgpr-form"]


def _run(cmd):
    print("+", " ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)


def build_library() -> str:
    srcs = [os.path.join(CSRC, n) for n in ("hogwild_kernels.hip", "hogwild_wide.hip", "hogwild_paged.hip", "hogwild_cache.hip", "hogwild_capi.hip", "hogwild_plan.cpp")]
    cmd = [HIPCC, f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-shared", "-fno-gpu-rdc",
           "-munsafe-fp-atomics", *DEVICE_FLAGS, "-I", os.path.join(ROOT, "include"), "-o", LIB, *srcs]
    _run(cmd)
    return LIB


def build_bench_library() -> str:
    cmd = [HIPCC, f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-shared", "-fno-gpu-rdc", *DEVICE_FLAGS,
           "-I", os.path.join(ROOT, "include"), "-o", BENCH_LIB, os.path.join(CSRC, "hogwild_bench.hip")]
    _run(cmd)
    return BENCH_LIB


def build_torch_binding() -> str:
    import torch
    from torch.utils import cpp_extension

    inc = cpp_extension.include_paths()
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           "-I", os.path.join(ROOT, "include"), "-I", "/opt/rocm/include", "-I", sysconfig.get_paths()["include"]]
    for i in inc:
        cmd += ["-isystem", i]
    cmd += [os.path.join(CSRC, "hogatt_binding.cpp"), "-o", TORCH_EXT,
            "-L", HERE, "-lhogwild_hip", "-L", torch_lib, "-ltorch", "-ltorch_cpu", "-lc10", "-lc10_hip", "-ltorch_hip",
            "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{torch_lib}"]
    _run(cmd)
    return TORCH_EXT


C_EXAMPLE = os.path.join(ROOT, "tests", "c_abi", "decode_step")


def build_c_example() -> str:
    """A caller of the C ABI in plain C (tests/c_abi/decode_step.c), linked against the library and the HIP runtime."""
    cmd = ["gcc", "-std=c11", "-O1", "-Wall", "-D__HIP_PLATFORM_AMD__=1", "-I", os.path.join(ROOT, "include"), "-I", "/opt/rocm/include",
           os.path.join(ROOT, "tests", "c_abi", "decode_step.c"), "-o", C_EXAMPLE, "-L", HERE, "-lhogwild_hip",
           "-L", "/opt/rocm/lib", "-lamdhip64", "-lm", "-Wl,-rpath,$ORIGIN/../../inference_lib_amd", "-Wl,-rpath,/opt/rocm/lib"]
    _run(cmd)
    return C_EXAMPLE


def build_all(with_torch: bool = True) -> None:
    build_library()
    build_bench_library()
    build_c_example()
    if with_torch:
        build_torch_binding()


if __name__ == "__main__":
    build_all(with_torch="--no-torch" not in sys.argv)
