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
    ("hogwild_wide.hip", ["-DHW_CLOCKS"]),
])
def test_tuning_switches_still_compile(tmp_path, unit, flags):
    if shutil.which(HIPCC) is None and not os.path.exists(HIPCC):
        pytest.skip("no hipcc")
    from inference_lib_amd import build
    cmd = [HIPCC, f"--offload-arch={build.ARCH}", "-O1", "-std=c++17", "-fno-gpu-rdc", "--cuda-device-only", *build.DEVICE_FLAGS,
           "-I", os.path.join(ROOT, "include"), *flags, "-c", os.path.join(build.CSRC, unit), "-o", str(tmp_path / "unit.o")]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-3000:]


def test_tile_loops_of_the_128_row_kernels_wait_only_for_their_own_transfers(tmp_path):
    """The 128-row kernels issue their global->LDS tile transfers from inline assembly and count them by hand (s_waitcnt
    vmcnt(n) in front of each barrier, n = the transfers of the look-ahead that may stay in flight).  The compiler does not
    know of them, and every wait it inserts itself for one of ITS loads inside a tile loop -- vmcnt(0), vmcnt(1): it counts
    only the loads it knows -- also waits for the look-ahead tiles and empties the pipeline at every tile; it has done so
    when a load's only use sat under a condition in front of the loop and the wait was left to the next touch of the
    register, and when a register spilled in front of the loop was reloaded there.  Checked in the generated code: inside
    the innermost loops of both kernels no wait for vector memory below the look-ahead, and no scratch memory at all."""
    if shutil.which(HIPCC) is None and not os.path.exists(HIPCC):
        pytest.skip("no hipcc")
    import re
    from inference_lib_amd import build
    asm = tmp_path / "wide.s"
    cmd = [HIPCC, f"--offload-arch={build.ARCH}", "-O3", "-std=c++17", "-fno-gpu-rdc", "-munsafe-fp-atomics", "--cuda-device-only",
           *build.DEVICE_FLAGS, "-I", os.path.join(ROOT, "include"), "-S", os.path.join(build.CSRC, "hogwild_wide.hip"), "-o", str(asm)]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=900)
    assert r.returncode == 0, r.stderr[-3000:]
    text = asm.read_text()
    kernels = re.findall(r"^(_ZN2hw(?:17paged_wide_kernel|21attention_wide_kernel)\S*):", text, re.M)
    assert len(kernels) >= 12, kernels
    checked = 0
    for name in kernels:
        body = text[text.index(name + ":"):]
        end = body.index("; -- End function")
        # (a register spilled anywhere is reloaded with a wait for "all loads", which in front of the tile loops also waits
        # for the first tiles' transfers)
        scratch = re.search(r"; ScratchSize: (\d+)", body[end:end + 4000])
        assert scratch and int(scratch.group(1)) == 0, f"{name}: {scratch and scratch.group(0)}"
        body = body[:end]
        parts = re.split(r"\n(\.LBB\d+_\d+):", body)
        for label, block in zip(parts[1::2], parts[2::2]):
            if "Depth=2" not in block:
                continue                                   # not inside a tile loop (the loop over fragments / segments is depth 1)
            # a wave issues E / (8 * waves) transfers per tile (K + V bytes of a tile / 1 KB / waves), a step is `par` tiles
            # requested behind the barrier, and one step stays in flight; head dimension, ring slots, waves and tiles per
            # step from the name
            m = re.search(r"attention_wide_kernel\S*?ELi(\d+)ELi\d+ELi(\d+)ELb[01]ELi(\d+)ELi(\d+)E", name) or \
                re.search(r"paged_wide_kernel\S*?ELi(\d+)ELi\d+ELi(\d+)ELi(\d+)ELi(\d+)E", name)
            assert m, name
            e, ns, nw, par = (int(x) for x in m.groups())
            ahead = (ns // par - 2) * par * e // (8 * nw)
            assert ahead >= 1, name
            assert "scratch_" not in block, f"{name} {label}: scratch memory inside a tile loop"
            for m in re.finditer(r"s_waitcnt[^\n]*vmcnt\((\d+)\)", block):
                checked += 1
                assert int(m.group(1)) >= ahead, f"{name} {label}: {m.group(0)} inside a tile loop"
    assert checked >= 2 * len(kernels)                    # every kernel has its own hand-counted waits there
    # Outside the tile loops: a wait the COMPILER places (outside the inline-assembly brackets) behind transfers of the
    # same block must leave those in flight -- the rotation of the queries runs beside the look-ahead steps requested just
    # before it.
    for name in kernels:
        body = text[text.index(name + ":"):]
        body = body[:body.index("; -- End function")]
        parts = re.split(r"\n(\.LBB\d+_\d+):", body)
        for label, block in zip(["entry"] + parts[1::2], parts[0::2]):
            issued, in_asm = 0, False
            for line in block.splitlines():
                if "#ASMSTART" in line:
                    in_asm = True
                elif "#ASMEND" in line:
                    in_asm = False
                elif re.search(r"(buffer_load_dwordx4|global_load_lds_dwordx4)[^\n]*\b(lds|nt)\b", line) and in_asm:
                    issued += 1
                elif not in_asm:
                    m = re.search(r"s_waitcnt[^\n]*vmcnt\((\d+)\)", line)
                    assert not (m and issued and int(m.group(1)) < issued), f"{name} {label}: {line.strip()} behind {issued} transfers"


def test_one_buffer_kernels_wait_for_the_transfers_of_the_tile_they_multiply(tmp_path):
    """The fp32 kernels keep one K tile per wave in LDS: a tile is requested (global->LDS transfers, then the V loads into
    registers) and multiplied right away, so between a tile's last transfer and the first operand read out of LDS there
    has to be a wait that leaves at most the loads issued behind the transfers in flight.  The compiler derives that wait
    from its own count of the operations in flight and stopped placing it when a tile became 64 of them (256-wide fp32
    rows: 32 transfers + 32 loads); the kernel states it itself there.  Checked in the generated code of every
    one-buffer instantiation."""
    if shutil.which(HIPCC) is None and not os.path.exists(HIPCC):
        pytest.skip("no hipcc")
    import re
    from inference_lib_amd import build
    asm = tmp_path / "kernels.s"
    cmd = [HIPCC, f"--offload-arch={build.ARCH}", "-O3", "-std=c++17", "-fno-gpu-rdc", "-munsafe-fp-atomics", "--cuda-device-only",
           *build.DEVICE_FLAGS, "-I", os.path.join(ROOT, "include"), "-S", os.path.join(build.CSRC, "hogwild_kernels.hip"), "-o", str(asm)]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=900)
    assert r.returncode == 0, r.stderr[-3000:]
    text = asm.read_text()
    # attention_kernel<DT, E, EV, RB, MINW, PF, ...>: PF == 1 is the one-buffer form
    kernels = re.findall(r"^(_ZN2hw16attention_kernelINS_\w+?ELi\d+ELi\d+ELi\d+ELi\d+ELi1ELb\S*):", text, re.M)
    assert len(kernels) >= 12 and any("ELi256ELi256" in k for k in kernels), kernels
    groups = 0
    for name in kernels:
        body = text[text.index(name + ":"):]
        body = body[:body.index("; -- End function")]
        pending, younger = False, 0
        for line in body.splitlines():
            t = line.strip()
            if re.match(r"buffer_load_dwordx4 .*\blds\b", t):
                if not pending:
                    groups += 1
                pending, younger = True, 0
            elif re.match(r"(global|buffer)_load_", t):
                younger += 1
            elif t.startswith("s_waitcnt"):
                m = re.search(r"vmcnt\((\d+)\)", t)
                if m and int(m.group(1)) <= younger:
                    pending = False
            elif t.startswith("ds_read"):
                assert not pending, f"{name}: {t} with the tile's transfers possibly in flight ({younger} loads behind them)"
    assert groups >= len(kernels)
