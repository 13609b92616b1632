"""Host-side checks of the C ABI that need no GPU: the shared library loads, exports every symbol the header
declares, rejects bad arguments before touching a device, and plans the split sensibly."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _lib():
    from inference_lib_amd import _lib
    return _lib


def test_library_exports_every_declared_symbol():
    L = _lib()
    header = open(os.path.join(ROOT, "include", "hogwild_hip.h")).read()
    declared = set(re.findall(r"^\s*(?:int|const char\*)\s+(hw_\w+)\s*\(", header, flags=re.M))
    assert declared, "no declarations found in the header"
    assert declared == set(L.EXPORTS), (declared ^ set(L.EXPORTS))
    for name in declared:
        assert hasattr(L.lib, name), name
    assert L.lib.hw_version() == 6 == L.HW_ABI_VERSION
    # constants the ctypes mirror repeats
    for name in ("HW_ABI_VERSION", "HW_MAX_FRAGMENTS", "HW_MAX_LAUNCH_FRAGMENTS", "HW_MAX_SPLITS"):
        m = re.search(rf"#define\s+{name}\s+(\d+)", header)
        assert m and int(m.group(1)) == getattr(L, name), name
    m = re.search(r"#define\s+HW_STATIC_SCRATCH_BYTES\s+\((\d+)u\s*<<\s*(\d+)\)", header)
    assert m and int(m.group(1)) << int(m.group(2)) == L.HW_STATIC_SCRATCH_BYTES


def test_calibration_kernels_live_in_their_own_library():
    """What only the benchmark needs is not part of the product ABI: libhogwild_bench.so exports what
    include/hogwild_bench.h declares, and the product library exports none of it (no event or stream helpers either)."""
    L = _lib()
    header = open(os.path.join(ROOT, "include", "hogwild_bench.h")).read()
    declared = set(re.findall(r"^\s*int\s+(hw_\w+)\s*\(", header, flags=re.M))
    assert declared == {"hw_stream_read", "hw_stream_read_shaped", "hw_stream_copy"}, declared
    bench = C.CDLL(os.path.join(ROOT, "inference_lib_amd", "libhogwild_bench.so"))
    for name in declared:
        assert hasattr(bench, name), name
        assert not hasattr(L.lib, name), f"{name} leaked into the product library"
    for name in ("hw_event_create", "hw_event_record", "hw_event_elapsed_ms", "hw_stream_create"):
        assert not hasattr(L.lib, name), name


def test_struct_layout_matches_header():
    """ctypes mirror and C struct must agree; sizeof is probed through a tiny C program when gcc is around."""
    import shutil
    import subprocess
    import tempfile
    L = _lib()
    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    with tempfile.TemporaryDirectory() as d:
        src = os.path.join(d, "s.c")
        open(src, "w").write('#include <stdio.h>\n#include <stddef.h>\n#include "hogwild_hip.h"\nint main(){printf("%zu %zu %zu %zu %zu\\n",'
                             'sizeof(hw_problem),sizeof(hw_plan),offsetof(hw_problem,workspace),offsetof(hw_problem,len_dev),'
                             'offsetof(hw_plan,workspace_bytes));return 0;}\n')
        exe = os.path.join(d, "s")
        subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), src, "-o", exe], check=True)
        out = subprocess.run([exe], check=True, capture_output=True, text=True).stdout.split()
    assert int(out[0]) == C.sizeof(L.HwProblem)
    assert int(out[1]) == C.sizeof(L.HwPlan)
    assert int(out[2]) == L.HwProblem.workspace.offset
    assert int(out[3]) == L.HwProblem.len_dev.offset
    assert int(out[4]) == L.HwPlan.workspace_bytes.offset


def _problem(L, **over):
    F = over.pop("F", 2)
    p = L.HwProblem()
    p.dtype, p.F, p.W, p.Hq, p.Hkv, p.S, p.E, p.Ev, p.RotE = L.HW_BF16, F, 2, 8, 2, 1, 128, 128, 128
    p.scale = 0.1
    fake = 0x1000                                   # never dereferenced on the host
    for f in ("out", "q", "locations", "cosines", "sines"):
        setattr(p, f, fake)
    k = (C.c_void_p * F)(*[fake] * F)
    lens = (C.c_int32 * F)(*([64] * F))
    p.k = C.cast(k, C.POINTER(C.c_void_p))
    p.v = C.cast(k, C.POINTER(C.c_void_p))
    p.len = C.cast(lens, C.POINTER(C.c_int32))
    p._keep = (k, lens)
    for key, val in over.items():
        setattr(p, key, val)
    return p


def test_validation_happens_on_the_host():
    L = _lib()
    v = lambda p, fused=1: L.lib.hw_validate(C.byref(p), fused)
    assert v(_problem(L)) == 0
    assert L.lib.hw_validate(None, 1) == -1
    assert v(_problem(L, dtype=7)) == -2
    assert v(_problem(L, Hq=7)) == -3                       # not a multiple of Hkv
    assert v(_problem(L, W=0)) == -3
    assert v(_problem(L, RotE=130)) == -3                   # wider than the head
    assert v(_problem(L, RotE=63)) == -3                    # odd
    assert v(_problem(L, scale=float("nan"))) == -3
    assert v(_problem(L, scale=-1.0)) == -3
    assert v(_problem(L, E=96, Ev=96, RotE=96)) == -4       # valid but not instantiated: a hard error, never silent
    assert v(_problem(L, Ev=64)) == -4
    assert v(_problem(L, E=256, Ev=256, RotE=256)) == 0     # head dimension 256: the kernels with one 16-row block
    assert v(_problem(L, E=256, Ev=256, RotE=256, variant=1)) == -4
    assert v(_problem(L, E=512, Ev=512, RotE=512)) == -4
    assert v(_problem(L, F=65)) == 0                        # beyond one launch's 64 fragments: several launches
    assert v(_problem(L, F=512)) == 0 and v(_problem(L, F=513)) == -5
    assert v(_problem(L, F=65, len_dev=0x1000)) == -4       # device-resident lengths: one launch only
    assert v(_problem(L, F=65, variant=1)) == -4
    assert v(_problem(L, F=0)) == -5
    assert v(_problem(L, out=None)) == -1
    assert v(_problem(L, cosines=None)) == -1
    assert v(_problem(L, cosines=None), fused=0) == 0       # the pre-rotated entry needs no tables
    assert v(_problem(L, q=0x1004)) == -7                   # misaligned
    p = _problem(L)
    p.len[1] = -5
    assert v(p) == -3
    # the launching entry points run the same checks first, so these fail without any device present
    assert L.lib.hw_fused_attention(C.byref(_problem(L, dtype=9)), None) == -2
    assert L.lib.hw_sdpa(C.byref(_problem(L, Hq=7)), None) == -3
    assert L.lib.hw_rope(None, None, None, None, L.HW_BF16, 1, 1, 1, 1, 128, 128, None) == -1
    assert L.lib.hw_rope(0x1000, 0x1000, 0x1000, 0x1000, 5, 1, 1, 1, 1, 128, 128, None) == -2
    assert b"fragment" in L.lib.hw_status_string(-5)
    assert L.status_string(0) == "ok"


@pytest.mark.parametrize("lens,kw", [
    ([4096] + [2048] * 4 + [41, 16, 110, 73], dict(W=4, S=1, Hq=40, Hkv=8, Ev=128)),
    ([2048, 1024, 1024], dict(W=2, S=1, Hq=28, Hkv=4, Ev=128)),
    ([16384] + [3000, 17, 4000, 250, 1, 999, 2048, 3333] + [1] * 8, dict(W=8, S=1, Hq=32, Hkv=8, Ev=128)),
    ([8192] + [2048] * 4, dict(W=4, S=4, Hq=64, Hkv=8, Ev=128)),
    ([256, 64, 64], dict(W=2, S=1, Hq=8, Hkv=2, Ev=64)),
    ([0, 5, 0], dict(W=1, S=1, Hq=2, Hkv=1, Ev=64)),
    ([0], dict(W=1, S=1, Hq=2, Hkv=1, Ev=64)),
    ([1] * 32, dict(W=2, S=1, Hq=4, Hkv=2, Ev=128)),
])
def test_plan_invariants(lens, kw):
    L = _lib()
    for cus in (1, 8, 256, 304):
        for splits in (0, 1, 5, 1000):
            pl = L.plan(lens, num_cus=cus, splits=splits, **kw)
            G = kw["Hq"] // kw["Hkv"]
            assert pl.rows == kw["W"] * kw["S"] * G
            assert pl.row_blocks in (1, 2, 8) and pl.row_groups * 16 * pl.row_blocks >= pl.rows
            tiles = sum((x + 31) // 32 for x in lens)
            assert pl.tiles_per_head == tiles
            tb = list(pl.tile_begin)
            assert tb[0] == 0 and tb[len(lens)] == tiles and all(a <= b for a, b in zip(tb, tb[1:]))
            n = pl.wgs_per_head
            assert 1 <= n <= 256 and n <= max(tiles, 1)
            wb = list(pl.wg_tile_begin)[: n + 1]
            assert wb[0] == 0 and wb[-1] == tiles
            assert all(a < b for a, b in zip(wb, wb[1:])) or tiles == 0          # every workgroup owns at least one tile
            assert pl.workgroups == n * kw["Hkv"] * pl.row_groups
            assert pl.workspace_bytes >= kw["Hkv"] * n * pl.rows * (kw["Ev"] + 2) * 4


def test_device_length_entry_points_validate_on_the_host():
    L = _lib()
    # device-resident lengths exist for the fused entry with full rotary width only
    assert L.lib.hw_validate(C.byref(_problem(L, len_dev=0x1000)), 1) == 0
    assert L.lib.hw_validate(C.byref(_problem(L, len_dev=0x1000)), 0) == -4
    assert L.lib.hw_validate(C.byref(_problem(L, len_dev=0x1000, RotE=64)), 1) == -4
    orders = (C.c_int32 * 6)(0, 1, 2, 0, 2, 1)
    bi = lambda o, F=3, W=2, **kw: L.lib.hw_build_inputs_dev(kw.get("loc", 0x1000), 0x1000, 0x1000, kw.get("ld", 0x1000), o, 0x1000,
                                                            1.0, kw.get("rd", 0), F, W, 1, kw.get("rot", 64), None)
    assert bi(None) == -1 and bi(orders, loc=None) == -1 and bi(orders, ld=None) == -1
    assert bi(orders, rd=7) == -2 and bi(orders, rot=63) == -3 and bi(orders, F=65) == -3
    assert bi((C.c_int32 * 6)(0, 1, 1, 0, 2, 1)) == -3            # a fragment twice in one worker's order
    assert bi((C.c_int32 * 6)(0, 1, 3, 0, 2, 1)) == -3            # not a fragment
    add = (C.c_int32 * 3)(0, 1, 1)
    assert L.lib.hw_advance_lengths(None, add, 3, None) == -1 and L.lib.hw_advance_lengths(0x1000, None, 3, None) == -1
    assert L.lib.hw_advance_lengths(0x1000, add, 0, None) == -5 and L.lib.hw_advance_lengths(0x1000, add, 65, None) == -5


def test_plan_spreads_tiny_fragments():
    """Opening a fragment has a fixed cost, so a run of tiny fragments must not end up in one workgroup."""
    L = _lib()
    lens = [4096] + [2048] * 4 + [41, 16, 110, 73]
    pl = L.plan(lens, W=4, S=1, Hq=40, Hkv=8, Ev=128, num_cus=256)
    wb = list(pl.wg_tile_begin)[: pl.wgs_per_head + 1]
    tb = list(pl.tile_begin)[: len(lens) + 1]
    worst = 0
    for a, b in zip(wb, wb[1:]):
        worst = max(worst, sum(1 for f in range(len(lens)) if max(a, tb[f]) < min(b, tb[f + 1])))
    assert worst <= 2


def test_no_fallback_when_library_is_missing(tmp_path, monkeypatch):
    """The product path must fail loudly without the HIP library: importing the ctypes layer from a copy of the
    package that has no libhogwild_hip.so raises ImportError."""
    import shutil
    import subprocess
    import sys
    pkg = tmp_path / "inference_lib_amd"
    pkg.mkdir()
    for name in ("__init__.py", "_lib.py", "attention.py", "cases.py"):
        shutil.copy(os.path.join(ROOT, "inference_lib_amd", name), pkg / name)
    r = subprocess.run([sys.executable, "-c", "import inference_lib_amd.attention"], cwd=tmp_path, capture_output=True, text=True,
                       env={**os.environ, "PYTHONPATH": str(tmp_path)})
    assert r.returncode != 0 and "libhogwild_hip.so" in r.stderr


# ------------------------------------------------------------------------------------------------ paged entry points
def test_paged_struct_layouts_match_header():
    import shutil
    import subprocess
    import tempfile
    L = _lib()
    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    with tempfile.TemporaryDirectory() as d:
        src = os.path.join(d, "s.c")
        open(src, "w").write('#include <stdio.h>\n#include <stddef.h>\n#include "hogwild_hip.h"\nint main(){printf("%zu %zu %zu %zu %zu %zu %zu\\n",'
                             'sizeof(hw_paged_problem),sizeof(hw_paged_plan),sizeof(hw_copy_blocks),offsetof(hw_paged_problem,cu_seqlens_q),'
                             'offsetof(hw_paged_problem,row_blocks),offsetof(hw_copy_blocks,vs_s),offsetof(hw_copy_blocks,seq_lengths));return 0;}\n')
        exe = os.path.join(d, "s")
        subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), src, "-o", exe], check=True)
        out = [int(x) for x in subprocess.run([exe], check=True, capture_output=True, text=True).stdout.split()]
    assert out == [C.sizeof(L.HwPagedProblem), C.sizeof(L.HwPagedPlan), C.sizeof(L.HwCopyBlocks), L.HwPagedProblem.cu_seqlens_q.offset,
                   L.HwPagedProblem.row_blocks.offset, L.HwCopyBlocks.vs_s.offset, L.HwCopyBlocks.seq_lengths.offset]


def _paged(L, **over):
    p = L.HwPagedProblem()
    p.dtype, p.F, p.W, p.Hq, p.Hkv, p.E, p.Ev, p.S = L.HW_BF16, 1, 4, 40, 8, 128, 128, 1
    p.block_size, p.max_blocks, p.num_blocks = 16, 256, 2000
    p.scale = 0.1
    for f in ("out", "q", "locations", "fragment_lengths", "key_cache", "value_cache", "block_table"):
        setattr(p, f, 0x1000)                       # never dereferenced on the host
    for key, val in over.items():
        setattr(p, key, val)
    return p


def test_paged_validation_happens_on_the_host():
    L = _lib()
    v = lambda p: L.lib.hw_paged_validate(C.byref(p))
    assert v(_paged(L)) == 0
    assert L.lib.hw_paged_validate(None) == -1
    assert v(_paged(L, dtype=5)) == -2
    assert v(_paged(L, F=0)) == -5 and v(_paged(L, F=65)) == 0 and v(_paged(L, F=513)) == -5
    assert v(_paged(L, Hq=41)) == -3
    assert v(_paged(L, scale=0.0)) == -3 and v(_paged(L, scale=float("nan"))) == -3
    assert v(_paged(L, block_size=0)) == -3 and v(_paged(L, block_size=4096)) == -3
    assert v(_paged(L, max_blocks=70000)) == -3                      # more than 2^20 positions per sequence
    assert v(_paged(L, num_blocks=1 << 25)) == -3                    # 2^31 cache rows
    assert v(_paged(L, key_cache=None)) == -1
    assert v(_paged(L, q=0x1008)) == -7
    assert v(_paged(L, E=96, Ev=96)) == -4
    assert v(_paged(L, S=0)) == -3
    assert v(_paged(L, S=0, total_q=77, cu_seqlens_q=0x1000)) == 0   # the variable-length operator ignores S
    # entry points reject the wrong operator before any device work
    assert L.lib.hw_paged_sdpa(C.byref(_paged(L, cu_seqlens_q=0x1000)), None) == -3
    assert L.lib.hw_varlen_paged_sdpa(C.byref(_paged(L)), None) == -1
    assert L.lib.hw_paged_sdpa_stages(C.byref(_paged(L)), None, 0) == -3


def test_paged_plan_invariants():
    L = _lib()
    # plain decode at the headline model shape: one 16-row block per worker and kv head, the CUs filled once
    pl = L.paged_plan(W=4, Hq=40, Hkv=8, Ev=128, block_size=16, max_blocks=1024, num_cus=256, S=1)
    assert (pl.rows, pl.row_blocks, pl.row_groups) == (20, 1, 4)
    assert pl.workgroups == 8 * 4 * pl.splits and pl.workgroups <= 256 and pl.splits >= 1
    assert pl.workspace_bytes >= 8 * pl.splits * 20 * 130 * 4
    # short sequences: never more waves than tiles at the longest sequence the table allows
    pl = L.paged_plan(W=1, Hq=8, Hkv=8, Ev=128, block_size=16, max_blocks=8, num_cus=256, S=1)
    assert pl.splits == 1
    # more than 16 rows per worker: workgroups of up to 128 rows (16-bit types, at most 8192 table entries per sequence), the CUs filled once
    pl = L.paged_plan(W=2, Hq=40, Hkv=8, Ev=128, block_size=16, max_blocks=64, num_cus=256, S=12)
    assert pl.row_blocks == 8 and pl.row_groups == 2 * 1 and pl.device_planned == 0
    pl = L.paged_plan(W=2, Hq=40, Hkv=8, Ev=128, block_size=16, max_blocks=64, num_cus=256, S=20)
    assert pl.row_blocks == 8 and pl.row_groups == 2 * 1 and pl.splits == 8 and pl.workgroups == 128   # 32 tiles: four per workgroup at least
    pl = L.paged_plan(W=2, Hq=40, Hkv=8, Ev=128, block_size=1, max_blocks=9000, num_cus=256, S=20)   # table too long for LDS
    assert pl.row_blocks == 2 and pl.row_groups == 2 * 4
    pl = L.paged_plan(W=2, Hq=40, Hkv=8, Ev=128, block_size=16, max_blocks=64, num_cus=256, S=20, row_blocks=2)
    assert pl.row_blocks == 2 and pl.row_groups == 2 * 4
    # fp32 exists with one row block only
    pl = L.paged_plan(W=2, Hq=40, Hkv=8, Ev=128, block_size=16, max_blocks=64, num_cus=256, S=20, dtype=L.HW_F32)
    assert pl.row_blocks == 1 and pl.row_groups == 2 * 7
    # variable length: the row-group count is an upper bound over every way of cutting total_q into W sequences
    pl = L.paged_plan(W=8, Hq=40, Hkv=8, Ev=128, block_size=16, max_blocks=1024, num_cus=256, total_q=700, row_blocks=2)
    assert pl.rows == 3500 and pl.row_groups >= 8 + 3500 // 32 and pl.workgroups == 8 * pl.row_groups * pl.splits
    assert pl.device_planned == 0
    # ... and in 128-row workgroups the device deals the workgroups: a slot per possible row group at least, the CUs
    # filled once (more slots when the row groups alone oversubscribe the CUs), partial sums by slot
    pl = L.paged_plan(W=8, Hq=40, Hkv=8, Ev=128, block_size=16, max_blocks=1024, num_cus=256, total_q=700)
    groups = 8 + 3500 // 128
    assert pl.row_blocks == 8 and pl.device_planned == 1 and pl.splits == 1
    assert pl.row_groups == groups + 32 and pl.workgroups == 8 * pl.row_groups
    assert pl.workspace_bytes >= 8 * pl.row_groups * 128 * 130 * 4 + 8 * 3500 * 8
    pl = L.paged_plan(W=4, Hq=40, Hkv=8, Ev=128, block_size=16, max_blocks=783, num_cus=256, total_q=105)
    assert pl.row_blocks == 8 and pl.device_planned == 1 and pl.row_groups == 32 and pl.workgroups == 256
    # short tables: not more slots than there can be work for (four tiles per slot)
    pl = L.paged_plan(W=4, Hq=40, Hkv=8, Ev=128, block_size=16, max_blocks=8, num_cus=256, total_q=105)
    assert pl.device_planned == 1 and pl.row_groups == 8
    # a caller that fixes the split, too many sequences for the device-side planner, or few rows per sequence: as before
    pl = L.paged_plan(W=4, Hq=40, Hkv=8, Ev=128, block_size=16, max_blocks=783, num_cus=256, total_q=105, splits=4)
    assert pl.row_blocks == 8 and pl.device_planned == 0 and pl.row_groups == 8 and pl.splits == 4 and pl.workgroups == 256
    pl = L.paged_plan(W=300, Hq=40, Hkv=8, Ev=128, block_size=16, max_blocks=783, num_cus=256, total_q=3000)
    assert pl.row_blocks == 8 and pl.device_planned == 0
    pl = L.paged_plan(W=4, Hq=40, Hkv=8, Ev=128, block_size=16, max_blocks=783, num_cus=256, total_q=8)
    assert pl.row_blocks == 1 and pl.device_planned == 0
    # more (kv head, row group) pairs than half the CUs: about three workgroups per CU on long sequences, no
    # splitting at all on short ones or when the pairs alone oversubscribe the chip that far
    pl = L.paged_plan(W=4, Hq=40, Hkv=8, Ev=128, block_size=16, max_blocks=783, num_cus=256, total_q=105, row_blocks=2)
    assert pl.row_groups == 20 and pl.splits == 5 and 3 * 256 <= pl.workgroups < 4 * 256
    assert L.paged_plan(W=4, Hq=40, Hkv=8, Ev=128, block_size=16, max_blocks=30, num_cus=256, total_q=105, row_blocks=2).splits == 1
    assert L.paged_plan(W=64, Hq=40, Hkv=8, Ev=128, block_size=16, max_blocks=783, num_cus=256, total_q=640, row_blocks=2).splits == 1
    # explicit split factor is honoured (capped at 64)
    assert L.paged_plan(W=4, Hq=40, Hkv=8, Ev=128, block_size=16, max_blocks=1024, num_cus=256, S=1, splits=5).splits == 5
    assert L.paged_plan(W=4, Hq=40, Hkv=8, Ev=128, block_size=16, max_blocks=1024, num_cus=256, S=1, splits=500).splits == 64


def test_copy_to_blocks_validation():
    L = _lib()
    c = L.HwCopyBlocks()
    c.dtype, c.B, c.Hkv, c.S_new, c.E, c.Ev = L.HW_BF16, 2, 2, 1, 128, 128
    c.block_size, c.max_blocks, c.num_blocks = 16, 4, 10
    assert L.lib.hw_copy_to_blocks(None, None) == -1
    assert L.lib.hw_copy_to_blocks(C.byref(c), None) == -1           # pointers missing
    c.dtype = 9
    assert L.lib.hw_copy_to_blocks(C.byref(c), None) == -2
    c.dtype, c.block_size = L.HW_BF16, 0
    assert L.lib.hw_copy_to_blocks(C.byref(c), None) == -3
    c.block_size, c.S_new = 16, 0
    assert L.lib.hw_copy_to_blocks(C.byref(c), None) == 0            # nothing to append: success without a device


# ------------------------------------------------------------------------------------------------ caller-side steps
def test_append_struct_layout_matches_header():
    import shutil
    import subprocess
    import tempfile
    L = _lib()
    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    with tempfile.TemporaryDirectory() as d:
        src = os.path.join(d, "s.c")
        open(src, "w").write('#include <stdio.h>\n#include <stddef.h>\n#include "hogwild_hip.h"\nint main(){printf("%zu %zu %zu %zu %zu\\n",'
                             'sizeof(hw_append),offsetof(hw_append,key_states),offsetof(hw_append,cs_s),offsetof(hw_append,n_new),'
                             'offsetof(hw_problem,cap));return 0;}\n')
        exe = os.path.join(d, "s")
        subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), src, "-o", exe], check=True)
        out = [int(x) for x in subprocess.run([exe], check=True, capture_output=True, text=True).stdout.split()]
    assert out == [C.sizeof(L.HwAppend), L.HwAppend.key_states.offset, L.HwAppend.cs_s.offset, L.HwAppend.n_new.offset,
                   L.HwProblem.cap.offset]


def test_build_inputs_and_append_validate_on_the_host():
    L = _lib()
    pe = (C.c_int32 * 4)(5, 6, 7, 8)
    fake = 0x1000
    bi = lambda **k: L.lib.hw_build_inputs(k.get("loc", fake), k.get("cos", fake), k.get("sin", fake), k.get("pe", pe), k.get("inv", fake),
                                           1.0, k.get("rd", L.HW_F32), k.get("F", 2), k.get("W", 2), k.get("S", 1), k.get("R", 64), None)
    assert bi(F=0) == -3 and bi(S=0) == -3 and bi(R=63) == -3 and bi(R=-2) == -3
    assert bi(rd=9) == -2
    assert bi(loc=None) == -1 and bi(pe=None) == -1 and bi(inv=None) == -1 and bi(cos=None) == -1
    assert bi(W=769) == -4                                  # more workers than one launch can carry

    def app(**k):
        a = L.HwAppend()
        a.dtype, a.cs_dtype, a.mode = k.get("dtype", L.HW_BF16), k.get("cs_dtype", L.HW_BF16), k.get("mode", 0)
        a.W, a.Hkv, a.S, a.E, a.Ev, a.RotE = 1, 2, k.get("S", 4), 128, 128, k.get("RotE", 128)
        a.key_states = a.value_states = a.cosines = a.sines = fake
        kp = (C.c_void_p * 1)(k.get("dst", fake))
        ln, cp, nn = (C.c_int32 * 1)(k.get("len", 3)), (C.c_int32 * 1)(k.get("cap", 16)), (C.c_int32 * 1)(k.get("n_new", 4))
        a.k_dst = a.v_dst = C.cast(kp, C.POINTER(C.c_void_p))
        a.dst_len, a.dst_cap, a.n_new = C.cast(ln, C.POINTER(C.c_int32)), C.cast(cp, C.POINTER(C.c_int32)), C.cast(nn, C.POINTER(C.c_int32))
        a._keep = (kp, ln, cp, nn)
        return L.lib.hw_rope_append(C.byref(a), None)
    assert L.lib.hw_rope_append(None, None) == -1
    assert app(dtype=5) == -2 and app(cs_dtype=L.HW_F16) == -2          # tables: float32 or the dtype of the keys
    assert app(mode=2) == -3 and app(RotE=130) == -3 and app(RotE=7) == -3
    assert app(n_new=5) == -3 and app(n_new=-1) == -3
    assert app(len=13, n_new=4) == -3                                   # 13 + 4 rows do not fit a capacity of 16
    assert app(dst=None) == -1
    assert app(n_new=0) == 0                                            # nothing to append: success without a device


def test_head_dim_256_plans_with_one_row_block():
    """Head dimension 256 exists with one 16-row block per workgroup only: more rows become row groups of 16, one workgroup
    per CU, and a request for two blocks or for the 128-row kernel is not honoured."""
    L = _lib()
    lens = [4096] + [2048] * 4
    for rb in (0, 2, 8):
        pl = L.plan(lens, W=4, S=1, Hq=40, Hkv=8, Ev=256, num_cus=256, row_blocks=rb)
        assert pl.row_blocks == 1 and pl.row_groups == 2 and pl.workgroups <= 256
        assert pl.workgroups == 8 * 2 * pl.wgs_per_head
    pl = L.plan(lens, W=8, S=4, Hq=64, Hkv=8, Ev=256, num_cus=256)         # 256 rows per kv head
    assert pl.row_blocks == 1 and pl.row_groups == 16
    for rb in (0, 2, 8):
        pp = L.paged_plan(W=2, Hq=40, Hkv=8, Ev=256, block_size=16, max_blocks=64, num_cus=256, S=12, row_blocks=rb)
        assert pp.row_blocks == 1 and pp.row_groups == 2 * ((12 * 5 + 15) // 16)
    pp = L.paged_plan(W=3, Hq=40, Hkv=8, Ev=256, block_size=16, max_blocks=64, num_cus=256, total_q=100)
    assert pp.row_blocks == 1 and pp.device_planned == 0
