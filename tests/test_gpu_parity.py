"""GPU parity of the HIP path (through the C ABI) against the CPU oracle.  Tolerances: fp32 1e-4,
bf16/fp16 2e-2 max-abs on both the output and the LSE, against the oracle evaluated in fp64 on the
same already-quantised inputs."""
import numpy as np
import pytest
import torch

from helpers import TOL, assert_close, np64, oracle_fused, run_fused

pytestmark = pytest.mark.gpu


def _dev():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return torch.device("cuda:0")


@pytest.mark.parametrize("dtype", ["bf16", "f16", "f32"])
@pytest.mark.parametrize("E", [128, 64])
def test_small_fused(oracle, dtype, E):
    from inference_lib_amd import cases
    c = cases.small_case(dtype=dtype, W=2, S=1, Hq=8, Hkv=2, E=E, lens=(100, 37, 65), seed=11)
    print(f"case {c.name} E={E}", flush=True)
    out, lse, rq = run_fused(c.to(_dev()))
    o_ref, l_ref, rq_ref = oracle_fused(oracle, c)
    assert_close("rq", rq, rq_ref, 1e-5 if dtype == "f32" else 8e-3 * 4)
    assert_close("out", out, o_ref, TOL[dtype])
    assert_close("lse", lse, l_ref, TOL[dtype])


@pytest.mark.parametrize("idx", [1, 2, 3, 4, 5, 6])
def test_baseline_configs(oracle, idx):
    from inference_lib_amd import cases
    c = cases.baseline_case(idx)
    print(f"baseline case {idx}: {c.name} lens={c.lens}", flush=True)
    out, lse, rq = run_fused(c.to(_dev()))
    o_ref, l_ref, rq_ref = oracle_fused(oracle, c)
    e1 = assert_close("out", out, o_ref, TOL[c.dtype])
    e2 = assert_close("lse", lse, l_ref, TOL[c.dtype])
    print(f"  max err out {e1:.3e} lse {e2:.3e}", flush=True)


@pytest.mark.parametrize("dtype,W,S", [("f16", 1, 1), ("f16", 4, 1), ("bf16", 2, 3), ("f16", 8, 1), ("f32", 2, 1)])
def test_the_reference_kernels_compiled_shape(oracle, dtype, W, S):
    """E = Ev = 128 with 16 query heads per kv head is the one shape the reference's kernel is instantiated for
    (src/kernels/kernel_v21.cuh:982); here through the fused entry with 16, 64, 96 and 128 rows per kv head (one and two
    row blocks, several row groups, the 128-row kernel) and in fp32."""
    from inference_lib_amd import cases
    lens = tuple([300] + [70 + 9 * w for w in range(W)])
    c = cases.small_case(dtype=dtype, W=W, S=S, Hq=32, Hkv=2, E=128, lens=lens, seed=51)
    print(f"case {c.name} W={W} S={S} rows per kv head {W * S * 16}", flush=True)
    out, lse, rq = run_fused(c.to(_dev()))
    o_ref, l_ref, rq_ref = oracle_fused(oracle, c)
    assert_close("rq", rq, rq_ref, 1e-5 if dtype == "f32" else 3.2e-2)
    assert_close("out", out, o_ref, TOL[dtype])
    assert_close("lse", lse, l_ref, TOL[dtype])


@pytest.mark.parametrize("dtype,E", [("bf16", 128), ("f16", 64), ("f32", 64), ("f32", 128)])
def test_rope_and_sdpa_entries(oracle, dtype, E):
    """hw_rope and hw_sdpa (pre-rotated queries), the two halves the reference also exports separately
    (python/hogwild/attention.py:26-35, 70-74)."""
    from inference_lib_amd import _lib, cases
    c = cases.small_case(dtype=dtype, W=3, S=2, Hq=6, Hkv=2, E=E, lens=(70, 33, 1, 64), seed=5)
    cd = c.to(_dev())
    print(f"case {c.name} E={E}", flush=True)
    W, Hq, S, _ = cd.q.shape
    rq = torch.full((c.F, W, Hq, S, E), float("nan"), dtype=cd.q.dtype, device=_dev())
    _lib.rope(cd.q, cd.cos, cd.sin, rq)
    torch.cuda.synchronize()
    o_ref, l_ref, rq_ref = oracle_fused(oracle, c)
    assert_close("rope", rq, rq_ref, 1e-5 if dtype == "f32" else 3.2e-2)
    out = torch.full((W, Hq, S, E), float("nan"), dtype=cd.q.dtype, device=_dev())
    lse = torch.full((W, Hq, S), float("nan"), dtype=torch.float32, device=_dev())
    pr = _lib.Problem(q=rq, locations=cd.locations, keys=cd.keys, values=cd.values, scale=c.scale, out=out, lse=lse,
                      prerotated=True)
    pr.run()
    torch.cuda.synchronize()
    # the oracle attends with the GPU's own rotated queries so this checks the attention half alone
    o2, l2 = oracle.sdpa_fragments(np64(rq), c.locations.numpy(), [np64(k) for k in c.keys], [np64(v) for v in c.values], c.scale)
    assert_close("sdpa out", out, o2, TOL[dtype])
    assert_close("sdpa lse", lse, l2, TOL[dtype])


@pytest.mark.parametrize("dtype,E,rot", [("bf16", 128, 64), ("f16", 64, 32), ("f32", 64, 20), ("bf16", 128, 0)])
def test_partial_rotary(oracle, dtype, E, rot):
    """Rotary width smaller than the head dim (pass-through tail, src/rope.cuh:48-51), including widths that
    are not a multiple of the 16-byte vector width and no rotation at all."""
    from inference_lib_amd import cases
    c = cases.small_case(dtype=dtype, W=2, S=2, Hq=4, Hkv=2, E=E, lens=(90, 40, 47), seed=21, rot_dim=max(rot, 2))
    if rot == 0:   # zero-width tables: nothing is rotated
        c.cos = c.cos[..., :0].contiguous()
        c.sin = c.sin[..., :0].contiguous()
    print(f"case {c.name} E={E} rot={rot}", flush=True)
    out, lse, rq = run_fused(c.to(_dev()))
    o_ref, l_ref, rq_ref = oracle_fused(oracle, c)
    assert_close("rq", rq, rq_ref, 1e-5 if dtype == "f32" else 3.2e-2)
    assert_close("out", out, o_ref, TOL[dtype])
    assert_close("lse", lse, l_ref, TOL[dtype])
    out2, lse2, _ = run_fused(c.to(_dev()), with_rq=False)     # rotated queries go to the workspace instead
    assert torch.equal(out, out2) and torch.equal(lse, lse2)


@pytest.mark.parametrize("idx", [1, 2])
def test_valu_logits_variant_on_the_small_row_configs(oracle, idx):
    """HW_VARIANT_VALU_QK (logits by v_dot2 / v_fma instead of MFMA; at most 16 rows per kv head) against the oracle on the
    two workload configurations it is measured on, and refused where it does not exist."""
    from inference_lib_amd import _lib, cases
    c = cases.baseline_case(idx)
    cd = c.to(_dev())
    W, Hq, S, E = cd.q.shape
    out = torch.full((W, Hq, S, E), float("nan"), dtype=cd.q.dtype, device=_dev())
    lse = torch.full((W, Hq, S), float("nan"), dtype=torch.float32, device=_dev())
    pr = _lib.Problem(q=cd.q, locations=cd.locations, keys=cd.keys, values=cd.values, scale=cd.scale, out=out, cosines=cd.cos,
                      sines=cd.sin, lse=lse, variant=_lib.HW_VARIANT_VALU_QK)
    pr.run()
    torch.cuda.synchronize()
    o_ref, l_ref, _ = oracle_fused(oracle, c)
    assert_close("out", out, o_ref, TOL[c.dtype])
    assert_close("lse", lse, l_ref, TOL[c.dtype])


@pytest.mark.parametrize("dtype,E", [("bf16", 128), ("f16", 64), ("f32", 64), ("f32", 128), ("bf16", 64), ("f16", 128)])
def test_valu_logits_variant_small(oracle, dtype, E):
    from inference_lib_amd import _lib, cases
    c = cases.small_case(dtype=dtype, W=2, S=1, Hq=8, Hkv=2, E=E, lens=(100, 37, 65), seed=13)
    cd = c.to(_dev())
    W, Hq, S, _ = cd.q.shape
    out = torch.full((W, Hq, S, E), float("nan"), dtype=cd.q.dtype, device=_dev())
    lse = torch.full((W, Hq, S), float("nan"), dtype=torch.float32, device=_dev())
    pr = _lib.Problem(q=cd.q, locations=cd.locations, keys=cd.keys, values=cd.values, scale=cd.scale, out=out, cosines=cd.cos,
                      sines=cd.sin, lse=lse, variant=_lib.HW_VARIANT_VALU_QK)
    pr.run()
    torch.cuda.synchronize()
    o_ref, l_ref, _ = oracle_fused(oracle, c)
    assert_close("out", out, o_ref, TOL[dtype])
    assert_close("lse", lse, l_ref, TOL[dtype])
    # more than 16 rows per kv head: no such kernel
    c3 = cases.small_case(dtype=dtype, W=5, S=1, Hq=8, Hkv=2, E=E, lens=(40, 8, 8, 8, 8, 8), seed=1).to(_dev())
    out3 = torch.empty_like(c3.q)
    pr3 = _lib.Problem(q=c3.q, locations=c3.locations, keys=c3.keys, values=c3.values, scale=c3.scale, out=out3, cosines=c3.cos,
                       sines=c3.sin, variant=_lib.HW_VARIANT_VALU_QK)
    with pytest.raises(_lib.HogwildError) as ei:
        pr3.run()
    assert ei.value.status == -4
