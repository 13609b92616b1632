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


@pytest.mark.parametrize("idx", [1, 2, 3, 4, 5])
def test_baseline_configs(oracle, idx):
    from inference_lib_amd import cases
    c = cases.baseline_case(idx)
    print(f"baseline case {idx}: {c.name} lens={c.lens}", flush=True)
    out, lse, rq = run_fused(c.to(_dev()))
    o_ref, l_ref, rq_ref = oracle_fused(oracle, c)
    e1 = assert_close("out", out, o_ref, TOL[c.dtype])
    e2 = assert_close("lse", lse, l_ref, TOL[c.dtype])
    print(f"  max err out {e1:.3e} lse {e2:.3e}", flush=True)
