"""Golden fixtures (tests/golden/, written by tests/golden/make_golden.py): the oracle and the input generator
reproduce them on the CPU; the HIP path reproduces them on the GPU."""
import hashlib
import json
import os

import numpy as np
import pytest
import torch

from helpers import TOL, assert_close, np64, oracle_fused, run_fused

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _c1():
    z = np.load(os.path.join(GOLD, "c1_fp32.npz"))
    return {k: z[k] for k in z.files}


def _digest(c):
    h = hashlib.sha256()
    for t in [c.q, c.locations, c.cos, c.sin] + list(c.keys) + list(c.values):
        a = t.contiguous()
        h.update(a.numpy().tobytes() if a.dtype == torch.int32 else a.view(dtype=torch.uint8).numpy().tobytes())
    return h.hexdigest()


def test_generator_reproduces_fixture_inputs():
    from inference_lib_amd import cases
    g = _c1()
    c = cases.baseline_case(1)
    assert np.array_equal(c.q.numpy(), g["q"]) and np.array_equal(c.locations.numpy(), g["locations"])
    assert np.array_equal(c.cos.numpy(), g["cos"]) and np.array_equal(c.sin.numpy(), g["sin"])
    for f in range(c.F):
        assert np.array_equal(c.keys[f].numpy(), g[f"k{f}"]) and np.array_equal(c.values[f].numpy(), g[f"v{f}"])
    # the layout the configuration states: prompt 256 + one 64-token segment per worker, own segment last
    assert c.lens == [256, 64, 64]
    assert c.locations[:, :, 0].tolist() == [[383, 383], [127, 63], [63, 127]]


def test_oracle_reproduces_fixture_outputs(oracle):
    g = _c1()
    F = g["locations"].shape[0]
    out, lse, _ = oracle.fused_reference(g["q"].astype(np.float64), g["locations"], [g[f"k{f}"].astype(np.float64) for f in range(F)],
                                         [g[f"v{f}"].astype(np.float64) for f in range(F)], float(g["scale"]),
                                         g["cos"].astype(np.float64), g["sin"].astype(np.float64), storage="f32")
    assert out.shape == (2, 8, 1, 64) and lse.shape == (2, 8, 1)
    assert np.abs(out - g["out"]).max() < 1e-12 and np.abs(lse - g["lse"]).max() < 1e-12


@pytest.mark.parametrize("idx", [2, 3])
def test_generator_digest_of_larger_configs(idx):
    from inference_lib_amd import cases
    summary = json.load(open(os.path.join(GOLD, "configs_summary.json")))[str(idx)]
    c = cases.baseline_case(idx)
    assert c.lens == summary["lens"]
    assert _digest(c) == summary["inputs_sha256"]


@pytest.mark.gpu
def test_gpu_reproduces_c1_fixture():
    from inference_lib_amd import cases
    g = _c1()
    c = cases.baseline_case(1)
    out, lse, _ = run_fused(c.to(torch.device("cuda:0")))
    assert_close("out", out, g["out"], TOL["f32"])
    assert_close("lse", lse, g["lse"], TOL["f32"])


@pytest.mark.gpu
@pytest.mark.parametrize("idx", [2, 3, 4, 5])
def test_gpu_reproduces_summary_of_larger_configs(idx):
    from inference_lib_amd import cases
    s = json.load(open(os.path.join(GOLD, "configs_summary.json")))[str(idx)]
    c = cases.baseline_case(idx)
    assert _digest(c) == s["inputs_sha256"]
    print(f"golden summary case {idx}: {c.name}", flush=True)
    out, lse, _ = run_fused(c.to(torch.device("cuda:0")))
    o = np64(out).reshape(-1)
    tol = TOL[c.dtype]
    assert np.abs(o[s["sample_index"]] - np.array(s["sample_out"])).max() <= tol
    assert np.abs(np64(lse).reshape(-1)[:8] - np.array(s["sample_lse"])).max() <= tol
    assert abs(float(np64(lse).mean()) - s["lse_mean"]) <= tol
    assert abs(float(np.sqrt((o ** 2).sum())) - s["out_l2"]) <= tol * np.sqrt(o.size)
