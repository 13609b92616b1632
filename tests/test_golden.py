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
    # bounds relative to the recorded values: an output that is all zeros (or off by a few percent) fails every one
    want = np.array(s["sample_out"])
    t_out = tol.out_bound(np.array([s["out_abs_max"]]))
    assert np.abs(o[s["sample_index"]] - want).max() <= t_out
    assert np.abs(np64(lse).reshape(-1)[:8] - np.array(s["sample_lse"])).max() <= tol.lse_bound()
    assert abs(float(np64(lse).mean()) - s["lse_mean"]) <= tol.lse_bound()
    assert abs(float(np.sqrt((o ** 2).sum())) - s["out_l2"]) <= 2.0 ** -7 * s["out_l2"]
    assert abs(float(np.abs(o).max()) - s["out_abs_max"]) <= t_out


# ------------------------------------------------------------------------------------------------ paged / cache fixtures
def _npz(name):
    z = np.load(os.path.join(GOLD, name))
    return {k: z[k] for k in z.files}


def test_paged_oracle_reproduces_fixture():
    from oracle import paged_oracle as po
    g = _npz("paged_small.npz")
    kc, vc = g["key_cache"].astype(np.float64), g["value_cache"].astype(np.float64)
    po.copy_to_blocks(g["k_new"].astype(np.float64), g["v_new"].astype(np.float64), kc, vc, g["block_table"], g["seq_lengths"])
    assert np.array_equal(kc.astype(np.float32), g["key_cache_after"]) and np.array_equal(vc.astype(np.float32), g["value_cache_after"])
    out, lse = po.paged_sdpa(g["q"].astype(np.float64), g["locations"], g["fragment_lengths"], kc, vc, g["block_table"], float(g["scale"]))
    assert np.abs(out - g["out"]).max() < 1e-12 and np.array_equal(np.isneginf(lse), np.isneginf(g["lse"]))
    fin = np.isfinite(g["lse"])
    assert np.abs(lse[fin] - g["lse"][fin]).max() < 1e-12
    outv, lsev = po.varlen_paged_sdpa(g["q_varlen"].astype(np.float64), g["locations_varlen"], g["fragment_lengths_varlen"], kc, vc,
                                      g["block_table"], g["cu_seqlens_q"], float(g["scale"]))
    assert np.abs(outv - g["out_varlen"]).max() < 1e-12


def test_cache_oracle_reproduces_fixture():
    from oracle import cache_oracle as co
    g = _npz("cache_small.npz")
    loc, c32, s32 = co.build_inputs(g["pos_end"].astype(np.int64), 2, g["inv_freq"], table_dtype="f32")
    assert np.array_equal(loc, g["locations"]) and np.array_equal(c32, g["cos_f32"]) and np.array_equal(s32, g["sin_f32"])
    _, c16, s16 = co.build_inputs(g["pos_end"].astype(np.int64), 2, g["inv_freq"], table_dtype="bf16")
    assert np.array_equal(c16, g["cos_bf16"]) and np.array_equal(s16, g["sin_bf16"])
    for w in range(3):
        r = co.rope_keys(g["keys"][w].astype(np.float64), g["key_cos"][w][None].astype(np.float64), g["key_sin"][w][None].astype(np.float64),
                         storage="bf16", cs_storage="bf16", mode="eager")
        assert np.array_equal(r.astype(np.float32), g["keys_rotated"][w])
    m = co.merge_rerotate(g["keys_rotated"][0].astype(np.float64), 123, g["inv_freq"], storage="bf16", mode="eager")
    assert np.array_equal(m.astype(np.float32), g["merged_at_123"])


@pytest.mark.gpu
def test_hip_paged_path_reproduces_fixture():
    from inference_lib_amd import _lib
    g = _npz("paged_small.npz")
    dev = torch.device("cuda:0")
    t = lambda a: torch.from_numpy(a).to(dev)
    kc, vc = t(g["key_cache"]), t(g["value_cache"])
    _lib.copy_to_blocks(t(g["k_new"]), t(g["v_new"]), kc, vc, t(g["block_table"]), t(g["seq_lengths"]))
    torch.cuda.synchronize()
    assert np.array_equal(kc.cpu().numpy(), g["key_cache_after"]) and np.array_equal(vc.cpu().numpy(), g["value_cache_after"])
    out = torch.empty(g["out"].shape, dtype=torch.float32, device=dev)
    lse = torch.empty(g["lse"].shape, dtype=torch.float32, device=dev)
    _lib.PagedProblem(q=t(g["q"]), locations=t(g["locations"]), fragment_lengths=t(g["fragment_lengths"]), key_cache=kc, value_cache=vc,
                      block_table=t(g["block_table"]), scale=float(g["scale"]), out=out, lse=lse).run()
    outv = torch.empty(g["out_varlen"].shape, dtype=torch.float32, device=dev)
    lsev = torch.empty(g["lse_varlen"].shape, dtype=torch.float32, device=dev)
    _lib.PagedProblem(q=t(g["q_varlen"]), locations=t(g["locations_varlen"]), fragment_lengths=t(g["fragment_lengths_varlen"]), key_cache=kc,
                      value_cache=vc, block_table=t(g["block_table"]), scale=float(g["scale"]), out=outv, lse=lsev,
                      cu_seqlens_q=t(g["cu_seqlens_q"])).run()
    torch.cuda.synchronize()
    assert_close("out", out, g["out"], TOL["f32"])
    assert_close("lse", lse, g["lse"], TOL["f32"])
    assert_close("out varlen", outv, g["out_varlen"], TOL["f32"])
    assert_close("lse varlen", lsev, g["lse_varlen"], TOL["f32"])


@pytest.mark.gpu
def test_hip_cache_steps_reproduce_fixture():
    from inference_lib_amd import _lib
    g = _npz("cache_small.npz")
    dev = torch.device("cuda:0")
    loc, cos, sin = _lib.build_inputs(g["pos_end"].tolist(), 2, torch.from_numpy(g["inv_freq"]).to(dev))
    _, cos16, _ = _lib.build_inputs(g["pos_end"].tolist(), 2, torch.from_numpy(g["inv_freq"]).to(dev), table_dtype=torch.bfloat16)
    torch.cuda.synchronize()
    assert np.array_equal(loc.cpu().numpy(), g["locations"])
    assert np.abs(cos.cpu().numpy() - g["cos_f32"]).max() <= 5e-7 and np.abs(sin.cpu().numpy() - g["sin_f32"]).max() <= 5e-7
    assert np.mean(cos16.cpu().numpy() == g["cos_bf16"]) > 0.995
    keys = torch.from_numpy(g["keys"]).to(torch.bfloat16).to(dev)
    kd = [torch.zeros((2, 4, 64), dtype=torch.bfloat16, device=dev) for _ in range(3)]
    vd = [torch.zeros((2, 4, 64), dtype=torch.bfloat16, device=dev) for _ in range(3)]
    _lib.rope_append(keys, keys, kd, vd, [0, 0, 0], cosines=torch.from_numpy(g["key_cos"]).to(torch.bfloat16).to(dev),
                     sines=torch.from_numpy(g["key_sin"]).to(torch.bfloat16).to(dev))
    torch.cuda.synchronize()
    for w in range(3):
        assert np.array_equal(kd[w].float().cpu().numpy(), g["keys_rotated"][w])       # bit-exact
        assert torch.equal(vd[w], keys[w])
