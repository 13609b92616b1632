"""Writes the golden fixtures of the parity tests.

  c1_fp32.npz ......... workload configuration 1 complete: q, locations, cos, sin, every K/V fragment and the
                        expected out[2,8,64] / lse[2,8] (the fp64 oracle on the fp32 inputs, stored as fp64)
  configs_summary.json  for configurations 2..5: SHA-256 of the regenerated inputs, and of the expected outputs
                        a few statistics plus sampled values (the inputs regenerate from their seeds)

  paged_small.npz ..... a small paged problem (fp32 inputs): caches before and after a copy_to_blocks of 3 new tokens,
                        block table, queries, locations, fragment lengths and the expected out / lse of the
                        fixed-length and of a packed variable-length call
  cache_small.npz ..... inputs and expected results of the caller-side steps: pos_end -> locations and rotary tables
                        (fp32 and bf16-rounded), bf16 keys rotated in eager mode, a merge re-rotation

The expected values come from oracle/hogwild_oracle.py, oracle/paged_oracle.py and oracle/cache_oracle.py, whose
functions are pinned independently in tests/test_oracle_pins.py, tests/test_paged_oracle_pins.py and
tests/test_cache_oracle_pins.py; the reference itself ships no vectors for this path.  Run from the repo root:
    python tests/golden/make_golden.py
"""
import hashlib
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

from helpers import np64, oracle_fused  # noqa: E402
from inference_lib_amd import cases  # noqa: E402
from oracle import hogwild_oracle as oracle  # noqa: E402


def input_digest(c) -> str:
    h = hashlib.sha256()
    for t in [c.q, c.locations, c.cos, c.sin] + list(c.keys) + list(c.values):
        a = t.contiguous()
        h.update(a.view(dtype=__import__("torch").uint8).numpy().tobytes() if a.dtype != __import__("torch").int32 else a.numpy().tobytes())
    return h.hexdigest()


def main():
    c = cases.baseline_case(1)
    out, lse, rq = oracle_fused(oracle, c)
    arrays = {"q": c.q.numpy(), "locations": c.locations.numpy(), "cos": c.cos.numpy(), "sin": c.sin.numpy(),
              "out": out, "lse": lse, "scale": np.float64(c.scale)}
    for f in range(c.F):
        arrays[f"k{f}"] = c.keys[f].numpy()
        arrays[f"v{f}"] = c.values[f].numpy()
    np.savez(os.path.join(HERE, "c1_fp32.npz"), **arrays)

    summary = {}
    sample = np.random.default_rng(0)
    for idx in (2, 3, 4, 5):
        c = cases.baseline_case(idx)
        out, lse, _ = oracle_fused(oracle, c)
        flat = out.reshape(-1)
        pick = sample.choice(flat.size, size=16, replace=False)
        summary[str(idx)] = {
            "name": c.name, "lens": c.lens, "inputs_sha256": input_digest(c),
            "out_mean": float(out.mean()), "out_abs_max": float(np.abs(out).max()), "out_l2": float(np.sqrt((out ** 2).sum())),
            "lse_mean": float(lse.mean()), "lse_min": float(lse.min()), "lse_max": float(lse.max()),
            "sample_index": pick.tolist(), "sample_out": flat[pick].tolist(),
            "sample_lse": lse.reshape(-1)[:8].tolist(),
        }
        print(idx, c.name, summary[str(idx)]["inputs_sha256"][:16], flush=True)
    with open(os.path.join(HERE, "configs_summary.json"), "w") as fh:
        json.dump(summary, fh, indent=1)


def paged_and_cache():
    from oracle import cache_oracle as co
    from oracle import paged_oracle as po
    rng = np.random.default_rng(20240607)
    F, W, Hq, Hkv, S, D, bs, mb = 2, 3, 8, 2, 2, 64, 8, 4
    NB = W * mb + 2
    kc = rng.standard_normal((NB, Hkv, bs, D)).astype(np.float32)
    vc = rng.standard_normal((NB, Hkv, bs, D)).astype(np.float32)
    bt = rng.permutation(NB)[: W * mb].reshape(W, mb).astype(np.int32)
    seq = np.array([20, 7, 28], dtype=np.int32)
    k_new = rng.standard_normal((W, Hkv, 3, D)).astype(np.float32)
    v_new = rng.standard_normal((W, Hkv, 3, D)).astype(np.float32)
    kc2, vc2 = kc.astype(np.float64), vc.astype(np.float64)
    po.copy_to_blocks(k_new.astype(np.float64), v_new.astype(np.float64), kc2, vc2, bt, seq)
    q = rng.standard_normal((F, W, Hq, S, D)).astype(np.float32)
    loc = np.stack([seq[:, None] + 3 - S + np.arange(S)[None, :], seq[:, None] - 4 + np.arange(S)[None, :]]).astype(np.int32)
    fl = np.array([32, 9], dtype=np.int32)
    out, lse = po.paged_sdpa(q.astype(np.float64), loc, fl, kc2, vc2, bt, 0.125)
    cu = np.array([0, 2, 2, 5], dtype=np.int32)
    qv = rng.standard_normal((F, 5, Hq, D)).astype(np.float32)
    locv = rng.integers(-1, 31, size=(F, 5)).astype(np.int32)
    flv = np.minimum(np.array([[23, 10, 31], [5, 10, 20]]), (seq + 3)[None, :]).astype(np.int32)
    outv, lsev = po.varlen_paged_sdpa(qv.astype(np.float64), locv, flv, kc2, vc2, bt, cu, 0.125)
    np.savez(os.path.join(HERE, "paged_small.npz"), key_cache=kc, value_cache=vc, block_table=bt, seq_lengths=seq, k_new=k_new,
             v_new=v_new, key_cache_after=kc2.astype(np.float32), value_cache_after=vc2.astype(np.float32), q=q, locations=loc,
             fragment_lengths=fl, out=out, lse=lse, cu_seqlens_q=cu, q_varlen=qv, locations_varlen=locv, fragment_lengths_varlen=flv,
             out_varlen=outv, lse_varlen=lsev, scale=np.float64(0.125))

    inv_freq = (10000.0 ** (-np.arange(0, D, 2, dtype=np.float64) / D)).astype(np.float32)
    lens = [500, 40, 17, 3]
    orders = [[0, 2, 3, 1], [0, 1, 3, 2], [3, 0, 1, 2]]
    pe = co.pos_end_from_orders(orders, lens)
    loc_b, cos32, sin32 = co.build_inputs(pe, 2, inv_freq, attention_scaling=1.0, table_dtype="f32")
    _, cos16, sin16 = co.build_inputs(pe, 2, inv_freq, attention_scaling=1.0, table_dtype="bf16")
    from oracle.hogwild_oracle import round_to
    keys = round_to(rng.standard_normal((3, Hkv, 4, D)), "bf16").astype(np.float32)
    kpos = np.array([[10, 11, 12, 13], [0, 1, 2, 3], [70000, 70001, 70002, 70003]])
    kcos, ksin = co.rotary_tables(kpos, inv_freq, 1.0, "bf16")
    rotated = np.stack([co.rope_keys(keys[w].astype(np.float64), kcos[w][None].astype(np.float64), ksin[w][None].astype(np.float64),
                                     storage="bf16", cs_storage="bf16", mode="eager") for w in range(3)]).astype(np.float32)
    merged = co.merge_rerotate(rotated[0].astype(np.float64), 123, inv_freq, storage="bf16", mode="eager").astype(np.float32)
    np.savez(os.path.join(HERE, "cache_small.npz"), inv_freq=inv_freq, pos_end=pe.astype(np.int32), locations=loc_b, cos_f32=cos32,
             sin_f32=sin32, cos_bf16=cos16, sin_bf16=sin16, keys=keys, key_positions=kpos.astype(np.int32), key_cos=kcos, key_sin=ksin,
             keys_rotated=rotated, merged_at_123=merged)


if __name__ == "__main__":
    main()
    paged_and_cache()
