"""Writes the golden fixtures of the parity tests.

  c1_fp32.npz ......... workload configuration 1 complete: q, locations, cos, sin, every K/V fragment and the
                        expected out[2,8,64] / lse[2,8] (the fp64 oracle on the fp32 inputs, stored as fp64)
  configs_summary.json  for configurations 2..5: SHA-256 of the regenerated inputs, and of the expected outputs
                        a few statistics plus sampled values (the inputs regenerate from their seeds)

The expected values come from oracle/hogwild_oracle.py, whose functions are pinned independently in
tests/test_oracle_pins.py; the reference itself ships no vectors for this path.  Run from the repo root:
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


if __name__ == "__main__":
    main()
