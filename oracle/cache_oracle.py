"""CPU oracle for the caller-side steps of the Hogwild! decode step.  TEST INFRASTRUCTURE ONLY.

Nothing in the product package imports this module.  It restates, in numpy:

  * the layer-0 input construction of HogwildCache.update ...... python/hogwild/attention.py:164-196
    (locations :173-181; rotary tables from the model's rotary embedding module, returned in the model dtype and
    widened to float32, :191-193)
  * apply_rotary_pos_emb on new keys ............................. python/hogwild/attention.py:77-90, :313-315
  * the per-worker append with left masking ...................... python/hogwild/attention.py:148-158
  * merge_caches (re-rotation by the target's length + append) .... python/hogwild/attention.py:251-257

The rotary embedding module itself lives in the `transformers` dependency of the reference (Qwen2RotaryEmbedding and
its siblings; the reference pins no version).  Its published algorithm is restated in `rotary_tables`:
freqs = position.float() * inv_freq.float(); emb = cat(freqs, freqs); cos = emb.cos() * attention_scaling, cast to the
dtype of the activations.  Where `transformers` is installed the pins also run against its Qwen2RotaryEmbedding and
apply_rotary_pos_emb directly.

Pinning status (tests/test_cache_oracle_pins.py):
  pos_end_from_orders ... pinned: closed-form sums; consistency with hogwild_oracle.locations_from_order.
  rotary_tables ......... pinned: equals hogwild_oracle.rope_tables (itself pinned) for inv_freq = base^(-2i/D);
                          torch.cos/sin in float32 for the fp32 arithmetic; bf16/fp16 rounding via torch casts;
                          the installed transformers' Qwen2RotaryEmbedding.
  rope_keys ............. pinned: closed-form rotation per element pair; norm preservation; q.k after rotating both
                          sides depends only on the position difference (with the query rotation pinned separately
                          against the reference's rope_cpu); eager rounding order against torch's own tensor
                          arithmetic in bf16 / fp16 / fp32 on the CPU; transformers' apply_rotary_pos_emb bit for bit.
  append_left_masked .... pinned: torch.cat of the unmasked tails.
  merge_rerotate ........ pinned: rotating keys of position p by a further t equals rotating the raw keys by p + t.
The reference ships no tests, fixtures or golden vectors for these steps.
"""
from __future__ import annotations

from typing import List, Sequence, Tuple

import numpy as np

from .hogwild_oracle import round_to


def pos_end_from_orders(orders: List[List[int]], lens: Sequence[int]) -> np.ndarray:
    """pos_end[f, w] = sum of the lengths of fragment f and of every fragment after it in worker w's order
    (python/hogwild/attention.py:174-181; lengths already include the new tokens)."""
    F, W = len(lens), len(orders)
    out = np.zeros((F, W), dtype=np.int64)
    for w in range(W):
        pos = 0
        for f in reversed(orders[w]):
            pos += int(lens[f])
            out[f, w] = pos
    return out


def rotary_tables(positions: np.ndarray, inv_freq: np.ndarray, attention_scaling: float = 1.0, table_dtype: str = "f32"
                  ) -> Tuple[np.ndarray, np.ndarray]:
    """cos/sin [..., RotE] for integer positions [...]: float32 product position * inv_freq, cos/sin of that float32
    angle, times the scaling in float32, rounded to `table_dtype` ("f32" | "f16" | "bf16"), returned as float32."""
    ang = positions.astype(np.float32)[..., None] * inv_freq.astype(np.float32)            # fp32 product
    ang = np.concatenate([ang, ang], axis=-1)
    cos = (np.cos(ang.astype(np.float64)).astype(np.float32) * np.float32(attention_scaling)).astype(np.float32)
    sin = (np.sin(ang.astype(np.float64)).astype(np.float32) * np.float32(attention_scaling)).astype(np.float32)
    return round_to(cos, table_dtype).astype(np.float32), round_to(sin, table_dtype).astype(np.float32)


def build_inputs(pos_end: np.ndarray, S: int, inv_freq: np.ndarray, attention_scaling: float = 1.0, table_dtype: str = "f32"):
    """locations [F, W, S] = pos_end - S + s (python/hogwild/attention.py:180) and their tables [F, W, S, RotE]."""
    loc = (pos_end[..., None] - S + np.arange(S)).astype(np.int32)
    cos, sin = rotary_tables(loc, inv_freq, attention_scaling, table_dtype)
    return loc, cos, sin


def rope_keys(x: np.ndarray, cos: np.ndarray, sin: np.ndarray, *, storage: str = "f32", cs_storage: str = "f32",
              mode: str = "eager") -> np.ndarray:
    """(x * cos) + (rotate_half(x) * sin) on the first RotE = cos.shape[-1] elements (python/hogwild/attention.py:77-90).

    x [..., S, E] holds values of type `storage`, cos/sin [..., S, RotE] (broadcastable against x without its last
    dimension) values of type `cs_storage`.  mode "eager": every product and the sum are rounded to the common type
    of the operands (the 16-bit type if both are 16-bit, else float32), the result to `storage` -- what the tensor
    expression does.  mode "exact": float64 arithmetic, one rounding to `storage`.
    """
    rot = cos.shape[-1]
    h = rot // 2
    xr, xp = x[..., :rot], x[..., rot:]
    rh = np.concatenate([-xr[..., h:], xr[..., :h]], axis=-1)
    if mode == "exact":
        y = xr.astype(np.float64) * cos + rh.astype(np.float64) * sin
    else:
        common = storage if (storage != "f32" and cs_storage == storage) else "f32"
        a = round_to(xr.astype(np.float32) * cos.astype(np.float32), common).astype(np.float32)
        b = round_to(rh.astype(np.float32) * sin.astype(np.float32), common).astype(np.float32)
        y = round_to(a + b, common)
    out = np.concatenate([np.asarray(y, dtype=np.float64), xp.astype(np.float64)], axis=-1)
    return round_to(out, storage).astype(np.float64)


def append_left_masked(dst: np.ndarray, length: int, new: np.ndarray, n_new: int) -> int:
    """dst [Hkv, cap, D] holds `length` rows; append the last n_new of new [Hkv, S, D] (python/hogwild/attention.py:149-155).
    Returns the new length."""
    S = new.shape[1]
    dst[:, length:length + n_new] = new[:, S - n_new:]
    return length + n_new


def merge_rerotate(source_keys: np.ndarray, target_len: int, inv_freq: np.ndarray, attention_scaling: float = 1.0, *,
                   storage: str = "f32", mode: str = "eager") -> np.ndarray:
    """Keys of a source segment [Hkv, L, E] re-rotated for being appended behind target_len tokens: every key gets the
    rotation of position target_len (python/hogwild/attention.py:252-256), tables in the keys' own dtype."""
    pos = np.full((1,), target_len, dtype=np.int64)
    cos, sin = rotary_tables(pos, inv_freq, attention_scaling, storage)
    return rope_keys(source_keys, cos, sin, storage=storage, cs_storage=storage, mode=mode)
