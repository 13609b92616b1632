"""Pins for oracle/cache_oracle.py (input builder, key rotation, append, merge re-rotation): facts that do not depend
on the oracle's own formulas -- closed forms, invariants, the separately pinned query-side oracle, and torch's own
tensor arithmetic for the rounding order.  The reference ships no tests or fixtures for these steps."""
import math

import numpy as np
import pytest
import torch

from oracle import cache_oracle as co
from oracle import hogwild_oracle as fo

rng = np.random.default_rng(2024)
TDT = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}


def inv_freq(D, base=10000.0):
    return (base ** (-np.arange(0, D, 2, dtype=np.float64) / D)).astype(np.float32)


# ---------------------------------------------------------------------------------------------- input builder
def test_pos_end_closed_forms_and_locations_consistency():
    lens = [100, 7, 30, 2]                       # prompt, two worker segments, a shared scratch segment
    orders = [[0, 2, 3, 1], [0, 1, 3, 2], [3, 0, 1, 2]]
    pe = co.pos_end_from_orders(orders, lens)
    assert pe[1, 0] == 7 and pe[3, 0] == 9 and pe[2, 0] == 39 and pe[0, 0] == 139          # worker 0: 0,2,3,1
    assert pe[2, 1] == 30 and pe[3, 1] == 32 and pe[1, 1] == 39 and pe[0, 1] == 139
    assert pe[3, 2] == 139                       # first in worker 2's order: sees everything behind it
    # the last fragment of every order ends at its own length; the first at the total
    for w, o in enumerate(orders):
        assert pe[o[-1], w] == lens[o[-1]] and pe[o[0], w] == sum(lens)
    # same numbers as the (separately pinned) query-side contract: last new token sits at pos_end - 1
    S = 2
    loc = fo.locations_from_order(orders, lens, S)
    l2, _, _ = co.build_inputs(pe, S, inv_freq(8))
    assert np.array_equal(loc, l2)
    assert np.array_equal(l2[..., -1], pe - 1)


def test_rotary_tables_match_pinned_query_tables_and_torch():
    D = 64
    pos = np.array([[0, 1, 17], [1000, 65537, 999999]])
    c, s = co.rotary_tables(pos, inv_freq(D))
    c0, s0 = fo.rope_tables(pos[None], D, 10000.0, dtype=np.float64)       # fp64 angles
    small = pos < 2000                                                   # fp32 angle error grows with the position
    assert np.allclose(c[small], c0[0][small], atol=2e-4) and np.allclose(s[small], s0[0][small], atol=2e-4)
    # the fp32 pipeline itself: float32 product, float32 cos -- torch's routines on the same float32 angles
    ang = torch.from_numpy(pos).float()[..., None] * torch.from_numpy(inv_freq(D))
    emb = torch.cat([ang, ang], dim=-1)
    assert np.allclose(c, emb.cos().numpy(), atol=1.2e-7, rtol=0) and np.allclose(s, emb.sin().numpy(), atol=1.2e-7, rtol=0)
    # scaling and rounding to the model dtype
    cb, sb = co.rotary_tables(pos, inv_freq(D), attention_scaling=0.75, table_dtype="bf16")
    want = (emb.cos() * 0.75).to(torch.bfloat16).float().numpy()
    assert np.mean(cb == want) > 0.995 and np.abs(cb - want).max() <= 2 ** -8
    ch, _ = co.rotary_tables(pos, inv_freq(D), table_dtype="f16")
    assert np.mean(ch == emb.cos().half().float().numpy()) > 0.995


# ---------------------------------------------------------------------------------------------- key rotation
def test_rope_keys_is_a_rotation_by_pos_times_freq():
    D = 16
    x = rng.standard_normal((1, 1, 1, D))
    f = inv_freq(D).astype(np.float64)
    p = 11
    cos = np.cos(p * np.concatenate([f, f]))[None, None, None, :]
    sin = np.sin(p * np.concatenate([f, f]))[None, None, None, :]
    y = co.rope_keys(x, cos, sin, mode="exact", storage="f32")[0, 0, 0]
    for i in range(D // 2):
        a, b = x[0, 0, 0, i], x[0, 0, 0, i + D // 2]
        ang = p * f[i]
        assert y[i] == pytest.approx(a * math.cos(ang) - b * math.sin(ang), abs=1e-6)
        assert y[i + D // 2] == pytest.approx(b * math.cos(ang) + a * math.sin(ang), abs=1e-6)


def test_rope_keys_partial_rotary_passes_the_tail_through_and_keeps_norms():
    D, R = 32, 16
    x = rng.standard_normal((2, 3, 4, D))
    f = inv_freq(R).astype(np.float64)
    pos = np.arange(4)[None, None, :, None]
    cos, sin = np.cos(pos * np.concatenate([f, f])), np.sin(pos * np.concatenate([f, f]))
    y = co.rope_keys(x, cos, sin, mode="exact", storage="f32")
    assert np.array_equal(y[..., R:], x[..., R:].astype(np.float32))
    assert np.allclose(np.linalg.norm(y, axis=-1), np.linalg.norm(x, axis=-1), rtol=1e-6)
    assert np.allclose(y[:, :, 0], x[:, :, 0], atol=1e-7)                 # position 0 is the identity


def test_query_and_key_rotation_agree_on_relative_positions():
    """q rotated by the query-side oracle (pinned against the reference's rope_cpu) and k rotated here: the dot
    product depends only on the position difference, which fixes the sign and index conventions of rope_keys."""
    D = 32
    q = rng.standard_normal((1, 1, 1, D))         # [W, Hq, S, E]
    k = rng.standard_normal((1, 1, 1, D))
    f = inv_freq(D)

    def dot(pq, pk):
        cq, sq = co.rotary_tables(np.array([[[pq]]]), f)              # [F=1, W=1, S=1, D]
        ck, sk = co.rotary_tables(np.array([[pk]]), f)                # [W=1, S=1, D]
        rq = fo.rope_rotate(q, cq.astype(np.float64), sq.astype(np.float64))[0]
        rk = co.rope_keys(k, ck[:, None], sk[:, None], mode="exact", storage="f32")
        return float((rq * rk).sum())

    assert dot(5, 3) == pytest.approx(dot(105, 103), abs=2e-4)
    assert dot(9, 0) == pytest.approx(dot(40, 31), abs=2e-4)
    assert abs(dot(5, 3) - dot(5, 4)) > 1e-3


@pytest.mark.parametrize("storage,cs_storage", [("bf16", "bf16"), ("f16", "f16"), ("f32", "f32"), ("bf16", "f32"), ("f16", "f32")])
def test_rope_keys_eager_rounding_matches_torch_tensor_arithmetic(storage, cs_storage):
    """Same values through torch's own elementwise kernels in the same dtypes (rounding after every op)."""
    D, R = 64, 64
    x = torch.randn((3, 2, 5, D), generator=torch.Generator().manual_seed(1)).to(TDT[storage])
    pos = torch.tensor([[3, 4, 5, 6, 7], [100, 101, 102, 103, 104], [0, 1, 2, 3, 4]])
    ang = pos.float()[..., None] * torch.from_numpy(inv_freq(R))
    emb = torch.cat([ang, ang], -1)
    cos, sin = emb.cos().to(TDT[cs_storage]), emb.sin().to(TDT[cs_storage])
    x1, x2 = x[..., : R // 2], x[..., R // 2:]
    want = ((x * cos[:, None]) + (torch.cat((-x2, x1), dim=-1) * sin[:, None])).to(x.dtype)
    got = co.rope_keys(x.double().numpy(), cos.double().numpy()[:, None], sin.double().numpy()[:, None], storage=storage,
                       cs_storage=cs_storage, mode="eager")
    assert np.array_equal(got, want.double().numpy())


# ---------------------------------------------------------------------------------------------- append / merge
def test_append_left_masked_is_a_cat_of_the_unmasked_tail():
    dst = np.zeros((2, 10, 4))
    old = rng.standard_normal((2, 3, 4))
    dst[:, :3] = old
    new = rng.standard_normal((2, 5, 4))
    n = co.append_left_masked(dst, 3, new, 2)
    want = torch.cat([torch.from_numpy(old), torch.from_numpy(new)[:, -2:]], dim=1).numpy()
    assert n == 5 and np.array_equal(dst[:, :5], want) and (dst[:, 5:] == 0).all()


def test_merge_rerotation_composes_positions():
    """Keys stored rotated for positions 0..L-1, re-rotated by t, equal the raw keys rotated for t..t+L-1."""
    D, L, t = 32, 6, 41
    f = inv_freq(D)
    raw = rng.standard_normal((2, L, D))
    c0, s0 = co.rotary_tables(np.arange(L), f)
    stored = co.rope_keys(raw, c0[None], s0[None], mode="exact", storage="f32")
    merged = co.merge_rerotate(stored, t, f, storage="f32", mode="exact")
    c1, s1 = co.rotary_tables(np.arange(t, t + L), f)
    direct = co.rope_keys(raw, c1[None], s1[None], mode="exact", storage="f32")
    assert np.allclose(merged, direct, atol=5e-5)
    # and it is NOT the identity or a rotation by another offset
    assert np.abs(merged - stored).max() > 0.1


# ---------------------------------------------------------------------------------------------- the model library itself
def test_rotary_tables_match_the_model_librarys_rotary_embedding():
    """rotary_tables against the rotary embedding module of the installed `transformers` (the module the reference
    calls, python/hogwild/attention.py:191), for fp32 and bf16 activations and large positions."""
    transformers = pytest.importorskip("transformers")
    from transformers import Qwen2Config
    from transformers.models.qwen2.modeling_qwen2 import Qwen2RotaryEmbedding
    cfg = Qwen2Config(vocab_size=16, hidden_size=256, intermediate_size=64, num_hidden_layers=1, num_attention_heads=2,
                      num_key_value_heads=1, max_position_embeddings=4096)
    rot = Qwen2RotaryEmbedding(cfg)
    pos = torch.tensor([[0, 1, 2, 77, 4095, 31000]])
    inv = rot.inv_freq.numpy()
    for tdt, name in ((torch.float32, "f32"), (torch.bfloat16, "bf16"), (torch.float16, "f16")):
        cos, sin = rot(torch.zeros(1, 6, 256, dtype=tdt), pos)
        assert cos.dtype == tdt
        c, s = co.rotary_tables(pos.numpy(), inv, float(rot.attention_scaling), name)
        wc, ws = cos.float().numpy(), sin.float().numpy()
        if name == "f32":
            assert np.abs(c - wc).max() <= 1.2e-7 and np.abs(s - ws).max() <= 1.2e-7
        else:       # identical after rounding except where the fp32 values straddle a rounding boundary
            assert np.mean(c == wc) > 0.995 and np.mean(s == ws) > 0.995
            assert np.abs(c - wc).max() <= 2 ** -8 and np.abs(s - ws).max() <= 2 ** -8


def test_key_rotation_matches_the_model_librarys_apply_rotary_pos_emb():
    transformers = pytest.importorskip("transformers")
    from transformers.models.qwen2.modeling_qwen2 import apply_rotary_pos_emb
    D = 64
    g = torch.Generator().manual_seed(3)
    for tdt, name in ((torch.float32, "f32"), (torch.bfloat16, "bf16"), (torch.float16, "f16")):
        k = torch.randn((2, 3, 5, D), generator=g).to(tdt)
        pos = torch.tensor([[3, 4, 5, 6, 7], [100, 101, 102, 103, 104]])
        ang = pos.float()[..., None] * torch.from_numpy(inv_freq(D))
        emb = torch.cat([ang, ang], -1)
        cos, sin = emb.cos().to(tdt), emb.sin().to(tdt)
        _, want = apply_rotary_pos_emb(k, k, cos, sin)            # unsqueezes the tables over the head dimension
        got = co.rope_keys(k.double().numpy(), cos.double().numpy()[:, None], sin.double().numpy()[:, None], storage=name,
                           cs_storage=name, mode="eager")
        assert np.array_equal(got, want.double().numpy())
