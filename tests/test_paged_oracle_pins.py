"""Pins for oracle/paged_oracle.py: every function is checked against facts that do not depend on its own
(vectorised) formulation — python loops over flattened buffers with the reference's offset arithmetic, the
separately pinned fragment attention over gathered sequences, torch's scaled_dot_product_attention, and
layout equivalences.  The reference ships no tests or fixtures for the paged operators."""
import numpy as np
import pytest
import torch

from oracle import hogwild_oracle as fo
from oracle import paged_oracle as po

rng = np.random.default_rng(777)


def make_cache(num_blocks, Hkv, bs, E, Ev):
    kc = rng.standard_normal((num_blocks, Hkv, bs, E))
    vc = rng.standard_normal((num_blocks, Hkv, bs, Ev))
    return kc, vc


def random_table(W, max_blocks, num_blocks):
    """Every sequence gets distinct physical blocks, in shuffled order."""
    perm = rng.permutation(num_blocks)[: W * max_blocks]
    return perm.reshape(W, max_blocks).astype(np.int32)


# ------------------------------------------------------------------------------------------ gather / scatter
def test_gather_matches_flat_offsets():
    NB, Hkv, bs, E = 7, 3, 4, 6
    kc, _ = make_cache(NB, Hkv, bs, E, E)
    row = np.array([5, 0, 3], dtype=np.int32)
    L = 10
    got = po.gather_sequence(kc, row, L)
    flat = kc.reshape(-1)
    for h in range(Hkv):
        for l in range(L):
            off = ((int(row[l // bs]) * Hkv + h) * bs + l % bs) * E
            assert np.array_equal(got[h, l], flat[off:off + E])


def test_gather_identity_table_is_a_reshape():
    NB, Hkv, bs, E = 4, 2, 8, 5
    kc, _ = make_cache(NB, Hkv, bs, E, E)
    got = po.gather_sequence(kc, np.arange(NB, dtype=np.int32), NB * bs)
    want = np.transpose(kc, (1, 0, 2, 3)).reshape(Hkv, NB * bs, E)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("bs,S_new", [(4, 1), (4, 6), (1, 3), (16, 5)])
def test_copy_to_blocks_matches_flat_loops_and_round_trips(bs, S_new):
    B, Hkv, E, Ev, max_blocks = 3, 2, 6, 4, 5
    NB = B * max_blocks + 2
    kc, vc = make_cache(NB, Hkv, bs, E, Ev)
    bt = random_table(B, max_blocks, NB)
    seq = np.array([0, bs * 2 - 1 if bs * 2 - 1 + S_new <= bs * max_blocks else 0, 3 % (bs * max_blocks - S_new + 1)], dtype=np.int32)
    ks = rng.standard_normal((B, Hkv, S_new, E))
    vs = rng.standard_normal((B, Hkv, S_new, Ev))
    want_k, want_v = po.copy_to_blocks_bruteforce(ks, vs, kc, vc, bt, seq)
    got_k, got_v = kc.copy(), vc.copy()
    po.copy_to_blocks(ks, vs, got_k, got_v, bt, seq)
    assert np.array_equal(got_k, want_k) and np.array_equal(got_v, want_v)
    # exactly B*Hkv*S_new rows changed, everything else untouched
    assert int((got_k != kc).any(axis=-1).sum()) == B * Hkv * S_new
    for b in range(B):
        g = po.gather_sequence(got_k, bt[b], int(seq[b]) + S_new)
        assert np.array_equal(g[:, int(seq[b]):], ks[b])
        g = po.gather_sequence(got_v, bt[b], int(seq[b]) + S_new)
        assert np.array_equal(g[:, int(seq[b]):], vs[b])


# ------------------------------------------------------------------------------------------ paged attention
def paged_problem(F, W, Hq, Hkv, S, E, Ev, bs, max_blocks, lens=None):
    NB = W * max_blocks + 3
    kc, vc = make_cache(NB, Hkv, bs, E, Ev)
    bt = random_table(W, max_blocks, NB)
    q = rng.standard_normal((F, W, Hq, S, E))
    cap = bs * max_blocks
    fl = np.array(lens if lens is not None else rng.integers(1, cap + 1, size=F), dtype=np.int32)
    loc = rng.integers(-1, cap + 2, size=(F, W, S)).astype(np.int32)
    return q, loc, fl, kc, vc, bt


@pytest.mark.parametrize("F,S,bs", [(1, 1, 4), (2, 3, 3), (3, 2, 1)])
def test_paged_matches_bruteforce_flat_offsets(F, S, bs):
    q, loc, fl, kc, vc, bt = paged_problem(F, 2, 4, 2, S, 6, 5, bs, 4)
    loc[0, 0, 0] = -1 if F == 1 else loc[0, 0, 0]        # one row that sees nothing (F == 1 case)
    out, lse = po.paged_sdpa(q, loc, fl, kc, vc, bt, 0.37)
    bo, bl = po.paged_bruteforce(q, loc, fl, kc, vc, bt, 0.37)
    assert np.allclose(out, bo, atol=1e-12)
    assert np.array_equal(np.isneginf(lse), np.isneginf(bl))
    fin = np.isfinite(bl)
    assert np.allclose(lse[fin], bl[fin], atol=1e-12)
    if F == 1:
        assert np.isneginf(lse[0, :, 0]).all() and (out[0, :, 0] == 0).all()


def test_paged_equals_fragment_attention_over_gathered_sequences():
    """Each worker's result equals the (independently pinned) fragment attention with W = 1 whose fragment f is
    the worker's own sequence cut to fragment_lengths[f]."""
    F, W, Hq, Hkv, S, E, Ev, bs, mb = 3, 3, 6, 2, 2, 8, 8, 4, 6
    q, loc, fl, kc, vc, bt = paged_problem(F, W, Hq, Hkv, S, E, Ev, bs, mb)
    out, lse = po.paged_sdpa(q, loc, fl, kc, vc, bt, 0.25)
    for w in range(W):
        keys = [po.gather_sequence(kc, bt[w], int(fl[f])) for f in range(F)]
        vals = [po.gather_sequence(vc, bt[w], int(fl[f])) for f in range(F)]
        fo_out, fo_lse = fo.sdpa_fragments(q[:, w:w + 1], loc[:, w:w + 1], keys, vals, 0.25)
        assert np.allclose(out[w], fo_out[0], atol=1e-12)
        both = np.isfinite(fo_lse[0])
        assert np.allclose(lse[w][both], fo_lse[0][both], atol=1e-12)
        assert np.array_equal(np.isneginf(lse[w]), np.isneginf(fo_lse[0]))


def test_paged_single_fragment_is_causal_attention_torch():
    """F = 1, identity-free block table, locations = absolute positions: ordinary causal attention of the last S
    tokens over the sequence, checked with torch's library routine."""
    W, Hq, Hkv, S, E, bs, mb = 2, 4, 2, 5, 16, 4, 5
    L = 17
    q, _, _, kc, vc, bt = paged_problem(1, W, Hq, Hkv, S, E, E, bs, mb)
    loc = np.broadcast_to(np.arange(L - S, L, dtype=np.int32)[None, None, :], (1, W, S)).copy()
    fl = np.array([L], dtype=np.int32)
    scale = 1.0 / np.sqrt(E)
    out, _ = po.paged_sdpa(q, loc, fl, kc, vc, bt, scale)
    for w in range(W):
        k = torch.from_numpy(po.gather_sequence(kc, bt[w], L)).repeat_interleave(Hq // Hkv, dim=0)
        v = torch.from_numpy(po.gather_sequence(vc, bt[w], L)).repeat_interleave(Hq // Hkv, dim=0)
        mask = torch.arange(L)[None, :] <= torch.arange(L - S, L)[:, None]
        want = torch.nn.functional.scaled_dot_product_attention(torch.from_numpy(q[0, w]), k, v, attn_mask=mask, scale=scale)
        assert np.allclose(out[w], want.numpy(), atol=1e-10)


def test_fragment_length_bounds_visibility():
    """A location beyond fragment_lengths sees exactly fragment_lengths keys (min(L, loc + 1))."""
    q, loc, fl, kc, vc, bt = paged_problem(1, 1, 2, 1, 1, 4, 4, 4, 4, lens=[5])
    loc[:] = 100
    a, la = po.paged_sdpa(q, loc, fl, kc, vc, bt, 1.0)
    loc[:] = 4
    b, lb = po.paged_sdpa(q, loc, fl, kc, vc, bt, 1.0)
    assert np.array_equal(a, b) and np.array_equal(la, lb)
    # uniform logits (zero query): out is the mean of the 5 visible V rows, lse = ln 5
    q[:] = 0
    o, l = po.paged_sdpa(q, loc, fl, kc, vc, bt, 1.0)
    assert np.allclose(o[0, 0, 0], po.gather_sequence(vc, bt[0], 5)[0].mean(axis=0), atol=1e-12)
    assert np.allclose(l, np.log(5.0))


# ------------------------------------------------------------------------------------------ varlen
def test_varlen_equal_lengths_is_the_paged_layout_transposed():
    F, W, Hq, Hkv, S, E, bs, mb = 2, 3, 4, 2, 3, 8, 4, 5
    q, loc, fl, kc, vc, bt = paged_problem(F, W, Hq, Hkv, S, E, E, bs, mb)
    out, lse = po.paged_sdpa(q, loc, fl, kc, vc, bt, 0.3)
    qv = np.transpose(q, (0, 1, 3, 2, 4)).reshape(F, W * S, Hq, E)
    locv = loc.reshape(F, W * S)
    flv = np.repeat(fl[:, None], W, axis=1)
    cu = np.arange(W + 1, dtype=np.int32) * S
    vo, vl = po.varlen_paged_sdpa(qv, locv, flv, kc, vc, bt, cu, 0.3)
    assert np.allclose(vo, np.transpose(out, (0, 2, 1, 3)).reshape(W * S, Hq, E), atol=1e-13)
    want_l = np.transpose(lse, (0, 2, 1)).reshape(W * S, Hq)
    assert np.array_equal(np.isneginf(vl), np.isneginf(want_l))
    assert np.allclose(vl[np.isfinite(want_l)], want_l[np.isfinite(want_l)], atol=1e-13)


def test_varlen_ragged_matches_bruteforce():
    F, W, Hq, Hkv, E, Ev, bs, mb = 2, 4, 4, 2, 6, 5, 3, 5
    cu = np.array([0, 3, 3, 4, 9], dtype=np.int32)       # sequence 1 has no query tokens
    T = int(cu[-1])
    NB = W * mb + 1
    kc, vc = make_cache(NB, Hkv, bs, E, Ev)
    bt = random_table(W, mb, NB)
    q = rng.standard_normal((F, T, Hq, E))
    fl = rng.integers(0, bs * mb + 1, size=(F, W)).astype(np.int32)
    loc = rng.integers(-1, bs * mb + 2, size=(F, T)).astype(np.int32)
    out, lse = po.varlen_paged_sdpa(q, loc, fl, kc, vc, bt, cu, 0.41)
    bo, bl = po.paged_bruteforce(q, loc, fl, kc, vc, bt, 0.41, cu_seqlens_q=cu)
    assert np.allclose(out, bo, atol=1e-12)
    assert np.array_equal(np.isneginf(lse), np.isneginf(bl))
    assert np.allclose(lse[np.isfinite(bl)], bl[np.isfinite(bl)], atol=1e-12)
