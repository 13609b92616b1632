"""CPU oracle for the paged variants of the Hogwild! attention path.  TEST INFRASTRUCTURE ONLY.

Nothing in the product package imports this module.  It restates, in numpy, what the reference's paged
kernels compute:

  * paged KV append ................. src/cache.cuh:6-49                 (copy_to_blocks_kernel)
  * paged attention ................. src/kernels/kernel_v21.cuh:318-602 (block-table addressing :405-411,
                                      mask bound :386-388), launcher :998-1043
  * varlen paged attention .......... src/kernels/kernel_v21.cuh:658-899 (packed queries :698-699,733;
                                      locations [F,total_q] :725; fragment_lengths [F,W] :726;
                                      token -> sequence lookup :15-23), launcher :1045-1086

In both attention variants every "fragment" f reads the SAME paged sequence of worker w (the block-table row
w), from position 0, with its own queries, its own visibility bound min(fragment_lengths, location + 1) and
one softmax over the union of all fragments' visible keys (kernel_v21.cuh:385-495).

Pinning status (tests/test_paged_oracle_pins.py):
  copy_to_blocks ........ pinned: literal flat-offset python loops over the flattened caches; round trip
                          through gather_sequence.
  gather_sequence ....... pinned: literal flat-offset python loops; identity block table gives a reshape.
  paged_sdpa ............ pinned: brute-force python loops with the reference's flat offsets; equality with the
                          (separately pinned) fragment attention over gathered contiguous sequences; torch
                          scaled_dot_product_attention for a causal single-fragment case.
  varlen_paged_sdpa ..... pinned: equals paged_sdpa when all sequences have the same number of query tokens;
                          brute-force python loops for a ragged case (including an empty sequence).
The reference ships no tests, fixtures or golden vectors for these operators.
"""
from __future__ import annotations

import math
from typing import Tuple

import numpy as np

NEG_INF = float("-inf")


def copy_to_blocks(key_states: np.ndarray, value_states: np.ndarray, key_cache: np.ndarray, value_cache: np.ndarray,
                   block_table: np.ndarray, seq_lengths: np.ndarray) -> None:
    """Scatter new K/V rows into the paged caches, in place (src/cache.cuh:29-48).

    key_states [B, Hkv, S_new, E], value_states [B, Hkv, S_new, Ev]; caches [NumBlocks, Hkv, BlockSize, E|Ev];
    block_table int [B, max_blocks]; seq_lengths int [B] = tokens already in each sequence.  New token t of
    sequence b lands at position seq_lengths[b] + t of that sequence.
    """
    B, Hkv, S_new, _ = key_states.shape
    bs = key_cache.shape[2]
    for b in range(B):
        pos = int(seq_lengths[b]) + np.arange(S_new)
        blk = block_table[b, pos // bs]
        off = pos % bs
        # advanced indices (blk, off) separated by the head slice: result axes are [S_new, Hkv, E]
        key_cache[blk, :, off, :] = np.transpose(key_states[b], (1, 0, 2))
        value_cache[blk, :, off, :] = np.transpose(value_states[b], (1, 0, 2))


def gather_sequence(cache: np.ndarray, block_table_row: np.ndarray, length: int) -> np.ndarray:
    """The first `length` positions of one paged sequence as a contiguous [Hkv, length, D] array
    (position l lives in block block_table_row[l // BlockSize] at offset l % BlockSize, kernel_v21.cuh:406-411)."""
    bs = cache.shape[2]
    pos = np.arange(length)
    rows = cache[block_table_row[pos // bs], :, pos % bs, :]      # [length, Hkv, D]
    return np.ascontiguousarray(np.transpose(rows, (1, 0, 2)))


def _attend(q: np.ndarray, lims: np.ndarray, k: np.ndarray, v: np.ndarray, scale: float, dtype) -> Tuple[np.ndarray, np.ndarray]:
    """q [F, Hq, T, E] of one sequence, lims int [F, T] (visible keys: l < lims[f, t]); k [Hkv, L, E]; v [Hkv, L, Ev]."""
    F, Hq, T, E = q.shape
    Hkv, L, Ev = v.shape
    G = Hq // Hkv
    qg = q.astype(dtype).reshape(F, Hkv, G, T, E)
    a = np.einsum("fkgte,kle->kgtfl", qg, k.astype(dtype), optimize=True) * dtype(scale)      # [Hkv,G,T,F,L]
    vis = np.arange(L)[None, None, :] < np.transpose(lims, (1, 0))[:, :, None]                 # [T,F,L]
    a = np.where(vis[None, None], a, NEG_INF).reshape(Hkv, G, T, F * L)
    m = np.max(a, axis=-1, keepdims=True) if F * L > 0 else np.full(a.shape[:-1] + (1,), NEG_INF)
    m_safe = np.where(np.isfinite(m), m, 0.0)
    p = np.exp(a - m_safe)
    den = p.sum(axis=-1, keepdims=True)
    with np.errstate(divide="ignore"):
        lse = (np.log(den) + m_safe)[..., 0]
    pf = p.reshape(Hkv, G, T, F, L).sum(axis=3)                    # every fragment weights the same V rows
    out = np.einsum("kgtl,kle->kgte", pf, v.astype(dtype), optimize=True) / np.where(den > 0, den, 1.0)
    return out.reshape(Hq, T, Ev), lse.reshape(Hq, T)


def paged_sdpa(queries: np.ndarray, locations: np.ndarray, fragment_lengths: np.ndarray, key_cache: np.ndarray,
               value_cache: np.ndarray, block_table: np.ndarray, scale: float, dtype=np.float64) -> Tuple[np.ndarray, np.ndarray]:
    """queries [F, W, Hq, S, E] (already rotated); locations int [F, W, S]; fragment_lengths int [F];
    caches [NumBlocks, Hkv, BlockSize, E|Ev]; block_table int [W, max_blocks].
    Query (w, s) sees position l of sequence w through fragment f iff l < min(fragment_lengths[f], locations[f,w,s] + 1)
    (kernel_v21.cuh:386-388).  Returns out [W, Hq, S, Ev] and lse [W, Hq, S] (natural log; -inf and a zero row when
    nothing is visible)."""
    F, W, Hq, S, E = queries.shape
    Ev = value_cache.shape[-1]
    out = np.zeros((W, Hq, S, Ev), dtype=dtype)
    lse = np.full((W, Hq, S), NEG_INF, dtype=dtype)
    for w in range(W):
        lims = np.minimum(np.asarray(fragment_lengths)[:, None], locations[:, w, :] + 1)      # [F, S]
        lims = np.maximum(lims, 0)
        L = int(lims.max()) if lims.size else 0
        k = gather_sequence(key_cache, block_table[w], L)
        v = gather_sequence(value_cache, block_table[w], L)
        out[w], lse[w] = _attend(queries[:, w], lims, k, v, scale, dtype)
    return out, lse


def varlen_paged_sdpa(queries: np.ndarray, locations: np.ndarray, fragment_lengths: np.ndarray, key_cache: np.ndarray,
                      value_cache: np.ndarray, block_table: np.ndarray, cu_seqlens_q: np.ndarray, scale: float,
                      dtype=np.float64) -> Tuple[np.ndarray, np.ndarray]:
    """queries [F, total_q, Hq, E] packed over sequences; locations int [F, total_q]; fragment_lengths int [F, W];
    cu_seqlens_q int [W+1]: query tokens cu[w] .. cu[w+1]-1 belong to sequence w (kernel_v21.cuh:15-23).
    Returns out [total_q, Hq, Ev] and lse [total_q, Hq]."""
    F, T, Hq, E = queries.shape
    W = len(cu_seqlens_q) - 1
    Ev = value_cache.shape[-1]
    out = np.zeros((T, Hq, Ev), dtype=dtype)
    lse = np.full((T, Hq), NEG_INF, dtype=dtype)
    fl = np.asarray(fragment_lengths).reshape(F, W)
    for w in range(W):
        a, b = int(cu_seqlens_q[w]), int(cu_seqlens_q[w + 1])
        if b <= a:
            continue
        lims = np.maximum(np.minimum(fl[:, w][:, None], locations[:, a:b] + 1), 0)            # [F, S_w]
        L = int(lims.max())
        k = gather_sequence(key_cache, block_table[w], L)
        v = gather_sequence(value_cache, block_table[w], L)
        o, l = _attend(np.transpose(queries[:, a:b], (0, 2, 1, 3)), lims, k, v, scale, dtype)  # [Hq, S_w, *]
        out[a:b] = np.transpose(o, (1, 0, 2))
        lse[a:b] = np.transpose(l, (1, 0))
    return out, lse


# ----------------------------------------------------------------------------------------------
# brute force with the reference's flat offsets (tiny shapes only; used to pin the functions above)
# ----------------------------------------------------------------------------------------------
def paged_bruteforce(queries, locations, fragment_lengths, key_cache, value_cache, block_table, scale,
                     cu_seqlens_q=None):
    """Python loops over flattened buffers with the address arithmetic of kernel_v21.cuh:359,393,406-411
    (and :698-699,725-726,733 when cu_seqlens_q is given)."""
    kc = np.ascontiguousarray(key_cache).reshape(-1)
    vc = np.ascontiguousarray(value_cache).reshape(-1)
    _, Hkv, bs, E = key_cache.shape
    Ev = value_cache.shape[-1]
    bt = np.ascontiguousarray(block_table)
    max_blocks = bt.shape[1]
    btf = bt.reshape(-1)
    qf = np.ascontiguousarray(queries).reshape(-1)
    lf = np.ascontiguousarray(locations).reshape(-1)
    flf = np.ascontiguousarray(fragment_lengths).reshape(-1)
    varlen = cu_seqlens_q is not None
    if varlen:
        F, T, Hq, _ = queries.shape
        W = len(cu_seqlens_q) - 1
        out = np.zeros((T, Hq, Ev))
        lse = np.full((T, Hq), NEG_INF)
        rows = []
        for t in range(T):
            w = 0
            while w < W and t >= cu_seqlens_q[w + 1]:
                w += 1
            rows.append((w, t))
    else:
        F, W, Hq, S, _ = queries.shape
        out = np.zeros((W, Hq, S, Ev))
        lse = np.full((W, Hq, S), NEG_INF)
        rows = [(w, s) for w in range(W) for s in range(S)]
    G = Hq // Hkv
    for (w, x) in rows:
        for h in range(Hq):
            hkv = h // G
            sc, vv = [], []
            for f in range(F):
                if varlen:
                    q_loc = int(lf[f * T + x])
                    L = int(flf[f * W + w])
                    q_off = f * T * Hq * E + (x * Hq + h) * E
                else:
                    q_loc = int(lf[(f * W + w) * S + x])
                    L = int(flf[f])
                    q_off = f * (E * S * Hq * W) + ((w * Hq + h) * S + x) * E
                for l in range(min(L, q_loc + 1)):
                    blk = int(btf[w * max_blocks + l // bs])
                    k_off = ((blk * Hkv + hkv) * bs + l % bs) * E
                    v_off = ((blk * Hkv + hkv) * bs + l % bs) * Ev
                    sc.append(scale * sum(float(qf[q_off + e]) * float(kc[k_off + e]) for e in range(E)))
                    vv.append(vc[v_off:v_off + Ev].astype(np.float64))
            if not sc:
                continue
            m = max(sc)
            ws = [math.exp(v - m) for v in sc]
            den = sum(ws)
            acc = np.zeros(Ev)
            for wt, vrow in zip(ws, vv):
                acc += (wt / den) * vrow
            if varlen:
                out[x, h] = acc
                lse[x, h] = m + math.log(den)
            else:
                out[w, h, x] = acc
                lse[w, h, x] = m + math.log(den)
    return out, lse


def copy_to_blocks_bruteforce(key_states, value_states, key_cache, value_cache, block_table, seq_lengths):
    """Python loops over flattened buffers with the offsets of src/cache.cuh:29-48.  Returns new flat caches."""
    B, Hkv, S_new, E = key_states.shape
    Ev = value_states.shape[-1]
    bs = key_cache.shape[2]
    max_blocks = block_table.shape[1]
    kc = np.ascontiguousarray(key_cache).reshape(-1).copy()
    vc = np.ascontiguousarray(value_cache).reshape(-1).copy()
    ks = np.ascontiguousarray(key_states).reshape(-1)
    vs = np.ascontiguousarray(value_states).reshape(-1)
    btf = np.ascontiguousarray(block_table).reshape(-1)
    for b in range(B):
        for h in range(Hkv):
            for t in range(S_new):
                total_pos = int(seq_lengths[b]) + t
                blk = int(btf[b * max_blocks + total_pos // bs])
                off = total_pos % bs
                src_k = (b * Hkv + h) * S_new * E + t * E
                src_v = (b * Hkv + h) * S_new * Ev + t * Ev
                dst_k = (blk * Hkv + h) * bs * E + off * E
                dst_v = (blk * Hkv + h) * bs * Ev + off * Ev
                kc[dst_k:dst_k + E] = ks[src_k:src_k + E]
                vc[dst_v:dst_v + Ev] = vs[src_v:src_v + Ev]
    return kc.reshape(key_cache.shape), vc.reshape(value_cache.shape)
