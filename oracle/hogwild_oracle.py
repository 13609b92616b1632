"""CPU oracle for the Hogwild! fragmented-KV attention path.  TEST INFRASTRUCTURE ONLY.

Nothing in the product package imports this module: it exists so that tests, the smoke check and
the CPU-baseline leg of the benchmark have an independent statement of what the HIP kernels must
compute.  It is a fresh restatement (numpy for the exact fp64/fp32 forms, torch for a fast
multi-threaded fp32 form) of the reference's algorithm:

  * attention over fragments ......... python/hogwild/attention.py:38-67   (hogwild_sdpa_pt)
  * rotate-half RoPE on the query .... python/hogwild/attention.py:77-90   (apply_rotary_pos_emb)
                                       src/q_rope.h:3-35, src/rope.cuh:18-51 (index conventions)
  * mask bound ....................... src/kernels/kernel_v21.cuh:96-98    (maxL = min(L, loc+1))
  * base-2 LSE + split merge ......... src/kernels/kernel_v21.cuh:60,300,630-645
  * caller contract for `locations` .. python/hogwild/attention.py:164-196

Pinning status (what independent facts each function is checked against lives in
tests/test_oracle_pins.py):
  rope_rotate ............ pinned: closed-form 2-D rotation, norm preservation, relative-position
                           property, p=0 identity, and the reference's own rope_cpu (src/q_rope.h)
                           compiled into oracle/_ref when /root/reference is present.
  sdpa_fragments ......... pinned: torch scaled_dot_product_attention with an explicit mask,
                           brute-force python loops, uniform-logit and one-hot closed forms,
                           fragment-order/fragment-split invariance, logsumexp for the LSE.
  fused_reference ........ pinned: equals ordinary causal RoPE attention over the concatenation of
                           a worker's fragments with global positions (textbook equivalence).
  locations_from_order ... pinned: closed form sum of lengths.
The reference ships no tests, fixtures or golden vectors for this path, so none can be cited.
"""
from __future__ import annotations

import math
from typing import List, Sequence, Tuple

import numpy as np

NEG_INF = float("-inf")


# ----------------------------------------------------------------------------------------------
# RoPE
# ----------------------------------------------------------------------------------------------
def rope_tables(positions: np.ndarray, rot_dim: int, base: float, dtype=np.float32):
    """cos/sin tables in the layout HF rotary embeddings produce: angle_i = pos * base**(-2i/rot_dim)
    for i < rot_dim/2, duplicated to length rot_dim (`cat(freqs, freqs)`), returned with the shape
    positions.shape + (rot_dim,).  Caller side of python/hogwild/attention.py:190-193."""
    half = rot_dim // 2
    inv_freq = base ** (-(np.arange(half, dtype=np.float64) * 2.0) / rot_dim)
    ang = positions.astype(np.float64)[..., None] * inv_freq
    ang = np.concatenate([ang, ang], axis=-1)
    return np.cos(ang).astype(dtype), np.sin(ang).astype(dtype)


def rope_rotate(q: np.ndarray, cos: np.ndarray, sin: np.ndarray, *, second_half_index: str = "first",
                dtype=np.float64) -> np.ndarray:
    """Per-fragment rotate-half RoPE of the query.

    q   [W, Hq, S, E]          cos, sin [F, W, S, R]   ->   [F, W, Hq, S, E]
    For e < R/2 (h = R/2):   out[e]   = x[e]   * cos[e]  - x[e+h] * sin[e]
                             out[e+h] = x[e+h] * cos[j]  + x[e]   * sin[j]
    with j = e      when second_half_index == "first"  (the GPU op: src/rope.cuh:30-46)
         j = e + h  when second_half_index == "own"    (python/hogwild/attention.py:84-90, src/q_rope.h:18-25)
    e >= R passes through (src/rope.cuh:48-51).  The two conventions agree whenever cos/sin are
    `cat(c, c)` tables, which is what the caller produces.
    """
    F, W, S, R = cos.shape
    h = R // 2
    x = q.astype(dtype)
    c = cos.astype(dtype)[:, :, None, :, :]   # [F,W,1,S,R]
    s = sin.astype(dtype)[:, :, None, :, :]
    x1 = x[None, ..., :h]
    x2 = x[None, ..., h:R]
    if second_half_index == "first":
        c2, s2 = c[..., :h], s[..., :h]
    elif second_half_index == "own":
        c2, s2 = c[..., h:R], s[..., h:R]
    else:
        raise ValueError(second_half_index)
    lo = x1 * c[..., :h] - x2 * s[..., :h]
    hi = x2 * c2 + x1 * s2
    rest = np.broadcast_to(x[None, ..., R:], (F,) + x.shape[:-1] + (x.shape[-1] - R,))
    return np.concatenate([lo, hi, rest], axis=-1)


# ----------------------------------------------------------------------------------------------
# attention over fragments
# ----------------------------------------------------------------------------------------------
def _frag3(a: np.ndarray) -> np.ndarray:
    """K/V fragments are [Hkv, L, D] or [1, Hkv, L, D] (src/binding.cu:85-94)."""
    return a[0] if a.ndim == 4 else a


def sdpa_fragments(queries: np.ndarray, locations: np.ndarray, keys: Sequence[np.ndarray],
                   values: Sequence[np.ndarray], scale: float, dtype=np.float64
                   ) -> Tuple[np.ndarray, np.ndarray]:
    """Attention of pre-rotated queries over KV fragments (python/hogwild/attention.py:38-67).

    queries [F, W, Hq, S, E]; locations int [F, W, S]; keys[f] [Hkv, L_f, E]; values[f] [Hkv, L_f, Ev].
    Query (w, s) sees key l of fragment f iff l <= locations[f, w, s]  (attention.py:54: mask = kp > qp).
    q head h uses kv head h // (Hq/Hkv) (attention.py:47-48).  Softmax is over the union of the visible
    keys of all fragments (attention.py:60-63).
    Returns out [W, Hq, S, Ev] and lse [W, Hq, S] = ln sum_visible exp(scale * q.k)   (natural log;
    the reference kernel's internal value is this divided by ln 2, kernel_v21.cuh:60,300).
    Rows with no visible key give zeros and lse = -inf (the kernel's behaviour, kernel_v21.cuh:238-245,
    627-629; the torch function would give NaN).
    """
    F, W, Hq, S, E = queries.shape
    Hkv = _frag3(keys[0]).shape[0]
    G = Hq // Hkv
    logits = []
    vals = []
    for f in range(F):
        k = _frag3(keys[f]).astype(dtype)                            # [Hkv, L, E]
        v = _frag3(values[f]).astype(dtype)                          # [Hkv, L, Ev]
        L = k.shape[1]
        # q head h = kv*G + g reads kv head kv: group the q heads instead of replicating K
        qf = queries[f].astype(dtype).reshape(W, Hkv, G, S, E)
        a = (np.einsum("wkgse,kle->wkgsl", qf, k, optimize=True) * dtype(scale)).reshape(W, Hq, S, L)
        kp = np.arange(L)[None, None, None, :]
        qp = locations[f][:, None, :, None]
        a = np.where(kp > qp, NEG_INF, a)
        logits.append(a)
        vals.append(v)
    a = np.concatenate(logits, axis=-1)                              # [W,Hq,S,sumL]
    v = np.concatenate(vals, axis=-2)                                # [Hkv,sumL,Ev]
    m = np.max(a, axis=-1, keepdims=True)
    m_safe = np.where(np.isfinite(m), m, 0.0)
    p = np.exp(a - m_safe)
    den = p.sum(axis=-1, keepdims=True)
    with np.errstate(divide="ignore"):
        lse = (np.log(den) + m_safe)[..., 0]
    Ev = v.shape[-1]
    out = np.einsum("wkgsl,kle->wkgse", p.reshape(W, Hkv, G, S, -1), v, optimize=True).reshape(W, Hq, S, Ev)
    out = out / np.where(den > 0, den, 1.0)
    return out.astype(dtype), lse.astype(dtype)


def round_to(x: np.ndarray, kind: str) -> np.ndarray:
    """Round an fp32/fp64 array to the storage type `kind` ("f32" | "f16" | "bf16") and return it as
    float64-exact values of that type (RNE), as the reference stores rotated q in the tensor dtype
    (src/rope.cuh:43-45, attention.py:90)."""
    if kind == "f32":
        return x.astype(np.float32)
    if kind == "f16":
        return x.astype(np.float32).astype(np.float16).astype(np.float32)
    if kind == "bf16":
        u = np.ascontiguousarray(x.astype(np.float32)).view(np.uint32).astype(np.uint64)
        r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
        return r.astype(np.uint32).view(np.float32)
    raise ValueError(kind)


def fused_reference(q: np.ndarray, locations: np.ndarray, keys, values, scale: float,
                    cos: np.ndarray, sin: np.ndarray, *, storage: str = "f32",
                    second_half_index: str = "first", dtype=np.float64):
    """rope-then-attention, the semantics of the fused op (src/binding.cu:324-340): rotate q per
    fragment, round the rotated q to the storage dtype, attend.  Returns (out, lse, rotated_q)."""
    rq = rope_rotate(q, cos, sin, second_half_index=second_half_index, dtype=dtype)
    rq = round_to(rq, storage).astype(dtype)
    out, lse = sdpa_fragments(rq, locations, keys, values, scale, dtype=dtype)
    return out, lse, rq


def sdpa_bruteforce(queries, locations, keys, values, scale):
    """Pure-python triple loop in float (python floats are fp64).  Only for tiny shapes; used to pin
    sdpa_fragments independently of any vectorised indexing."""
    F, W, Hq, S, E = queries.shape
    Hkv = _frag3(keys[0]).shape[0]
    Ev = _frag3(values[0]).shape[-1]
    G = Hq // Hkv
    out = np.zeros((W, Hq, S, Ev))
    lse = np.full((W, Hq, S), NEG_INF)
    for w in range(W):
        for h in range(Hq):
            for s in range(S):
                sc, vv = [], []
                for f in range(F):
                    k = _frag3(keys[f])[h // G]
                    v = _frag3(values[f])[h // G]
                    for l in range(k.shape[0]):
                        if l <= int(locations[f, w, s]):
                            sc.append(scale * sum(float(queries[f, w, h, s, e]) * float(k[l, e]) for e in range(E)))
                            vv.append(v[l])
                if not sc:
                    continue
                m = max(sc)
                ws = [math.exp(x - m) for x in sc]
                den = sum(ws)
                lse[w, h, s] = m + math.log(den)
                for wt, vrow in zip(ws, vv):
                    out[w, h, s] += (wt / den) * vrow.astype(np.float64)
    return out, lse


def merge_partials(outs: Sequence[np.ndarray], lses: Sequence[np.ndarray]):
    """LSE-weighted merge of normalised partial results (kernel_v21.cuh:605-656), closed form:
    lse = ln sum_i exp(lse_i), out = sum_i exp(lse_i - lse) out_i."""
    L = np.stack(lses)
    m = np.max(L, axis=0)
    m_safe = np.where(np.isfinite(m), m, 0.0)
    wts = np.exp(L - m_safe)
    den = wts.sum(axis=0)
    with np.errstate(divide="ignore"):
        lse = np.log(den) + m_safe
    out = sum(w[..., None] * o for w, o in zip(wts, outs)) / np.where(den > 0, den, 1.0)[..., None]
    return out, lse


# ----------------------------------------------------------------------------------------------
# caller contract
# ----------------------------------------------------------------------------------------------
def locations_from_order(orders: List[List[int]], lens: Sequence[int], S: int) -> np.ndarray:
    """locations[f, w, s] for W workers whose cache orderings are `orders[w]` (lists of fragment ids,
    oldest first; a fragment absent from a worker's ordering is invisible to it, loc = -1).
    Restates python/hogwild/attention.py:173-181: walking worker w's ordering from the end,
    pos += len(fragment); loc = arange(pos - S, pos)."""
    F = len(lens)
    W = len(orders)
    loc = np.full((F, W, S), -1, dtype=np.int32)
    for w, order in enumerate(orders):
        pos = 0
        for f in reversed(order):
            pos += int(lens[f])
            loc[f, w, :] = np.arange(pos - S, pos, dtype=np.int32)
    return loc


# ----------------------------------------------------------------------------------------------
# fast multi-threaded fp32 form (torch) — the "CPU baseline" of the benchmark
# ----------------------------------------------------------------------------------------------
def torch_reference_step(q, locations, keys, values, scale, cos, sin):
    """The reference's eager path restated with torch ops so it can use all host cores:
    tile q over fragments, rotate (attention.py:321-322 -> :84-90), then the concatenated-fragment
    masked softmax attention with fp32 upcast (attention.py:38-67).  Returns (out fp32, lse fp32)."""
    import torch
    F = cos.shape[0]
    rot = cos.shape[-1]
    qf = q.unsqueeze(0).expand(F, *q.shape)
    c = cos.unsqueeze(2)
    s = sin.unsqueeze(2)
    x_rot, x_pass = qf[..., :rot], qf[..., rot:]
    x1, x2 = x_rot[..., : rot // 2], x_rot[..., rot // 2:]
    rq = torch.cat((x_rot * c + torch.cat((-x2, x1), dim=-1) * s, x_pass), dim=-1).to(q.dtype)
    Hq = q.shape[1]
    qk, vals = [], []
    for f in range(F):
        kf = keys[f] if keys[f].dim() == 3 else keys[f][0]
        vf = values[f] if values[f].dim() == 3 else values[f][0]
        G = Hq // kf.shape[0]
        key = kf.repeat_interleave(G, 0)
        val = vf.repeat_interleave(G, 0)
        kp = torch.arange(key.shape[-2], dtype=torch.int32)[None, None, None, :]
        qp = locations[f][:, None, :, None]
        att = rq[f].to(torch.float32) @ key.transpose(-1, -2).to(torch.float32)
        att.masked_fill_(kp > qp, NEG_INF)
        qk.append(att)
        vals.append(val)
    qk = torch.cat(qk, dim=-1) * scale
    vals = torch.cat(vals, dim=-2).to(torch.float32)
    lse = torch.logsumexp(qk, dim=-1)
    out = torch.softmax(qk, dim=-1) @ vals
    return out, lse
