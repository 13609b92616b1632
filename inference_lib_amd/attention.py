"""Host-side mirror of the reference's operator wrappers (python/hogwild/attention.py:19-35, 70-74)
for the MI355X HIP library.  Same names, argument order and defaults; every function runs the HIP
kernels through the C ABI and raises if the library is not built — there is no eager fallback here.

When the torch operator binding (hogatt.abi3.so, namespace `libhogatt`) has been built it is loaded
and used, so that `torch.ops.libhogatt.hogwild_fused(...)` call sites keep working; otherwise the same
C entry points are called through ctypes.
"""
from __future__ import annotations

import os
from typing import List, Optional

import torch

from . import _lib

_HERE = os.path.dirname(os.path.abspath(__file__))
_TORCH_EXT = os.path.join(_HERE, "hogatt.abi3.so")
HAVE_TORCH_OPS = False
if os.path.exists(_TORCH_EXT):
    torch.ops.load_library(_TORCH_EXT)
    HAVE_TORCH_OPS = True


def hogwild_fused(queries: torch.Tensor, locations: torch.Tensor, keys: List[torch.Tensor], values: List[torch.Tensor],
                  scale: float, fragment_lengths, cosines: torch.Tensor, sines: torch.Tensor, *, rotated_queries, out,
                  lse: Optional[torch.Tensor] = None, device_lengths: bool = False):
    """rope + attention in one pass (python/hogwild/attention.py:19-23).  `fragment_lengths` is accepted
    for signature compatibility; the lengths are taken from the fragment tensors, which the reference
    requires to agree with it (src/kernels/kernel_v21.cuh:116-117).  `lse` (float32 [W,Hq,S]) is an
    addition: natural-log log-sum-exp of the scaled visible logits.  device_lengths (an addition as well): the
    fragment tensors give bounds and `fragment_lengths` (int32 [F] in device memory) the current lengths, fragment f
    having min(size, fragment_lengths[f]) tokens -- for launches captured in a graph while segments grow in place."""
    if device_lengths:
        if HAVE_TORCH_OPS and lse is None:
            torch.ops.libhogatt.hogwild_fused_devlen(out, rotated_queries, scale, locations, queries.contiguous(), fragment_lengths,
                                                     keys, values, cosines, sines)
            return out
        pr = _lib.Problem(q=queries.contiguous(), locations=locations, keys=keys, values=values, scale=scale, out=out,
                          cosines=cosines, sines=sines, rq=rotated_queries, lse=lse, len_dev=fragment_lengths)
        pr.run()
        return out
    if HAVE_TORCH_OPS and lse is None:
        torch.ops.libhogatt.hogwild_fused(out, rotated_queries, scale, locations, queries.contiguous(), fragment_lengths,
                                          keys, values, cosines, sines)
        return out
    if HAVE_TORCH_OPS:
        torch.ops.libhogatt.hogwild_fused_lse(out, rotated_queries, lse, scale, locations, queries.contiguous(),
                                              fragment_lengths, keys, values, cosines, sines)
        return out
    keys = [k.contiguous() for k in keys]        # the reference op copies non-contiguous fragments too, binding.cu:330-337
    values = [v.contiguous() for v in values]
    pr = _lib.Problem(q=queries.contiguous(), locations=locations, keys=keys, values=values, scale=scale, out=out,
                      cosines=cosines, sines=sines, rq=rotated_queries, lse=lse)
    pr.run()
    return out


def _in_place_or_contiguous(keys: List[torch.Tensor], values: List[torch.Tensor]):
    ks, vs = [], []
    for k, v in zip(keys, values):
        k3, v3 = (k[0] if k.dim() == 4 else k), (v[0] if v.dim() == 4 else v)
        if k3.dim() == 3 and v3.dim() == 3 and _lib.fragment_capacity(k3, v3) is not None:
            ks.append(k)
            vs.append(v)
        else:
            ks.append(k.contiguous())
            vs.append(v.contiguous())
    return ks, vs


def hogwild_sdpa(queries: torch.Tensor, locations: torch.Tensor, keys: List[torch.Tensor], values: List[torch.Tensor],
                 scale: float, fragment_lengths=None, out=None, lse: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Attention with already-rotated queries [F,W,Hq,S,E] (python/hogwild/attention.py:26-35)."""
    if out is None:
        out = torch.empty((queries.size(1), queries.size(2), queries.size(3), values[0].size(-1)), dtype=queries.dtype,
                          device=queries.device)
    # the reference wrapper makes every fragment contiguous (:32-33); a segment that grows in place inside a larger
    # allocation (rows contiguous, kv heads a whole number of rows apart) is read where it is instead of being copied
    keys, values = _in_place_or_contiguous(keys, values)
    if HAVE_TORCH_OPS:
        if fragment_lengths is None:
            fragment_lengths = torch.tensor([k.size(-2) for k in keys], dtype=torch.int32, device=queries.device)
        if lse is None:
            torch.ops.libhogatt.hogwild_sdpa(out, scale, locations, queries.contiguous(), fragment_lengths, keys, values)
        else:
            torch.ops.libhogatt.hogwild_sdpa_lse(out, lse, scale, locations, queries.contiguous(), fragment_lengths, keys, values)
        return out
    pr = _lib.Problem(q=queries.contiguous(), locations=locations, keys=keys, values=values, scale=scale, out=out, lse=lse,
                      prerotated=True)
    pr.run()
    return out


def hogwild_rope(queries: torch.Tensor, cosines: torch.Tensor, sines: torch.Tensor, out=None):
    """Per-fragment rotation of the queries (python/hogwild/attention.py:70-74)."""
    if out is None:
        out = torch.empty((cosines.size(0), queries.size(0), queries.size(1), queries.size(2), queries.size(3)),
                          dtype=queries.dtype, device=queries.device)
    if HAVE_TORCH_OPS:
        torch.ops.libhogatt.hogwild_rope(out, queries, cosines, sines)
        return out
    return _lib.rope(queries, cosines, sines, out)


def hogwild_paged_sdpa(queries: torch.Tensor, locations: torch.Tensor, fragment_lengths: torch.Tensor, key_cache: torch.Tensor,
                       value_cache: torch.Tensor, block_table: torch.Tensor, scale: float, out=None,
                       lse: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Attention of rotated queries [F,W,Hq,S,E] over paged sequences (operator `hogwild_paged_sdpa`,
    src/binding.cu:269-281; the reference has no Python wrapper for it).  `lse` (float32 [W,Hq,S]) is an addition and
    goes through the C ABI directly."""
    if out is None:
        out = torch.empty((queries.size(1), queries.size(2), queries.size(3), value_cache.size(-1)), dtype=queries.dtype,
                          device=queries.device)
    if HAVE_TORCH_OPS and lse is None:
        torch.ops.libhogatt.hogwild_paged_sdpa(out, scale, locations, queries.contiguous(), fragment_lengths, key_cache,
                                               value_cache, block_table)
        return out
    _lib.PagedProblem(q=queries.contiguous(), locations=locations, fragment_lengths=fragment_lengths, key_cache=key_cache,
                      value_cache=value_cache, block_table=block_table, scale=scale, out=out, lse=lse).run()
    return out


def hogwild_varlen_paged_sdpa(queries: torch.Tensor, locations: torch.Tensor, fragment_lengths: torch.Tensor,
                              key_cache: torch.Tensor, value_cache: torch.Tensor, block_table: torch.Tensor,
                              cu_seqlens_q: torch.Tensor, cu_seqlens_k: Optional[torch.Tensor], scale: float, out=None,
                              lse: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Packed variable-length form: queries [F,total_q,Hq,E], locations [F,total_q], fragment_lengths [F,W]
    (operator `hogwild_varlen_paged_sdpa`, src/binding.cu:283-296).  `cu_seqlens_k` is accepted and unused, as in the
    reference's kernel."""
    if out is None:
        out = torch.empty((queries.size(1), queries.size(2), value_cache.size(-1)), dtype=queries.dtype, device=queries.device)
    if HAVE_TORCH_OPS and lse is None:
        torch.ops.libhogatt.hogwild_varlen_paged_sdpa(out, scale, locations, queries.contiguous(), fragment_lengths, key_cache,
                                                      value_cache, block_table, cu_seqlens_q,
                                                      cu_seqlens_k if cu_seqlens_k is not None else cu_seqlens_q)
        return out
    _lib.PagedProblem(q=queries.contiguous(), locations=locations, fragment_lengths=fragment_lengths, key_cache=key_cache,
                      value_cache=value_cache, block_table=block_table, scale=scale, out=out, cu_seqlens_q=cu_seqlens_q,
                      lse=lse).run()
    return out


def copy_to_blocks(key_states: torch.Tensor, value_states: torch.Tensor, key_cache: torch.Tensor, value_cache: torch.Tensor,
                   block_table: torch.Tensor, seq_lengths: torch.Tensor) -> None:
    """Append new K/V rows [B,Hkv,S_new,D] to the paged caches at positions seq_lengths[b] + t (operator
    `copy_to_blocks`, src/binding.cu:310-322)."""
    if HAVE_TORCH_OPS:
        torch.ops.libhogatt.copy_to_blocks(key_states, value_states, key_cache, value_cache, block_table, seq_lengths)
        return
    _lib.copy_to_blocks(key_states, value_states, key_cache, value_cache, block_table, seq_lengths)
