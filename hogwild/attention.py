"""`hogwild.attention` as the reference ships it (python/hogwild/attention.py), served by the MI355X implementation.

The operator wrappers (`hogwild_fused` :19-23, `hogwild_sdpa` :26-35, `hogwild_rope` :70-74) keep their names, argument
order and defaults; loading this module loads `hogatt.abi3.so`, so `torch.ops.libhogatt.*` call sites work as well
(:12-16).  `CacheStructure`, `HogwildCache`, `merge_caches`, `AttentionModule` and `model_surgery` (:105-257, :263-354)
are the re-designed host-side objects of `inference_lib_amd.cache` / `.model`.  Not provided on purpose: the pure-torch
`hogwild_sdpa_pt` (:38-67) and a fallback to it when the library is missing -- without the built library this import
fails instead of degrading to an eager path.
"""
from inference_lib_amd.attention import (HAVE_TORCH_OPS, copy_to_blocks, hogwild_fused, hogwild_paged_sdpa, hogwild_rope,
                                         hogwild_sdpa, hogwild_varlen_paged_sdpa)
from inference_lib_amd.cache import CacheStructure, HogwildCache, SegmentCache, merge_caches
from inference_lib_amd.model import AttentionModule, decode_step, model_surgery

__all__ = ["hogwild_fused", "hogwild_sdpa", "hogwild_rope", "hogwild_paged_sdpa", "hogwild_varlen_paged_sdpa", "copy_to_blocks",
           "CacheStructure", "HogwildCache", "SegmentCache", "merge_caches", "AttentionModule", "model_surgery", "decode_step",
           "HAVE_TORCH_OPS"]
