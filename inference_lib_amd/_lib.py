"""ctypes view of the C ABI in include/hogwild_hip.h.

The library is required: importing this module without a built libhogwild_hip.so raises, and no entry
point here has a CPU or eager fallback.  Tensors are torch tensors on the GPU; only their pointers,
sizes and the current HIP stream cross the boundary.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import List, Optional, Sequence

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libhogwild_hip.so")

HW_MAX_FRAGMENTS = 512          # per call
HW_MAX_LAUNCH_FRAGMENTS = 64    # per attention launch (what hw_plan describes)
HW_ABI_VERSION = 6              # the version the structures below mirror
HW_MAX_SPLITS = 256
HW_STATIC_SCRATCH_BYTES = 8 << 20
HW_F32, HW_F16, HW_BF16 = 0, 1, 2
_DTYPE_CODE = {torch.float32: HW_F32, torch.float16: HW_F16, torch.bfloat16: HW_BF16}

EXPORTS = [
    "hw_version", "hw_status_string", "hw_validate", "hw_plan_debug", "hw_workspace_bytes",
    "hw_fused_attention", "hw_fused_attention_stages", "hw_sdpa", "hw_rope", "hw_device_cus",
    "hw_paged_validate", "hw_paged_plan_debug", "hw_paged_workspace_bytes", "hw_paged_sdpa", "hw_varlen_paged_sdpa",
    "hw_paged_sdpa_stages", "hw_copy_to_blocks", "hw_build_inputs", "hw_rope_append",
    "hw_build_inputs_dev", "hw_advance_lengths", "hw_fused_attention_static", "hw_sdpa_workspace_bytes",
]


class HwProblem(C.Structure):
    _fields_ = [
        ("dtype", C.c_int32),
        ("F", C.c_int32), ("W", C.c_int32), ("Hq", C.c_int32), ("Hkv", C.c_int32), ("S", C.c_int32),
        ("E", C.c_int32), ("Ev", C.c_int32), ("RotE", C.c_int32),
        ("scale", C.c_float),
        ("out", C.c_void_p), ("lse", C.c_void_p), ("rq", C.c_void_p),
        ("q", C.c_void_p), ("locations", C.c_void_p), ("cosines", C.c_void_p), ("sines", C.c_void_p),
        ("k", C.POINTER(C.c_void_p)), ("v", C.POINTER(C.c_void_p)), ("len", C.POINTER(C.c_int32)),
        ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t),
        ("splits", C.c_int32), ("row_blocks", C.c_int32),
        ("cap", C.POINTER(C.c_int32)),
        ("len_dev", C.c_void_p),
        ("variant", C.c_int32),
    ]


class HwPlan(C.Structure):
    _fields_ = [
        ("rows", C.c_int32), ("row_blocks", C.c_int32), ("row_groups", C.c_int32), ("tile_tokens", C.c_int32),
        ("tiles_per_head", C.c_int32), ("wgs_per_head", C.c_int32), ("workgroups", C.c_int32),
        ("tile_begin", C.c_int32 * (HW_MAX_LAUNCH_FRAGMENTS + 1)),
        ("wg_tile_begin", C.c_int32 * (HW_MAX_SPLITS + 1)),
        ("workspace_bytes", C.c_size_t),
    ]


class HwPagedProblem(C.Structure):
    _fields_ = [
        ("dtype", C.c_int32),
        ("F", C.c_int32), ("W", C.c_int32), ("Hq", C.c_int32), ("Hkv", C.c_int32), ("E", C.c_int32), ("Ev", C.c_int32),
        ("S", C.c_int32), ("total_q", C.c_int32),
        ("block_size", C.c_int32), ("max_blocks", C.c_int32), ("num_blocks", C.c_int32),
        ("scale", C.c_float),
        ("out", C.c_void_p), ("lse", C.c_void_p), ("q", C.c_void_p), ("locations", C.c_void_p),
        ("fragment_lengths", C.c_void_p), ("key_cache", C.c_void_p), ("value_cache", C.c_void_p),
        ("block_table", C.c_void_p), ("cu_seqlens_q", C.c_void_p),
        ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t),
        ("splits", C.c_int32), ("row_blocks", C.c_int32),
    ]


class HwPagedPlan(C.Structure):
    _fields_ = [
        ("rows", C.c_int32), ("row_blocks", C.c_int32), ("row_groups", C.c_int32), ("splits", C.c_int32),
        ("workgroups", C.c_int32), ("device_planned", C.c_int32), ("workspace_bytes", C.c_size_t),
    ]


class HwCopyBlocks(C.Structure):
    _fields_ = [
        ("dtype", C.c_int32),
        ("B", C.c_int32), ("Hkv", C.c_int32), ("S_new", C.c_int32), ("E", C.c_int32), ("Ev", C.c_int32),
        ("block_size", C.c_int32), ("max_blocks", C.c_int32), ("num_blocks", C.c_int32),
        ("key_states", C.c_void_p), ("value_states", C.c_void_p),
        ("ks_b", C.c_int64), ("ks_h", C.c_int64), ("ks_s", C.c_int64),
        ("vs_b", C.c_int64), ("vs_h", C.c_int64), ("vs_s", C.c_int64),
        ("key_cache", C.c_void_p), ("value_cache", C.c_void_p),
        ("block_table", C.c_void_p), ("seq_lengths", C.c_void_p),
    ]


class HwAppend(C.Structure):
    _fields_ = [
        ("dtype", C.c_int32), ("cs_dtype", C.c_int32), ("mode", C.c_int32),
        ("W", C.c_int32), ("Hkv", C.c_int32), ("S", C.c_int32), ("E", C.c_int32), ("Ev", C.c_int32), ("RotE", C.c_int32),
        ("key_states", C.c_void_p), ("value_states", C.c_void_p),
        ("ks_w", C.c_int64), ("ks_h", C.c_int64), ("ks_s", C.c_int64),
        ("vs_w", C.c_int64), ("vs_h", C.c_int64), ("vs_s", C.c_int64),
        ("cosines", C.c_void_p), ("sines", C.c_void_p),
        ("cs_w", C.c_int64), ("cs_s", C.c_int64),
        ("k_dst", C.POINTER(C.c_void_p)), ("v_dst", C.POINTER(C.c_void_p)),
        ("dst_len", C.POINTER(C.c_int32)), ("dst_cap", C.POINTER(C.c_int32)), ("n_new", C.POINTER(C.c_int32)),
        ("len_dev", C.c_void_p),
    ]


HW_ROPE_EAGER, HW_ROPE_FUSED = 0, 1
HW_VARIANT_MFMA, HW_VARIANT_VALU_QK = 0, 1


class HogwildError(RuntimeError):
    def __init__(self, status: int, where: str):
        self.status = status
        super().__init__(f"{where}: status {status}: {status_string(status)}")


def _load() -> C.CDLL:
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m inference_lib_amd.build` "
            "(there is no fallback path for the Hogwild attention operators)")
    lib = C.CDLL(LIB_PATH)
    lib.hw_version.restype = C.c_int
    if lib.hw_version() != HW_ABI_VERSION:      # a stale library would be driven with structures of another layout
        raise ImportError(f"{LIB_PATH} has ABI version {lib.hw_version()}, this module mirrors version {HW_ABI_VERSION}: "
                          "rebuild it with `python -m inference_lib_amd.build`")
    lib.hw_status_string.restype = C.c_char_p
    lib.hw_status_string.argtypes = [C.c_int]
    lib.hw_validate.argtypes = [C.POINTER(HwProblem), C.c_int]
    lib.hw_plan_debug.argtypes = [C.POINTER(HwProblem), C.c_int, C.POINTER(HwPlan)]
    lib.hw_workspace_bytes.argtypes = [C.POINTER(HwProblem), C.POINTER(C.c_size_t)]
    lib.hw_sdpa_workspace_bytes.argtypes = [C.POINTER(HwProblem), C.POINTER(C.c_size_t)]
    lib.hw_fused_attention.argtypes = [C.POINTER(HwProblem), C.c_void_p]
    lib.hw_sdpa.argtypes = [C.POINTER(HwProblem), C.c_void_p]
    lib.hw_fused_attention_static.argtypes = [C.POINTER(HwProblem), C.c_void_p]
    lib.hw_fused_attention_stages.argtypes = [C.POINTER(HwProblem), C.c_void_p, C.c_int]
    lib.hw_rope.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int,
                            C.c_int, C.c_int, C.c_int, C.c_void_p]
    lib.hw_paged_validate.argtypes = [C.POINTER(HwPagedProblem)]
    lib.hw_paged_plan_debug.argtypes = [C.POINTER(HwPagedProblem), C.c_int, C.POINTER(HwPagedPlan)]
    lib.hw_paged_workspace_bytes.argtypes = [C.POINTER(HwPagedProblem), C.POINTER(C.c_size_t)]
    lib.hw_paged_sdpa.argtypes = [C.POINTER(HwPagedProblem), C.c_void_p]
    lib.hw_varlen_paged_sdpa.argtypes = [C.POINTER(HwPagedProblem), C.c_void_p]
    lib.hw_paged_sdpa_stages.argtypes = [C.POINTER(HwPagedProblem), C.c_void_p, C.c_int]
    lib.hw_copy_to_blocks.argtypes = [C.POINTER(HwCopyBlocks), C.c_void_p]
    lib.hw_build_inputs.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(C.c_int32), C.c_void_p, C.c_float, C.c_int,
                                    C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p]
    lib.hw_rope_append.argtypes = [C.POINTER(HwAppend), C.c_void_p]
    lib.hw_build_inputs_dev.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(C.c_int32), C.c_void_p, C.c_float,
                                        C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p]
    lib.hw_advance_lengths.argtypes = [C.c_void_p, C.POINTER(C.c_int32), C.c_int, C.c_void_p]
    return lib


lib = _load()


def status_string(status: int) -> str:
    return lib.hw_status_string(int(status)).decode()


def check(status: int, where: str) -> None:
    if status != 0:
        raise HogwildError(status, where)


def fragment_capacity(k: torch.Tensor, v: torch.Tensor) -> Optional[int]:
    """Row capacity of a fragment whose tensors [Hkv, L, D] are views into [Hkv, cap, D] allocations (rows contiguous,
    kv heads `cap` rows apart), or None if the pair is not of that form.  Packed fragments give cap == L."""
    Hkv, L, E = k.shape
    Ev = v.size(2)
    if L == 0:
        return 0
    if (E > 1 and k.stride(2) != 1) or (Ev > 1 and v.stride(2) != 1) or (L > 1 and (k.stride(1) != E or v.stride(1) != Ev)):
        return None
    if Hkv == 1:
        return L
    if k.stride(0) % E != 0 or v.stride(0) % Ev != 0 or k.stride(0) // E != v.stride(0) // Ev or k.stride(0) // E < L:
        return None
    return k.stride(0) // E


def _frag3(t: torch.Tensor) -> torch.Tensor:
    """Fragments come as [Hkv, L, D] or [1, Hkv, L, D] (src/binding.cu:85-94)."""
    if t.dim() == 4:
        if t.size(0) != 1:
            raise ValueError("4-D KV fragment must have a leading dimension of 1")
        return t[0]
    if t.dim() != 3:
        raise ValueError("KV fragment must be [Hkv, L, D] or [1, Hkv, L, D]")
    return t


class Problem:
    """Owns the ctypes arrays of one hw_problem and keeps the tensors alive."""

    def __init__(self, *, q: torch.Tensor, locations: torch.Tensor, keys: Sequence[torch.Tensor],
                 values: Sequence[torch.Tensor], scale: float, out: torch.Tensor,
                 cosines: Optional[torch.Tensor] = None, sines: Optional[torch.Tensor] = None,
                 rq: Optional[torch.Tensor] = None, lse: Optional[torch.Tensor] = None,
                 prerotated: bool = False, splits: int = 0, row_blocks: int = 0, len_dev: Optional[torch.Tensor] = None,
                 variant: int = 0):
        keys = [_frag3(k) for k in keys]
        values = [_frag3(v) for v in values]
        F = len(keys)
        if len(values) != F or locations.size(0) != F:
            raise ValueError("fragment count mismatch between keys, values and locations")
        if F < 1 or F > HW_MAX_FRAGMENTS:
            raise HogwildError(-5, "Problem")
        W, Hq, S, Ev = out.shape
        E = q.size(-1)
        Hkv = keys[0].size(0)
        if out.dtype not in _DTYPE_CODE:
            raise HogwildError(-2, "Problem")
        expect_q = (F, W, Hq, S, E) if prerotated else (W, Hq, S, E)
        if tuple(q.shape) != expect_q:
            raise ValueError(f"queries have shape {tuple(q.shape)}, expected {expect_q}")
        if tuple(locations.shape) != (F, W, S) or locations.dtype != torch.int32:
            raise ValueError("locations must be int32 [F, W, S]")
        tensors = [out, q, locations]
        caps = []
        for f in range(F):
            if keys[f].size(0) != Hkv or values[f].size(0) != Hkv or keys[f].size(1) != values[f].size(1) \
                    or keys[f].size(2) != E or values[f].size(2) != Ev:
                raise ValueError(f"fragment {f} has inconsistent shape")
            if keys[f].dtype != out.dtype or values[f].dtype != out.dtype:
                raise ValueError("KV fragments must have the dtype of the output")
            cap = fragment_capacity(keys[f], values[f])
            if cap is None:
                raise ValueError(f"fragment {f}: rows must be contiguous and kv heads a whole number of rows apart "
                                 "(the same number for keys and values)")
            caps.append(cap)
            if keys[f].device != out.device or values[f].device != out.device:
                raise ValueError("all tensors must live on the output's device")
        if q.dtype != out.dtype:
            raise ValueError("queries must have the dtype of the output")
        rot = 0
        if not prerotated:
            if cosines is None or sines is None:
                raise ValueError("the fused operator needs cosines and sines")
            rot = cosines.size(-1)
            if tuple(cosines.shape) != (F, W, S, rot) or tuple(sines.shape) != (F, W, S, rot):
                raise ValueError("cosines / sines must be [F, W, S, RotE]")
            if cosines.dtype != torch.float32 or sines.dtype != torch.float32:
                raise ValueError("cosines / sines must be float32")
            tensors += [cosines, sines]
        if rq is not None:
            if tuple(rq.shape) != (F, W, Hq, S, E) or rq.dtype != out.dtype:
                raise ValueError("rotated-query buffer must be [F, W, Hq, S, E] in the output dtype")
            tensors.append(rq)
        if lse is not None:
            if tuple(lse.shape) != (W, Hq, S) or lse.dtype != torch.float32:
                raise ValueError("lse must be float32 [W, Hq, S]")
            tensors.append(lse)
        if len_dev is not None:      # current lengths in device memory; the fragment tensors then give the planned bounds
            if len_dev.dtype != torch.int32 or tuple(len_dev.shape) != (F,):
                raise ValueError("len_dev must be int32 [F]")
            tensors.append(len_dev)
        for t in tensors:
            if not t.is_contiguous():
                raise ValueError("all tensors must be contiguous")
            if t.device != out.device:
                raise ValueError("all tensors must live on the output's device")
        self._keep = tensors + keys + values
        self.device = out.device
        self._cap = (C.c_int32 * F)(*caps)
        self._k = (C.c_void_p * F)(*[k.data_ptr() for k in keys])
        self._v = (C.c_void_p * F)(*[v.data_ptr() for v in values])
        self._len = (C.c_int32 * F)(*[k.size(1) for k in keys])
        p = HwProblem()
        p.dtype = _DTYPE_CODE[out.dtype]
        p.F, p.W, p.Hq, p.Hkv, p.S, p.E, p.Ev, p.RotE = F, W, Hq, Hkv, S, E, Ev, rot
        p.scale = float(scale)
        p.out = out.data_ptr()
        p.lse = lse.data_ptr() if lse is not None else None
        p.rq = rq.data_ptr() if rq is not None else None
        p.q = q.data_ptr()
        p.locations = locations.data_ptr()
        p.cosines = cosines.data_ptr() if cosines is not None else None
        p.sines = sines.data_ptr() if sines is not None else None
        p.k = C.cast(self._k, C.POINTER(C.c_void_p))
        p.v = C.cast(self._v, C.POINTER(C.c_void_p))
        p.len = C.cast(self._len, C.POINTER(C.c_int32))
        p.cap = C.cast(self._cap, C.POINTER(C.c_int32))
        p.len_dev = len_dev.data_ptr() if len_dev is not None else None
        p.splits = int(splits)
        p.row_blocks = int(row_blocks)
        p.variant = int(variant)      # 0 = matrix cores; 1 = logits by VALU dot products (HW_VARIANT_VALU_QK, for A/B measurements)
        self.p = p
        self.prerotated = prerotated
        self._ws = None

    def workspace_bytes(self) -> int:
        n = C.c_size_t(0)
        with torch.cuda.device(self.device):
            fn = lib.hw_sdpa_workspace_bytes if self.prerotated else lib.hw_workspace_bytes
            check(fn(C.byref(self.p), C.byref(n)), fn.__name__)
        return n.value

    def set_workspace(self, ws: Optional[torch.Tensor] = None) -> None:
        if ws is None:
            ws = torch.empty(self.workspace_bytes(), dtype=torch.uint8, device=self.device)
        self._ws = ws
        self.p.workspace = ws.data_ptr()
        self.p.workspace_bytes = ws.numel() * ws.element_size()

    def run(self, stages: int = 3) -> None:
        """stages: 1 = attention kernel only (partials stay in the workspace), 2 = merge only, 3 = both."""
        if self._ws is None:
            self.set_workspace()
        with torch.cuda.device(self.device):
            stream = torch.cuda.current_stream(self.device).cuda_stream
            if stages != 3:
                if self.prerotated:
                    raise ValueError("separate stages exist for the fused entry only")
                check(lib.hw_fused_attention_stages(C.byref(self.p), C.c_void_p(stream), stages), "hw_fused_attention_stages")
                return
            fn = lib.hw_sdpa if self.prerotated else lib.hw_fused_attention
            check(fn(C.byref(self.p), C.c_void_p(stream)), fn.__name__)


    def run_static(self) -> None:
        """hw_fused_attention_static: the same step with the partials in the library's own device array; allocates nothing."""
        if self.prerotated:
            raise ValueError("the static-scratch entry exists for the fused operator only")
        with torch.cuda.device(self.device):
            stream = torch.cuda.current_stream(self.device).cuda_stream
            check(lib.hw_fused_attention_static(C.byref(self.p), C.c_void_p(stream)), "hw_fused_attention_static")


def plan(lens: Sequence[int], *, W: int, S: int, Hq: int, Hkv: int, Ev: int, num_cus: int, splits: int = 0,
         dtype: int = HW_BF16, row_blocks: int = 0) -> HwPlan:
    """Host-only split plan (no GPU needed)."""
    F = len(lens)
    arr = (C.c_int32 * max(F, 1))(*lens)
    p = HwProblem()
    p.F, p.W, p.S, p.Hq, p.Hkv, p.Ev, p.E = F, W, S, Hq, Hkv, Ev, Ev
    p.len = C.cast(arr, C.POINTER(C.c_int32))
    p.splits = splits
    p.dtype = dtype
    p.row_blocks = row_blocks
    out = HwPlan()
    check(lib.hw_plan_debug(C.byref(p), num_cus, C.byref(out)), "hw_plan_debug")
    return out


class PagedProblem:
    """One call of the paged attention operators (hw_paged_sdpa, or hw_varlen_paged_sdpa when cu_seqlens_q is given).

    fixed length:    q [F, W, Hq, S, E], locations [F, W, S], fragment_lengths [F], out [W, Hq, S, Ev], lse [W, Hq, S]
    variable length: q [F, T, Hq, E], locations [F, T], fragment_lengths [F, W], cu_seqlens_q [W+1], out [T, Hq, Ev],
                     lse [T, Hq]
    key_cache / value_cache [num_blocks, Hkv, block_size, E|Ev], block_table int32 [W, max_blocks].
    """

    def __init__(self, *, q: torch.Tensor, locations: torch.Tensor, fragment_lengths: torch.Tensor,
                 key_cache: torch.Tensor, value_cache: torch.Tensor, block_table: torch.Tensor, scale: float,
                 out: torch.Tensor, cu_seqlens_q: Optional[torch.Tensor] = None, lse: Optional[torch.Tensor] = None,
                 splits: int = 0, row_blocks: int = 0):
        varlen = cu_seqlens_q is not None
        if out.dtype not in _DTYPE_CODE:
            raise HogwildError(-2, "PagedProblem")
        if key_cache.dim() != 4 or value_cache.dim() != 4 or key_cache.shape[:3] != value_cache.shape[:3]:
            raise ValueError("key_cache / value_cache must be [num_blocks, Hkv, block_size, E|Ev]")
        NB, Hkv, BS, E = key_cache.shape
        Ev = value_cache.size(3)
        if block_table.dim() != 2:
            raise ValueError("block_table must be [W, max_blocks]")
        W = block_table.size(0)
        F = locations.size(0)
        if varlen:
            T, Hq = out.size(0), out.size(1)
            S = 0
            if tuple(out.shape) != (T, Hq, Ev) or tuple(q.shape) != (F, T, Hq, E) or tuple(locations.shape) != (F, T):
                raise ValueError("variable-length layout: q [F,T,Hq,E], locations [F,T], out [T,Hq,Ev]")
            if tuple(fragment_lengths.shape) != (F, W) or tuple(cu_seqlens_q.shape) != (W + 1,):
                raise ValueError("variable-length layout: fragment_lengths [F,W], cu_seqlens_q [W+1]")
            lse_shape = (T, Hq)
        else:
            if out.dim() != 4 or out.size(0) != W:
                raise ValueError("out must be [W, Hq, S, Ev] with one block-table row per worker")
            _, Hq, S, _ = out.shape
            T = 0
            if tuple(out.shape) != (W, Hq, S, Ev) or tuple(q.shape) != (F, W, Hq, S, E) or tuple(locations.shape) != (F, W, S):
                raise ValueError("fixed-length layout: q [F,W,Hq,S,E], locations [F,W,S], out [W,Hq,S,Ev]")
            if tuple(fragment_lengths.shape) != (F,):
                raise ValueError("fixed-length layout: fragment_lengths [F]")
            lse_shape = (W, Hq, S)
        tensors = [out, q, locations, fragment_lengths, key_cache, value_cache, block_table]
        if varlen:
            tensors.append(cu_seqlens_q)
        if lse is not None:
            if tuple(lse.shape) != lse_shape or lse.dtype != torch.float32:
                raise ValueError(f"lse must be float32 {lse_shape}")
            tensors.append(lse)
        for t in (locations, fragment_lengths, block_table) + ((cu_seqlens_q,) if varlen else ()):
            if t.dtype != torch.int32:
                raise ValueError("locations, fragment_lengths, block_table and cu_seqlens_q must be int32")
        for t in (q, key_cache, value_cache):
            if t.dtype != out.dtype:
                raise ValueError("queries and caches must have the dtype of the output")
        for t in tensors:
            if not t.is_contiguous():
                raise ValueError("all tensors must be contiguous")
            if t.device != out.device:
                raise ValueError("all tensors must live on the output's device")
        self._keep = tensors
        self.device = out.device
        p = HwPagedProblem()
        p.dtype = _DTYPE_CODE[out.dtype]
        p.F, p.W, p.Hq, p.Hkv, p.E, p.Ev, p.S, p.total_q = F, W, Hq, Hkv, E, Ev, S, T
        p.block_size, p.max_blocks, p.num_blocks = BS, block_table.size(1), NB
        p.scale = float(scale)
        p.out = out.data_ptr()
        p.lse = lse.data_ptr() if lse is not None else None
        p.q = q.data_ptr()
        p.locations = locations.data_ptr()
        p.fragment_lengths = fragment_lengths.data_ptr()
        p.key_cache = key_cache.data_ptr()
        p.value_cache = value_cache.data_ptr()
        p.block_table = block_table.data_ptr()
        p.cu_seqlens_q = cu_seqlens_q.data_ptr() if varlen else None
        p.splits = int(splits)
        p.row_blocks = int(row_blocks)
        self.p = p
        self.varlen = varlen
        self._ws = None

    def workspace_bytes(self) -> int:
        n = C.c_size_t(0)
        with torch.cuda.device(self.device):
            check(lib.hw_paged_workspace_bytes(C.byref(self.p), C.byref(n)), "hw_paged_workspace_bytes")
        return n.value

    def set_workspace(self, ws: Optional[torch.Tensor] = None) -> None:
        if ws is None:
            ws = torch.empty(max(self.workspace_bytes(), 256), dtype=torch.uint8, device=self.device)
        self._ws = ws
        self.p.workspace = ws.data_ptr()
        self.p.workspace_bytes = ws.numel() * ws.element_size()

    def run(self, stages: int = 3) -> None:
        if self._ws is None:
            self.set_workspace()
        with torch.cuda.device(self.device):
            stream = torch.cuda.current_stream(self.device).cuda_stream
            if stages != 3:
                check(lib.hw_paged_sdpa_stages(C.byref(self.p), C.c_void_p(stream), stages), "hw_paged_sdpa_stages")
                return
            fn = lib.hw_varlen_paged_sdpa if self.varlen else lib.hw_paged_sdpa
            check(fn(C.byref(self.p), C.c_void_p(stream)), fn.__name__)


def paged_plan(*, W: int, Hq: int, Hkv: int, Ev: int, block_size: int, max_blocks: int, num_cus: int, S: int = 0,
               total_q: Optional[int] = None, splits: int = 0, dtype: int = HW_BF16, row_blocks: int = 0) -> HwPagedPlan:
    """Host-only plan of the paged operators (no GPU needed); total_q selects the variable-length operator."""
    p = HwPagedProblem()
    p.dtype = dtype
    p.F, p.W, p.Hq, p.Hkv, p.E, p.Ev, p.S = 1, W, Hq, Hkv, Ev, Ev, S
    p.block_size, p.max_blocks, p.num_blocks = block_size, max_blocks, 1
    if total_q is not None:
        p.total_q = total_q
        p.cu_seqlens_q = 16       # only tested for being non-NULL by the planner
    p.splits = splits
    p.row_blocks = row_blocks
    out = HwPagedPlan()
    check(lib.hw_paged_plan_debug(C.byref(p), num_cus, C.byref(out)), "hw_paged_plan_debug")
    return out


def copy_to_blocks(key_states: torch.Tensor, value_states: torch.Tensor, key_cache: torch.Tensor, value_cache: torch.Tensor,
                   block_table: torch.Tensor, seq_lengths: torch.Tensor) -> None:
    """Append key_states / value_states [B, Hkv, S_new, E|Ev] (any strides with a contiguous last dimension) to the
    paged caches at positions seq_lengths[b] + t."""
    if key_states.dim() != 4 or value_states.dim() != 4 or key_states.shape[:3] != value_states.shape[:3]:
        raise ValueError("key_states / value_states must be [B, Hkv, S_new, E|Ev]")
    B, Hkv, S_new, E = key_states.shape
    Ev = value_states.size(3)
    if key_cache.dim() != 4 or value_cache.dim() != 4 or key_cache.size(1) != Hkv or key_cache.size(3) != E \
            or value_cache.size(3) != Ev or key_cache.shape[:3] != value_cache.shape[:3]:
        raise ValueError("caches must be [num_blocks, Hkv, block_size, E|Ev]")
    if key_states.dtype not in _DTYPE_CODE:
        raise HogwildError(-2, "copy_to_blocks")
    for t in (value_states, key_cache, value_cache):
        if t.dtype != key_states.dtype:
            raise ValueError("states and caches must share one dtype")
    if tuple(seq_lengths.shape) != (B,) or block_table.dim() != 2 or block_table.size(0) != B:
        raise ValueError("block_table must be [B, max_blocks], seq_lengths [B]")
    for t in (block_table, seq_lengths):
        if t.dtype != torch.int32 or not t.is_contiguous():
            raise ValueError("block_table and seq_lengths must be contiguous int32")
    if not key_cache.is_contiguous() or not value_cache.is_contiguous():
        raise ValueError("caches must be contiguous")
    if (E > 1 and key_states.stride(3) != 1) or (Ev > 1 and value_states.stride(3) != 1):
        key_states, value_states = key_states.contiguous(), value_states.contiguous()
    for t in (key_states, value_states, value_cache, block_table, seq_lengths):
        if t.device != key_cache.device:
            raise ValueError("all tensors must live on the caches' device")
    c = HwCopyBlocks()
    c.dtype = _DTYPE_CODE[key_states.dtype]
    c.B, c.Hkv, c.S_new, c.E, c.Ev = B, Hkv, S_new, E, Ev
    c.block_size, c.max_blocks, c.num_blocks = key_cache.size(2), block_table.size(1), key_cache.size(0)
    c.key_states, c.value_states = key_states.data_ptr(), value_states.data_ptr()
    c.ks_b, c.ks_h, c.ks_s = key_states.stride(0), key_states.stride(1), key_states.stride(2)
    c.vs_b, c.vs_h, c.vs_s = value_states.stride(0), value_states.stride(1), value_states.stride(2)
    c.key_cache, c.value_cache = key_cache.data_ptr(), value_cache.data_ptr()
    c.block_table, c.seq_lengths = block_table.data_ptr(), seq_lengths.data_ptr()
    with torch.cuda.device(key_cache.device):
        stream = torch.cuda.current_stream(key_cache.device).cuda_stream
        check(lib.hw_copy_to_blocks(C.byref(c), C.c_void_p(stream)), "hw_copy_to_blocks")


def build_inputs(pos_end: Sequence[Sequence[int]], S: int, inv_freq: Optional[torch.Tensor], *, attention_scaling: float = 1.0,
                 table_dtype: Optional[torch.dtype] = None, device=None):
    """locations int32 [F, W, S], cosines / sines float32 [F, W, S, RotE] of a decode step.  pos_end[f][w] = position one
    past the newest token of worker w as seen through fragment f (host numbers).  table_dtype = dtype the tables are
    rounded to before being stored as float32 (None / float32: no rounding)."""
    F, W = len(pos_end), len(pos_end[0])
    flat = [int(x) for row in pos_end for x in row]
    if len(flat) != F * W:
        raise ValueError("pos_end must be a full [F][W] table")
    rot = 0 if inv_freq is None else 2 * inv_freq.numel()
    if inv_freq is not None:
        if inv_freq.dtype != torch.float32 or not inv_freq.is_contiguous():
            raise ValueError("inv_freq must be contiguous float32 [RotE/2]")
        device = inv_freq.device
    if device is None:
        raise ValueError("a device is needed when there is no inv_freq tensor")
    device = torch.device(device)
    loc = torch.empty((F, W, S), dtype=torch.int32, device=device)
    cos = torch.empty((F, W, S, rot), dtype=torch.float32, device=device)
    sin = torch.empty((F, W, S, rot), dtype=torch.float32, device=device)
    arr = (C.c_int32 * (F * W))(*flat)
    rd = HW_F32 if table_dtype is None else _DTYPE_CODE[table_dtype]
    with torch.cuda.device(device):
        stream = torch.cuda.current_stream(device).cuda_stream
        check(lib.hw_build_inputs(loc.data_ptr(), cos.data_ptr(), sin.data_ptr(), arr,
                                  inv_freq.data_ptr() if inv_freq is not None else None, float(attention_scaling), rd,
                                  F, W, S, rot, C.c_void_p(stream)), "hw_build_inputs")
    return loc, cos, sin


def build_inputs_dev(len_dev: torch.Tensor, orders: Sequence[Sequence[int]], S: int, inv_freq: Optional[torch.Tensor], *,
                     attention_scaling: float = 1.0, table_dtype: Optional[torch.dtype] = None, out=None):
    """build_inputs with the fragment lengths in device memory: len_dev int32 [F] (lengths including this step's new
    tokens), orders[w] = the fragments in worker w's order.  out = (locations, cosines, sines) to write into (so that a
    captured graph keeps its addresses), else fresh tensors."""
    F, W = len_dev.numel(), len(orders)
    flat = [int(x) for row in orders for x in row]
    if len(flat) != F * W:
        raise ValueError("every worker's order must list all F fragments")
    if len_dev.dtype != torch.int32 or not len_dev.is_contiguous():
        raise ValueError("len_dev must be contiguous int32 [F]")
    device = len_dev.device
    rot = 0 if inv_freq is None else 2 * inv_freq.numel()
    if inv_freq is not None and (inv_freq.dtype != torch.float32 or not inv_freq.is_contiguous() or inv_freq.device != device):
        raise ValueError("inv_freq must be contiguous float32 [RotE/2] on the device of len_dev")
    if out is None:
        out = (torch.empty((F, W, S), dtype=torch.int32, device=device), torch.empty((F, W, S, rot), dtype=torch.float32, device=device),
               torch.empty((F, W, S, rot), dtype=torch.float32, device=device))
    loc, cos, sin = out
    if tuple(loc.shape) != (F, W, S) or loc.dtype != torch.int32 or tuple(cos.shape) != (F, W, S, rot) or tuple(sin.shape) != (F, W, S, rot) \
            or cos.dtype != torch.float32 or sin.dtype != torch.float32 or not (loc.is_contiguous() and cos.is_contiguous() and sin.is_contiguous()):
        raise ValueError("out must be (int32 [F, W, S], float32 [F, W, S, RotE], float32 [F, W, S, RotE]), contiguous")
    arr = (C.c_int32 * (F * W))(*flat)
    rd = HW_F32 if table_dtype is None else _DTYPE_CODE[table_dtype]
    with torch.cuda.device(device):
        stream = torch.cuda.current_stream(device).cuda_stream
        check(lib.hw_build_inputs_dev(loc.data_ptr(), cos.data_ptr(), sin.data_ptr(), len_dev.data_ptr(), arr,
                                      inv_freq.data_ptr() if inv_freq is not None else None, float(attention_scaling), rd,
                                      F, W, S, rot, C.c_void_p(stream)), "hw_build_inputs_dev")
    return loc, cos, sin


def advance_lengths(len_dev: torch.Tensor, add: Sequence[int]) -> None:
    """len_dev[f] += add[f] on the device (add: host numbers)."""
    F = len_dev.numel()
    if len_dev.dtype != torch.int32 or not len_dev.is_contiguous() or len(add) != F:
        raise ValueError("len_dev must be contiguous int32 [F] and add one number per entry")
    arr = (C.c_int32 * F)(*[int(x) for x in add])
    with torch.cuda.device(len_dev.device):
        stream = torch.cuda.current_stream(len_dev.device).cuda_stream
        check(lib.hw_advance_lengths(len_dev.data_ptr(), arr, F, C.c_void_p(stream)), "hw_advance_lengths")


def rope_append(key_states: torch.Tensor, value_states: torch.Tensor, k_dst: Sequence[torch.Tensor], v_dst: Sequence[torch.Tensor],
                dst_len: Sequence[int], *, cosines: Optional[torch.Tensor] = None, sines: Optional[torch.Tensor] = None,
                n_new: Optional[Sequence[int]] = None, mode: int = HW_ROPE_EAGER, len_dev: Optional[torch.Tensor] = None) -> None:
    """Rotate key_states [W, Hkv, S, E] with cosines / sines [W, S, RotE] (or [W, 1, RotE]: one row for all tokens) and
    append keys and value_states [W, Hkv, S, Ev] to the segment buffers k_dst[w] / v_dst[w] ([Hkv, cap, E|Ev], contiguous)
    behind their first dst_len[w] rows.  Without cosines the keys are appended as they are.  n_new[w] < S appends only
    the last n_new[w] tokens of worker w.  With len_dev (int32 device tensor of segment lengths) dst_len[w] is an index
    into it and len_dev[dst_len[w]] the length of worker w's segment after this append."""
    if key_states.dim() != 4 or value_states.dim() != 4 or key_states.shape[:3] != value_states.shape[:3]:
        raise ValueError("key_states / value_states must be [W, Hkv, S, E|Ev]")
    W, Hkv, S, E = key_states.shape
    Ev = value_states.size(3)
    if key_states.dtype not in _DTYPE_CODE or value_states.dtype != key_states.dtype:
        raise HogwildError(-2, "rope_append")
    if (E > 1 and key_states.stride(3) != 1) or (Ev > 1 and value_states.stride(3) != 1):
        key_states, value_states = key_states.contiguous(), value_states.contiguous()
    if len(k_dst) != W or len(v_dst) != W or len(dst_len) != W:
        raise ValueError("one destination segment and length per worker")
    for kd, vd in zip(k_dst, v_dst):
        if kd.dim() != 3 or vd.dim() != 3 or kd.size(0) != Hkv or vd.size(0) != Hkv or kd.size(2) != E or vd.size(2) != Ev \
                or kd.size(1) != vd.size(1) or not kd.is_contiguous() or not vd.is_contiguous():
            raise ValueError("segment buffers must be contiguous [Hkv, cap, E|Ev] with one capacity for keys and values")
        if kd.dtype != key_states.dtype or vd.dtype != key_states.dtype or kd.device != key_states.device:
            raise ValueError("segment buffers must have the dtype and device of the new states")
    a = HwAppend()
    a.dtype = _DTYPE_CODE[key_states.dtype]
    a.mode = int(mode)
    a.W, a.Hkv, a.S, a.E, a.Ev = W, Hkv, S, E, Ev
    a.key_states, a.value_states = key_states.data_ptr(), value_states.data_ptr()
    a.ks_w, a.ks_h, a.ks_s = key_states.stride(0), key_states.stride(1), key_states.stride(2)
    a.vs_w, a.vs_h, a.vs_s = value_states.stride(0), value_states.stride(1), value_states.stride(2)
    a.cs_dtype = HW_F32
    keep = [key_states, value_states]
    if cosines is not None:
        if sines is None or cosines.shape != sines.shape or cosines.dim() != 3 or cosines.size(0) != W or cosines.size(1) not in (1, S):
            raise ValueError("cosines / sines must be [W, S, RotE] or [W, 1, RotE]")
        if cosines.dtype != sines.dtype or cosines.dtype not in (torch.float32, key_states.dtype):
            raise ValueError("cosines / sines must be float32 or have the dtype of the keys")
        cosines, sines = cosines.contiguous(), sines.contiguous()
        a.RotE = cosines.size(2)
        a.cs_dtype = _DTYPE_CODE[cosines.dtype]
        a.cosines, a.sines = cosines.data_ptr(), sines.data_ptr()
        a.cs_w = cosines.stride(0)
        a.cs_s = 0 if cosines.size(1) == 1 else cosines.stride(1)
        keep += [cosines, sines]
    kp = (C.c_void_p * W)(*[t.data_ptr() for t in k_dst])
    vp = (C.c_void_p * W)(*[t.data_ptr() for t in v_dst])
    ln = (C.c_int32 * W)(*[int(x) for x in dst_len])
    cp = (C.c_int32 * W)(*[t.size(1) for t in k_dst])
    nn = (C.c_int32 * W)(*([S] * W if n_new is None else [int(x) for x in n_new]))
    a.k_dst, a.v_dst = C.cast(kp, C.POINTER(C.c_void_p)), C.cast(vp, C.POINTER(C.c_void_p))
    a.dst_len, a.dst_cap, a.n_new = C.cast(ln, C.POINTER(C.c_int32)), C.cast(cp, C.POINTER(C.c_int32)), C.cast(nn, C.POINTER(C.c_int32))
    if len_dev is not None:
        if len_dev.dtype != torch.int32 or len_dev.dim() != 1 or not len_dev.is_contiguous() or len_dev.device != key_states.device:
            raise ValueError("len_dev must be a contiguous int32 vector on the device of the new states")
        if any(int(x) < 0 or int(x) >= len_dev.numel() for x in dst_len):
            raise ValueError("with len_dev, dst_len holds indices into it")
        a.len_dev = len_dev.data_ptr()
    with torch.cuda.device(key_states.device):
        stream = torch.cuda.current_stream(key_states.device).cuda_stream
        check(lib.hw_rope_append(C.byref(a), C.c_void_p(stream)), "hw_rope_append")


class AppendPlan:
    """hw_rope_append with everything that stays the same from step to step prepared once: destination buffers,
    capacities, tokens per worker, and the segment lengths in device memory.  run() fills in the new states and their
    rotary tables and launches; it checks only what can change between calls."""

    def __init__(self, k_dst: Sequence[torch.Tensor], v_dst: Sequence[torch.Tensor], seg_index: Sequence[int], n_new: Sequence[int],
                 len_dev: torch.Tensor, mode: int = HW_ROPE_EAGER):
        W = len(k_dst)
        if len(v_dst) != W or len(seg_index) != W or len(n_new) != W:
            raise ValueError("one destination segment, length index and token count per worker")
        kd0 = k_dst[0]
        for kd, vd in zip(k_dst, v_dst):
            if kd.dim() != 3 or vd.dim() != 3 or kd.shape[:2] != vd.shape[:2] or not kd.is_contiguous() or not vd.is_contiguous() \
                    or kd.size(0) != kd0.size(0) or kd.size(2) != kd0.size(2) or vd.size(2) != v_dst[0].size(2) \
                    or kd.dtype != kd0.dtype or vd.dtype != kd0.dtype or kd.device != kd0.device:
                raise ValueError("segment buffers must be contiguous [Hkv, cap, E|Ev] of one dtype on one device")
        if len_dev.dtype != torch.int32 or len_dev.dim() != 1 or not len_dev.is_contiguous() or len_dev.device != kd0.device:
            raise ValueError("len_dev must be a contiguous int32 vector on the device of the segments")
        if any(int(x) < 0 or int(x) >= len_dev.numel() for x in seg_index):
            raise ValueError("seg_index holds indices into len_dev")
        self.W, self.Hkv, self.E, self.Ev = W, kd0.size(0), kd0.size(2), v_dst[0].size(2)
        self.dtype, self.device = kd0.dtype, kd0.device
        self._keep = (list(k_dst), list(v_dst), len_dev)
        self._kp = (C.c_void_p * W)(*[t.data_ptr() for t in k_dst])
        self._vp = (C.c_void_p * W)(*[t.data_ptr() for t in v_dst])
        self._ln = (C.c_int32 * W)(*[int(x) for x in seg_index])
        self._cp = (C.c_int32 * W)(*[t.size(1) for t in k_dst])
        self._nn = (C.c_int32 * W)(*[int(x) for x in n_new])
        a = HwAppend()
        a.dtype = _DTYPE_CODE[self.dtype]
        a.mode = int(mode)
        a.W, a.Hkv, a.E, a.Ev = W, self.Hkv, self.E, self.Ev
        a.k_dst, a.v_dst = C.cast(self._kp, C.POINTER(C.c_void_p)), C.cast(self._vp, C.POINTER(C.c_void_p))
        a.dst_len, a.dst_cap, a.n_new = (C.cast(self._ln, C.POINTER(C.c_int32)), C.cast(self._cp, C.POINTER(C.c_int32)),
                                         C.cast(self._nn, C.POINTER(C.c_int32)))
        a.len_dev = len_dev.data_ptr()
        self.a = a

    def run(self, key_states: torch.Tensor, value_states: torch.Tensor, cosines: Optional[torch.Tensor] = None,
            sines: Optional[torch.Tensor] = None) -> None:
        a = self.a
        W, Hkv, S, E = key_states.shape
        if (W, Hkv, E) != (self.W, self.Hkv, self.E) or tuple(value_states.shape) != (W, Hkv, S, self.Ev) \
                or key_states.dtype != self.dtype or value_states.dtype != self.dtype or key_states.device != self.device:
            raise ValueError("new states do not match the prepared append")
        if (E > 1 and key_states.stride(3) != 1) or (self.Ev > 1 and value_states.stride(3) != 1):
            key_states, value_states = key_states.contiguous(), value_states.contiguous()
        a.S = S
        a.key_states, a.value_states = key_states.data_ptr(), value_states.data_ptr()
        a.ks_w, a.ks_h, a.ks_s = key_states.stride(0), key_states.stride(1), key_states.stride(2)
        a.vs_w, a.vs_h, a.vs_s = value_states.stride(0), value_states.stride(1), value_states.stride(2)
        if cosines is None:
            a.RotE, a.cs_dtype, a.cosines, a.sines = 0, HW_F32, None, None
        else:
            if sines is None or cosines.shape != sines.shape or cosines.dim() != 3 or cosines.size(0) != W or cosines.size(1) not in (1, S) \
                    or cosines.dtype != sines.dtype or cosines.dtype not in (torch.float32, self.dtype):
                raise ValueError("cosines / sines must be [W, S, RotE] or [W, 1, RotE], float32 or in the dtype of the keys")
            cosines, sines = cosines.contiguous(), sines.contiguous()
            a.RotE = cosines.size(2)
            a.cs_dtype = _DTYPE_CODE[cosines.dtype]
            a.cosines, a.sines = cosines.data_ptr(), sines.data_ptr()
            a.cs_w = cosines.stride(0)
            a.cs_s = 0 if cosines.size(1) == 1 else cosines.stride(1)
        stream = torch.cuda.current_stream(self.device).cuda_stream
        check(lib.hw_rope_append(C.byref(a), C.c_void_p(stream)), "hw_rope_append")


def rope(q: torch.Tensor, cosines: torch.Tensor, sines: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    F, W, Hq, S, E = out.shape
    if tuple(q.shape) != (W, Hq, S, E) or q.dtype != out.dtype:
        raise ValueError("queries must be [W, Hq, S, E] in the output dtype")
    rot = cosines.size(-1)
    if tuple(cosines.shape) != (F, W, S, rot) or tuple(sines.shape) != (F, W, S, rot):
        raise ValueError("cosines / sines must be [F, W, S, RotE]")
    if cosines.dtype != torch.float32 or sines.dtype != torch.float32:
        raise ValueError("cosines / sines must be float32")
    for t in (q, cosines, sines, out):
        if not t.is_contiguous():
            raise ValueError("all tensors must be contiguous")
    with torch.cuda.device(out.device):
        stream = torch.cuda.current_stream(out.device).cuda_stream
        check(lib.hw_rope(out.data_ptr(), q.data_ptr(), cosines.data_ptr(), sines.data_ptr(), _DTYPE_CODE[out.dtype],
                          F, W, Hq, S, E, rot, C.c_void_p(stream)), "hw_rope")
    return out
