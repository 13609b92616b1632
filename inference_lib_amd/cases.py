"""Synthetic decode-step workloads for the Hogwild! attention path.

Each case is what one call of the fused operator sees for one decoder layer: the un-rotated query
`q[W,Hq,S,E]`, the KV fragments `keys[f]/values[f] : [Hkv, L_f, E]` (shared prompt first, then one
segment per worker, then optional per-worker "current step" fragments), `locations[F,W,S]`
(mask bound and RoPE angle of the query per fragment) and the fp32 `cos/sin[F,W,S,E]` tables.
The way `locations` is formed follows the caller's contract, python/hogwild/attention.py:164-196:
walking a worker's own ordering of fragments from the end, pos += len; loc = arange(pos-S, pos).

All data is drawn on the CPU from torch.Generator().manual_seed(seed) in a fixed order
(ragged lengths, then q, then K_f, V_f for f in fragment order) so that every process regenerates
identical inputs.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch

DTYPES = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}


@dataclass
class Case:
    name: str
    dtype: str                      # "f32" | "f16" | "bf16"
    W: int
    S: int
    Hq: int
    Hkv: int
    E: int
    scale: float
    rope_base: float
    lens: List[int]                 # fragment lengths, fragment order
    orders: List[List[int]]         # per worker: fragment ids it sees, oldest first
    q: torch.Tensor = None
    keys: List[torch.Tensor] = field(default_factory=list)
    values: List[torch.Tensor] = field(default_factory=list)
    locations: torch.Tensor = None  # int32 [F,W,S]
    cos: torch.Tensor = None        # fp32 [F,W,S,E]
    sin: torch.Tensor = None

    @property
    def F(self) -> int:
        return len(self.lens)

    def visible_tokens(self) -> int:
        """sum over fragments of the longest visible prefix over all query rows."""
        loc = self.locations
        tot = 0
        for f, L in enumerate(self.lens):
            tot += int(min(L, max(0, int(loc[f].max()) + 1)))
        return tot

    def kv_bytes(self) -> int:
        """Algorithmic bytes of one step: every visible K and V element read once."""
        esz = torch.empty((), dtype=DTYPES[self.dtype]).element_size()
        return self.visible_tokens() * self.Hkv * (self.E + self.E) * esz

    def to(self, device) -> "Case":
        c = Case(**{k: getattr(self, k) for k in
                    ("name", "dtype", "W", "S", "Hq", "Hkv", "E", "scale", "rope_base", "lens", "orders")})
        c.q = self.q.to(device)
        c.keys = [k.to(device) for k in self.keys]
        c.values = [v.to(device) for v in self.values]
        c.locations = self.locations.to(device)
        c.cos = self.cos.to(device)
        c.sin = self.sin.to(device)
        return c


def locations_for(orders: List[List[int]], lens: List[int], S: int) -> torch.Tensor:
    F, W = len(lens), len(orders)
    loc = torch.full((F, W, S), -1, dtype=torch.int32)
    for w, order in enumerate(orders):
        pos = 0
        for f in reversed(order):
            pos += lens[f]
            loc[f, w] = torch.arange(pos - S, pos, dtype=torch.int32)
    return loc


def rope_tables(locations: torch.Tensor, rot_dim: int, base: float):
    """fp32 cos/sin [F,W,S,rot_dim] with inv_freq_i = base**(-2i/rot_dim), duplicated halves."""
    half = rot_dim // 2
    inv = base ** (-(torch.arange(half, dtype=torch.float64) * 2.0) / rot_dim)
    ang = locations.to(torch.float64)[..., None] * inv
    ang = torch.cat([ang, ang], dim=-1)
    return torch.cos(ang).to(torch.float32), torch.sin(ang).to(torch.float32)


def build_case(name: str, dtype: str, W: int, S: int, Hq: int, Hkv: int, E: int, rope_base: float,
               lens: List[int], orders: List[List[int]], gen: torch.Generator,
               q_scale: float = 1.0, rot_dim: Optional[int] = None) -> Case:
    td = DTYPES[dtype]
    c = Case(name=name, dtype=dtype, W=W, S=S, Hq=Hq, Hkv=Hkv, E=E, scale=E ** -0.5,
             rope_base=rope_base, lens=list(lens), orders=orders)
    c.q = (torch.randn((W, Hq, S, E), generator=gen) * q_scale).to(td)
    for L in lens:
        c.keys.append(torch.randn((Hkv, L, E), generator=gen).to(td))
        c.values.append(torch.randn((Hkv, L, E), generator=gen).to(td))
    c.locations = locations_for(orders, c.lens, S)
    c.cos, c.sin = rope_tables(c.locations, rot_dim or E, rope_base)
    return c


def _prompt_segments_orders(W: int, with_cur: bool) -> List[List[int]]:
    """Fragment ids: 0 = prompt, 1..W = worker segments, W+1..2W = per-worker current-step fragments.
    Worker w sees [prompt, other workers' segments..., own segment, own current-step fragment]."""
    orders = []
    for w in range(W):
        o = [0] + [1 + x for x in range(W) if x != w] + [1 + w]
        if with_cur:
            o.append(1 + W + w)
        orders.append(o)
    return orders


def baseline_case(idx: int) -> Case:
    """The five workload configurations, numbered 1..5 (config 3 is the benchmark headline), and 6: head dimension 256."""
    g = torch.Generator().manual_seed(idx - 1)
    if idx == 1:   # fp32 parity case: prompt 256 + one 64-token segment per worker, fragment order
        # = worker 0's ordering [prompt, seg1, seg0]
        lens = [256, 64, 64]
        orders = [[0, 1, 2], [0, 2, 1]]
        return build_case("c1_fp32_w2_gqa4_d64", "f32", 2, 1, 8, 2, 64, 1e4, lens, orders, g)
    if idx == 2:   # Qwen2.5-7B shape
        lens = [2048, 1024, 1024]
        return build_case("c2_qwen7b_w2", "bf16", 2, 1, 28, 4, 128, 1e6, lens, _prompt_segments_orders(2, False), g)
    if idx == 3:   # QwQ-32B shape, 4 workers, ragged current-step fragments
        cur = torch.randint(1, 129, (4,), generator=g).tolist()
        lens = [4096] + [2048] * 4 + cur
        return build_case("c3_qwq32b_w4", "bf16", 4, 1, 40, 8, 128, 1e6, lens, _prompt_segments_orders(4, True), g)
    if idx == 4:   # Llama-3-8B shape long context, 8 workers, ragged segments + 1-token current step
        seg = torch.randint(1, 4097, (8,), generator=g).tolist()
        lens = [16384] + seg + [1] * 8
        return build_case("c4_llama8b_w8", "bf16", 8, 1, 32, 8, 128, 5e5, lens, _prompt_segments_orders(8, True), g)
    if idx == 5:   # multi-token step, fp16
        lens = [8192] + [2048] * 4
        return build_case("c5_multitoken_w4s4", "f16", 4, 4, 64, 8, 128, 1e6, lens, _prompt_segments_orders(4, False), g)
    if idx == 6:   # not one of the reference's configurations: the headline's fragments at head dimension 256
        # (the Gemma-2-9B head shape: 16 query heads on 8 kv heads), 4 workers
        cur = torch.randint(1, 129, (4,), generator=g).tolist()
        lens = [4096] + [2048] * 4 + cur
        return build_case("c6_gemma9b_w4_d256", "bf16", 4, 1, 16, 8, 256, 1e4, lens, _prompt_segments_orders(4, True), g)
    raise ValueError(f"no such baseline case: {idx}")


def small_case(dtype: str = "bf16", W: int = 2, S: int = 1, Hq: int = 8, Hkv: int = 2, E: int = 128,
               lens=(100, 37, 65), seed: int = 11, with_cur: bool = False, rope_base: float = 1e4,
               rot_dim: Optional[int] = None) -> Case:
    """A small ragged case for parity tests (lens[0] = prompt, then W segments, then optional W
    current-step fragments)."""
    g = torch.Generator().manual_seed(seed)
    lens = list(lens)
    assert len(lens) == 1 + W * (2 if with_cur else 1)
    return build_case(f"small_{dtype}_w{W}s{S}", dtype, W, S, Hq, Hkv, E, rope_base, lens,
                      _prompt_segments_orders(W, with_cur), g, rot_dim=rot_dim)
