"""Host-side mirror of the reference's cache bookkeeping (python/hogwild/attention.py:97-257) on top of the HIP
library: the objects a model's attention layer talks to during a Hogwild! decode step.

  SegmentCache ...... one KV segment (a prompt, a worker's private continuation, ...).  Plays the part the
                      transformers `Cache` objects play in the reference (`cache_structure` entries), with the
                      members the reference uses: get_seq_length, key_cache[layer], value_cache[layer], update.
                      K/V live in preallocated [Hkv, capacity, D] buffers per layer and grow in place, so appending
                      never reallocates and the attention kernel reads the segments where they are.
  HogwildCache ...... HogwildCache of the reference (attention.py:115-248): same constructor order, update() returning a
                      CacheStructure, get_queries_buffer / get_att_buffer / get_input_kwargs.  The per-worker Python
                      loop of update (:148-158) is one `hw_rope_append` launch; the layer-0 construction of locations and
                      rotary tables (:164-196) is one `hw_build_inputs` launch.
  merge_caches ...... attention.py:251-257: re-rotate a segment by the target's length and append it.

Everything numeric runs in the HIP library; there is no torch fallback.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, List, Optional, Sequence

import torch

from . import _lib


class _LayerViews:
    """`segment.key_cache[layer]` -> the [1, Hkv, L, D] view of what has been written so far."""

    def __init__(self, seg: "SegmentCache", bufs: List[torch.Tensor]):
        self._seg, self._bufs = seg, bufs

    def __getitem__(self, layer: int) -> torch.Tensor:
        return self._bufs[layer][:, : self._seg.lengths[layer], :].unsqueeze(0)

    def __len__(self) -> int:
        return len(self._bufs)


class SegmentCache:
    def __init__(self, num_layers: int, num_kv_heads: int, head_dim: int, capacity: int, *, dtype=torch.bfloat16, device="cuda",
                 value_head_dim: Optional[int] = None):
        ev = head_dim if value_head_dim is None else value_head_dim
        self.capacity = int(capacity)
        self.k = [torch.empty((num_kv_heads, self.capacity, head_dim), dtype=dtype, device=device) for _ in range(num_layers)]
        self.v = [torch.empty((num_kv_heads, self.capacity, ev), dtype=dtype, device=device) for _ in range(num_layers)]
        self.lengths = [0] * num_layers
        self.key_cache = _LayerViews(self, self.k)
        self.value_cache = _LayerViews(self, self.v)

    def get_seq_length(self, layer_idx: Optional[int] = 0) -> int:
        return self.lengths[layer_idx or 0]

    def reserve(self, layer_idx: int, n_new: int) -> None:
        """Room for n_new more tokens in one layer's buffers.  A full segment moves into buffers of twice the size (the
        transformers caches of the reference grow by torch.cat on every update); the copy is the only reallocation
        a segment ever sees, and the capacity becomes the new row distance between its kv heads."""
        need = self.lengths[layer_idx] + int(n_new)
        cap = self.k[layer_idx].size(1)
        if need <= cap:
            return
        new_cap = max(need, 2 * cap)
        for bufs in (self.k, self.v):
            old = bufs[layer_idx]
            grown = torch.empty((old.size(0), new_cap, old.size(2)), dtype=old.dtype, device=old.device)
            grown[:, : self.lengths[layer_idx]].copy_(old[:, : self.lengths[layer_idx]])
            bufs[layer_idx] = grown
        self.capacity = max(self.capacity, new_cap)

    def update(self, key_states: torch.Tensor, value_states: torch.Tensor, layer_idx: int, cache_kwargs: Optional[Dict[str, Any]] = None):
        """Append [1, Hkv, n, D] keys (already rotated) and values; returns the views of the grown segment."""
        self.reserve(layer_idx, key_states.size(2))
        _lib.rope_append(key_states, value_states, [self.k[layer_idx]], [self.v[layer_idx]], [self.lengths[layer_idx]])
        self.lengths[layer_idx] += key_states.size(2)
        return self.key_cache[layer_idx], self.value_cache[layer_idx]


@dataclass
class CacheStructure:                      # attention.py:105-112
    keys: List[torch.Tensor]
    values: List[torch.Tensor]
    frags: torch.Tensor
    cos: torch.Tensor
    sin: torch.Tensor
    loc: torch.Tensor


def _rotary_parameters(model, inv_freq, attention_scaling):
    if inv_freq is None:
        rot = model.model.rotary_emb if hasattr(model, "model") else model.rotary_emb     # attention.py:122,191
        inv_freq = rot.inv_freq
        attention_scaling = float(getattr(rot, "attention_scaling", 1.0))
    return inv_freq.detach().to(torch.float32).contiguous(), float(attention_scaling)


class HogwildCache:
    def __init__(self, cache_structure: List[List[SegmentCache]], model=None, write_to: Optional[List[SegmentCache]] = None, *,
                 inv_freq: Optional[torch.Tensor] = None, attention_scaling: float = 1.0, table_dtype: Optional[torch.dtype] = None):
        """cache_structure[w] = the segments worker w attends to, in its order; write_to[w] = where its new tokens go
        (default: the last segment of its order).  The rotary parameters come from `model.model.rotary_emb`
        (inv_freq, attention_scaling) or are given directly.  table_dtype: dtype the query tables are rounded to before
        being widened to float32, as the model library returns them in the model dtype (attention.py:191-193);
        default = the dtype of the keys."""
        if model is None and inv_freq is None:
            raise ValueError("either a model with a rotary embedding or inv_freq is needed")
        self.cache_structure = cache_structure
        self.write_to = write_to if write_to else [cl[-1] for cl in cache_structure]
        self.inv_freq, self.attention_scaling = _rotary_parameters(model, inv_freq, attention_scaling)
        self.table_dtype = table_dtype
        ids = {id(cs) for cs in cache_structure[0]}
        for order in cache_structure:
            if {id(cs) for cs in order} != ids or len(order) != len(ids):
                raise ValueError("every worker must list the same segments, each once (attention.py:168-181)")
        self.cosines = self.sines = self.locations = self.frags = None
        self.segments: List[SegmentCache] = []
        self.queries_buffer = None
        self.att_buffer = None
        self._dev = None        # state of the device-resident-lengths mode, see use_device_lengths

    # ---- lengths in device memory: decode steps that can be captured once and replayed ------------------------------
    def use_device_lengths(self, headroom: int, new_tokens: int = 1, n_new: Optional[Sequence[int]] = None) -> None:
        """From now on the segment lengths live in a device tensor that every step advances on the device, so a decode
        step (update_fused + hogwild_fused for every layer) can be captured in a HIP graph once and replayed while the
        segments grow: nothing about a step depends on host numbers any more.  Every step brings `new_tokens` tokens per
        worker, of which worker w appends the last n_new[w] (left masking with the same mask in every step; default: all
        of them).  The attention split is planned for lengths up to `headroom` tokens
        beyond the present ones, and the buffers are grown to hold them now, so a capture is good for
        headroom // new_tokens steps; call this again to re-plan.  The host-side lengths are not touched by the steps:
        sync_lengths() reads them back.  No counterpart in the reference, whose segments are re-allocated on every
        update (attention.py:148-158)."""
        segments = list(self.cache_structure[0])
        index = {id(cs): f for f, cs in enumerate(segments)}
        for seg in segments:
            if len(set(seg.lengths)) != 1:
                raise ValueError("all layers of a segment must hold the same number of tokens (call between decode steps)")
        if len({id(seg) for seg in self.write_to}) != len(self.write_to):
            raise ValueError("with device-resident lengths every worker needs a segment of its own to write to")
        if any(seg is not order[-1] for seg, order in zip(self.write_to, self.cache_structure)):
            # position ids are formed from the last segment of a worker's order (attention.py:238-246) in both modes
            raise ValueError("with device-resident lengths every worker must write to the last segment of its order")
        n_new = [int(new_tokens)] * len(self.write_to) if n_new is None else [int(x) for x in n_new]
        if len(n_new) != len(self.write_to) or any(x < 0 or x > int(new_tokens) for x in n_new):
            raise ValueError("n_new: one number per worker, between 0 and new_tokens")
        add = [0] * len(segments)
        for seg, n in zip(self.write_to, n_new):
            add[index[id(seg)]] += n
        bound = [seg.get_seq_length() + (int(headroom) if add[f] else 0) for f, seg in enumerate(segments)]
        for f, seg in enumerate(segments):
            for layer in range(len(seg.k)):
                seg.reserve(layer, bound[f] - seg.lengths[layer])
        dev = segments[0].k[0].device
        self._dev = {
            "segments": segments, "orders": [[index[id(cs)] for cs in order] for order in self.cache_structure],
            "write_index": [index[id(seg)] for seg in self.write_to], "add": add, "S": int(new_tokens), "bound": bound,
            "n_new": n_new, "n_new_dev": torch.tensor(n_new, dtype=torch.int64, device=dev),
            "len_dev": torch.tensor([seg.get_seq_length() for seg in segments], dtype=torch.int32, device=dev),
            "write_index_dev": torch.tensor([index[id(seg)] for seg in self.write_to], dtype=torch.int64, device=dev),
            "tables": None, "views": {}, "appends": {},
        }

    @property
    def device_lengths(self) -> bool:
        return self._dev is not None

    def sync_lengths(self) -> None:
        """Device-resident lengths -> host-side lengths of every segment and layer (synchronises with the device)."""
        if self._dev is None:
            return
        lens = self._dev["len_dev"].tolist()
        over = [f for f, (n, b) in enumerate(zip(lens, self._dev["bound"])) if n > b]
        if over:
            raise RuntimeError(f"segments {over} grew beyond the lengths the steps were planned for ({lens} vs {self._dev['bound']}): "
                               "the captured step was replayed more often than headroom // new_tokens; the tokens beyond the bounds "
                               "were not attended to")
        for seg, n in zip(self._dev["segments"], lens):
            seg.lengths = [int(n)] * len(seg.lengths)

    def device_steps_left(self) -> int:
        """How many more steps the current plan covers (reads the lengths back: synchronises with the device)."""
        if self._dev is None:
            raise ValueError("not in the device-resident-lengths mode")
        lens = self._dev["len_dev"].tolist()
        return min(((b - n) // a for n, b, a in zip(lens, self._dev["bound"], self._dev["add"]) if a > 0), default=0)

    def use_host_lengths(self) -> None:
        """Leave the device-resident-lengths mode (after reading the lengths back).  The mode is left even if the read-back
        finds an overrun: the host lengths are then clamped to the planned bounds (what was attended to) and the error is
        raised afterwards."""
        d = self._dev
        if d is None:
            return
        self._dev = None
        lens = d["len_dev"].tolist()
        for seg, n, b in zip(d["segments"], lens, d["bound"]):
            seg.lengths = [int(min(n, b))] * len(seg.lengths)
        over = [f for f, (n, b) in enumerate(zip(lens, d["bound"])) if n > b]
        if over:
            raise RuntimeError(f"segments {over} grew beyond the lengths the steps were planned for ({lens} vs {d['bound']}): "
                               "the captured step was replayed more often than headroom // new_tokens; the tokens beyond the "
                               "bounds were dropped")

    def _update_dev(self, key_states, value_states, cos, sin, layer_idx, mode) -> CacheStructure:
        d = self._dev
        W, S = key_states.size(0), key_states.size(2)
        if W != len(self.cache_structure) or S != d["S"]:
            raise ValueError(f"device-resident lengths were set up for {len(self.cache_structure)} workers x {d['S']} new tokens")
        if layer_idx == 0:
            _lib.advance_lengths(d["len_dev"], d["add"])                  # lengths including this step's tokens
            tdt = self.table_dtype if self.table_dtype is not None else key_states.dtype
            d["tables"] = _lib.build_inputs_dev(d["len_dev"], d["orders"], S, self.inv_freq.to(key_states.device),
                                                attention_scaling=self.attention_scaling,
                                                table_dtype=None if tdt == torch.float32 else tdt, out=d["tables"])
            self.locations, self.cosines, self.sines = d["tables"]
            self.segments = d["segments"]
            self.frags = d["len_dev"]
        plan = d["appends"].get((layer_idx, mode))
        if plan is None:        # destinations, capacities and token counts stay the same from step to step
            segs = self.write_to
            plan = _lib.AppendPlan([s.k[layer_idx] for s in segs], [s.v[layer_idx] for s in segs], d["write_index"], d["n_new"],
                                   d["len_dev"], mode)
            d["appends"][(layer_idx, mode)] = plan
        plan.run(key_states, value_states, cos, sin)
        # the fragments as the operator sees them: views up to the planned bounds (the same in every step, so they are
        # made once per layer), current lengths in `frags`
        views = d["views"].get(layer_idx)
        if views is None:
            views = ([seg.k[layer_idx][:, :b, :].unsqueeze(0) for seg, b in zip(d["segments"], d["bound"])],
                     [seg.v[layer_idx][:, :b, :].unsqueeze(0) for seg, b in zip(d["segments"], d["bound"])])
            d["views"][layer_idx] = views
        return CacheStructure(keys=views[0], values=views[1], cos=self.cosines, sin=self.sines, loc=self.locations, frags=self.frags)

    def get_seq_length(self, layer_idx: Optional[int] = 0) -> int:
        if self._dev is not None:      # the host-side lengths are stale in this mode: read the device's (synchronises)
            f = [id(cs) for cs in self._dev["segments"]].index(id(self.cache_structure[0][-1]))
            return int(self._dev["len_dev"][f].item())
        return self.cache_structure[0][-1].get_seq_length()        # attention.py:133-135

    # ---- the append ------------------------------------------------------------------------------------------------
    def _append(self, key_states, value_states, layer_idx, mask, cosines, sines, mode):
        W = key_states.size(0)
        assert W == len(self.cache_structure)                       # attention.py:145
        S = key_states.size(2)
        n_new = [S] * W if mask is None else [int(x) for x in torch.sum(mask, dim=1).tolist()]   # left masking, :149-155
        segs = self.write_to
        # workers that write to the same segment append one behind the other, in worker order (the reference's loop, :148-158)
        end: Dict[int, int] = {}
        dst = []
        for s, n in zip(segs, n_new):
            start = end.get(id(s), s.lengths[layer_idx])
            dst.append(start)
            end[id(s)] = start + n
        for s in segs:
            s.reserve(layer_idx, end[id(s)] - s.lengths[layer_idx])
        _lib.rope_append(key_states, value_states, [s.k[layer_idx] for s in segs], [s.v[layer_idx] for s in segs],
                         dst, cosines=cosines, sines=sines, n_new=n_new, mode=mode)
        for s in segs:
            s.lengths[layer_idx] = end[id(s)]

    def _structure(self, key_states, layer_idx) -> CacheStructure:
        W, S = key_states.size(0), key_states.size(2)
        if layer_idx == 0:
            segments = list(self.cache_structure[0])                # the order of the first worker, attention.py:168-170,186-188
            index = {id(cs): f for f, cs in enumerate(segments)}
            pos_end = [[0] * W for _ in segments]
            for w in range(W):
                pos = 0
                for cs in reversed(self.cache_structure[w]):        # attention.py:174-181
                    pos += cs.get_seq_length(layer_idx)
                    pos_end[index[id(cs)]][w] = pos
            tdt = self.table_dtype if self.table_dtype is not None else key_states.dtype
            self.locations, self.cosines, self.sines = _lib.build_inputs(
                pos_end, S, self.inv_freq.to(key_states.device), attention_scaling=self.attention_scaling,
                table_dtype=None if tdt == torch.float32 else tdt)
            self.segments = segments
            self.frags = torch.tensor([cs.get_seq_length(layer_idx) for cs in segments], dtype=torch.int32, device=key_states.device)
        keys = [cs.key_cache[layer_idx] for cs in self.segments]    # views; no .contiguous() copies (attention.py:160-162,199-203)
        vals = [cs.value_cache[layer_idx] for cs in self.segments]
        return CacheStructure(keys=keys, values=vals, cos=self.cosines, sin=self.sines, loc=self.locations, frags=self.frags)

    def update(self, key_states: torch.Tensor, value_states: torch.Tensor, layer_idx: int,
               cache_kwargs: Optional[Dict[str, Any]] = None) -> CacheStructure:
        """key_states [W, Hkv, S, D] already rotated (the reference rotates them before the call, attention.py:315)."""
        mask = (cache_kwargs or {}).get("mask", None)
        if self._dev is not None:
            return self._update_dev(key_states, value_states, None, None, layer_idx, _lib.HW_ROPE_EAGER)
        self._append(key_states, value_states, layer_idx, mask, None, None, _lib.HW_ROPE_EAGER)
        return self._structure(key_states, layer_idx)

    def update_fused(self, key_states: torch.Tensor, value_states: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, layer_idx: int,
                     mask: Optional[torch.Tensor] = None, mode: int = _lib.HW_ROPE_EAGER) -> CacheStructure:
        """The same with un-rotated keys and the model's position embeddings cos/sin [W, S, RotE] of the new tokens:
        rotation (attention.py:313-315) and append (:148-158) in one launch."""
        if self._dev is not None:      # (a mask, if given, must be the one n_new was derived from; it is not read here)
            return self._update_dev(key_states, value_states, cos, sin, layer_idx, mode)
        self._append(key_states, value_states, layer_idx, mask, cos, sin, mode)
        return self._structure(key_states, layer_idx)

    # ---- buffers and model inputs -----------------------------------------------------------------------------------
    def get_queries_buffer(self, queries: torch.Tensor, layer_idx: int) -> torch.Tensor:      # attention.py:206-211
        if layer_idx == 0:
            self.queries_buffer = torch.empty((self.cosines.size(0), queries.size(0), queries.size(1), queries.size(2), queries.size(3)),
                                              dtype=queries.dtype, device=queries.device)
        return self.queries_buffer

    def get_att_buffer(self, r_queries: torch.Tensor, layer_idx: int) -> torch.Tensor:        # attention.py:213-218
        if layer_idx == 0:
            self.att_buffer = torch.empty((r_queries.size(1), r_queries.size(2), r_queries.size(3), self.cache_structure[0][0].v[layer_idx].size(2)),
                                          dtype=r_queries.dtype, device=r_queries.device)
        return self.att_buffer

    def get_input_kwargs(self, input_ids: torch.Tensor, attention_mask: Optional[torch.Tensor] = None) -> Dict[str, Any]:   # :220-248
        nw = len(self.cache_structure)
        assert input_ids.shape[0] == nw, (input_ids.shape, nw)
        S = input_ids.shape[1]
        if self._dev is not None:      # positions from the lengths in device memory (before this step's append)
            ends = self._dev["len_dev"].index_select(0, self._dev["write_index_dev"]).to(torch.int64) + self._dev["n_new_dev"]
            pos_ids = ends[:, None] - S + torch.arange(S, dtype=torch.int64, device=input_ids.device)[None, :]
            return {"input_ids": input_ids, "attention_mask": attention_mask, "past_key_values": self, "use_cache": True,
                    "position_ids": pos_ids}
        new = [S] * nw if attention_mask is None else [int(x) for x in torch.sum(attention_mask, dim=1).tolist()]
        ends = torch.tensor([self.cache_structure[w][-1].get_seq_length() + new[w] for w in range(nw)], dtype=torch.int64, device=input_ids.device)
        pos_ids = ends[:, None] - S + torch.arange(S, dtype=torch.int64, device=input_ids.device)[None, :]
        return {"input_ids": input_ids, "attention_mask": attention_mask, "past_key_values": self, "use_cache": True, "position_ids": pos_ids}


def merge_caches(target: SegmentCache, source: SegmentCache, model=None, *, inv_freq: Optional[torch.Tensor] = None,
                 attention_scaling: float = 1.0, table_dtype: Optional[torch.dtype] = None, mode: int = _lib.HW_ROPE_EAGER) -> None:
    """Append `source` to `target`, rotating its keys further by target's length (attention.py:251-257): every key of
    the source gets the same rotation, that of position target.get_seq_length()."""
    inv_freq, attention_scaling = _rotary_parameters(model, inv_freq, attention_scaling)
    n = source.get_seq_length()
    if n == 0:
        return
    dev = source.k[0].device
    tdt = table_dtype if table_dtype is not None else source.k[0].dtype
    # one table row: the position is target's length for every source token (S = 1 and pos_end = length + 1)
    _, cos, sin = _lib.build_inputs([[target.get_seq_length() + 1]], 1, inv_freq.to(dev), attention_scaling=attention_scaling,
                                    table_dtype=None if tdt == torch.float32 else tdt)
    cos = cos.reshape(1, 1, -1).to(tdt)
    sin = sin.reshape(1, 1, -1).to(tdt)
    for layer in range(len(target.k)):
        m = source.lengths[layer]
        target.reserve(layer, m)          # grow like every other append (the reference's merge goes through target.update)
        _lib.rope_append(source.k[layer][:, :m, :].unsqueeze(0), source.v[layer][:, :m, :].unsqueeze(0), [target.k[layer]], [target.v[layer]],
                         [target.lengths[layer]], cosines=cos, sines=sin, mode=mode)
        target.lengths[layer] += m
