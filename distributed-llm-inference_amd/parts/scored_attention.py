"""Grouped-query attention over the paged cache whose scores are changed by parameters: unit-RMS
queries and keys or a rotary position encoding, a per-head logarithmic distance penalty, a chunked
mask, a window that keeps the first positions, a softmax with a sink, value mixing across layers, a sigmoid
output gate, biases on the projections, several score maps a head over the same values whose results are
subtracted (differential attention), and keys and values read from another layer's cache. Each is a
parameter, so another design may take any subset.

Order of work for the rows ``h`` of a step (``x`` may be a 32-bit residual stream; the products read
it in the runtime's type):

1. one product gives q, k, v and the gate's pre-activation (the checkpoint's matrices stacked at
   load), as 32-bit sums;
2. one kernel divides every head's q and k by its root mean square over ``dim`` (``qk_unit``), mixes
   v with the values that the first such layer of the step computed for the same token
   (``value_mix``: ``v <- (1 - m) v + m v_first``), and writes k and the mixed v into the cache pages;
   with ``qk_unit=False`` the kernel instead rotates q and k as the ``position`` part's rotary table
   says (any leading part of a head, pairs side by side or half a head apart; no table: q and k as
   projected) and writes k and v into the pages;
3. the attention kernel: ``s_ij = scale (q_i . k_j) - r1_h log(1 + r2_h (i - j))`` for ``j <= i`` in
   the same chunk of ``chunk`` positions (counted from the request's position 0), weights
   ``exp(s_ij) / (sink + sum_j exp(s_ij))`` with ``sink = 1`` (a key of score 0 that has no value),
   the result multiplied by ``sigmoid(gate)``;
4. the output product, 32-bit sums.

With ``maps=2`` every query head and every kv head has two sets of ``head_dim`` components (the checkpoint lays
them out head by head as map 1, map 2; they are reordered at load to all heads' first maps, then all second
maps, so that each map is a head of its own to the kernels, and the value pages hold one head per kv head
that both maps read). Each map is a softmax attention of its own; with ``a1, a2`` their results and
``lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff`` (four vectors of ``head_dim`` values, one number a layer),
the head's result is ``d / sqrt(mean(d^2) + norm_eps) * (1 - diff)`` with ``d = a1 - lambda a2``, times
``sigmoid(W_g h)_head`` where ``head_gate`` (one number a head). ``own_kv=False``: the layer has no key and value
projections and reads the cache of the schedule entry it is given (keys as that layer rotated them).

Scores, weights, norms and the mixing are 32-bit; keys and values are cached in the runtime's type.
"""

from __future__ import annotations

import math
from typing import Any, Mapping, Optional

import torch

from ..kernels import ops
from .base import Mixer, PagedKVSpec, PositionEncoding, Runtime
from .linear import as_operand, linear_f32, stack_rows
from .registry import build_part, register_part
from .spec import PartSpec, WeightSpec


def paged_scored_attention(rt: Runtime, ctx: Any, cache: Any, q: torch.Tensor, out: torch.Tensor, num_heads: int,
                           head_dim: int, value_dim: int, scale: float, *, gate: Optional[torch.Tensor] = None,
                           **changes: Any) -> None:
    """The attention of a step's rows over a paged cache, for any mixer that has written its keys and
    values there: steps of single tokens go to the kernel that reads the context's device arrays alone,
    the portions of other steps to the matrix cores where they take the sizes (single tokens, which come
    first, to their kernel), else to the vector-unit tile kernel. ``changes``: ``window``, ``chunk``, ``sink``,
    ``r1``, ``r2`` as :func:`dli_amd.kernels.ops.attention_scored` takes them."""
    grp = ctx.groups[cache.group]
    nd = ctx.num_decode
    if nd == ctx.num_entries:
        # every entry is one row: nothing is derived from the step's lengths on the host
        ops.attention_scored(q, cache.k_pages, cache.v_pages, out, ctx.q_start, ctx.kv_len, grp.block_tables,
                             None, None, num_heads, scale, gate=gate, **changes)
    elif ops.attention_scored_mfma_supports(head_dim, value_dim, ctx.page_size, rt.dtype):
        if nd:
            ops.attention_scored(q[:nd], cache.k_pages, cache.v_pages, out[:nd], ctx.q_start[:nd + 1], ctx.kv_len[:nd],
                                 grp.block_tables[:nd], None, None, num_heads, scale,
                                 gate=None if gate is None else gate[:nd], **changes)
        tiles = ctx.q_tiles(ops.SCORED_MFMA_TILE_ROWS, first_entry=nd)
        ops.attention_scored_mfma(q, cache.k_pages, cache.v_pages, out, ctx.q_start, ctx.kv_len, grp.block_tables,
                                  tiles[0], tiles[1], num_heads, scale, gate=gate, **changes)
    else:
        tiles = ctx.q_tiles(ops.attention_generic_tile_rows(max(head_dim, value_dim)))
        ops.attention_scored(q, cache.k_pages, cache.v_pages, out, ctx.q_start, ctx.kv_len, grp.block_tables,
                             tiles[0], tiles[1], num_heads, scale, gate=gate, **changes)


@register_part("mixer", "scored_attention")
class ScoredAttention(Mixer):
    VALUE_MIX = ("none", "source", "mix")

    def __init__(self, runtime: Runtime, *, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 value_dim: Optional[int] = None, scale: Optional[float] = None, qk_unit: bool = True,
                 norm_eps: float = 1e-6, distance_penalty: bool = False, chunk: int = 0, window: int = 0,
                 sink: bool = False, output_gate: bool = False, value_mix: str = "none",
                 value_mix_key: str = "first_values", names: Optional[Mapping[str, str]] = None,
                 position: Optional[PartSpec] = None, bias: bool = False, keep_first: int = 0, maps: int = 1,
                 diff: float = 0.0, head_gate: bool = False, own_kv: bool = True, cache_window: Optional[int] = None) -> None:
        """``cache_window``: how many of the latest keys the pages must keep where that is not this layer's own
        window (0: all): other layers that read this layer's cache may look further back than it does."""
        super().__init__(runtime)
        if cache_window is not None and (cache_window < 0 or (cache_window and (not window or keep_first or cache_window < window))):
            raise ValueError("scored_attention: the pages must keep at least what this layer's own mask sees")
        self.cache_window = cache_window
        if maps not in (1, 2):
            raise ValueError("one score map a head, or two whose results are subtracted")
        if maps == 2 and (qk_unit or output_gate or value_mix != "none"):
            raise ValueError("scored_attention: two maps a head go with rotary or plain keys and a gate per head")
        if head_gate and maps != 2:
            raise ValueError("scored_attention: the gate per head belongs to the kernel that combines two maps")
        if (bias or not own_kv) and qk_unit:
            raise ValueError("scored_attention: biases and borrowed keys go with rotary or plain keys")
        if keep_first < 0 or (keep_first and not window):
            raise ValueError("scored_attention: kept first positions belong to a window")
        self.bias, self.keep_first, self.maps, self.diff = bool(bias), int(keep_first), int(maps), float(diff)
        self.head_gate, self.own_kv = bool(head_gate), bool(own_kv)
        self.b_in = None
        self.lam = 0.0
        if num_heads < 1 or num_kv_heads < 1 or num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads do not group onto {num_kv_heads} kv heads")
        value_dim = head_dim if value_dim is None else value_dim
        if not 0 < head_dim <= 256 or not 0 < value_dim <= 256:
            raise ops.KernelArgumentError(f"attention takes heads of 1 to 256, not {head_dim} / {value_dim}")
        if value_mix not in self.VALUE_MIX:
            raise ValueError(f"value_mix must be one of {self.VALUE_MIX}")
        if chunk < 0 or window < 0:
            raise ValueError("chunk and window must not be negative")
        self.hidden_size, self.num_heads, self.num_kv_heads = hidden_size, num_heads, num_kv_heads
        self.head_dim, self.value_dim = head_dim, value_dim
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)
        self.qk_unit, self.norm_eps = bool(qk_unit), float(norm_eps)
        self.distance_penalty, self.chunk, self.window = bool(distance_penalty), int(chunk), int(window)
        self.sink, self.output_gate = bool(sink), bool(output_gate)
        self.value_mix, self.value_mix_key = value_mix, value_mix_key
        self.position = build_part("position", position or PartSpec("none"), runtime)
        if self.qk_unit and position is not None and position.kind != "none":
            raise ValueError("scored_attention: unit keys and a position encoding together have no kernel")
        if not self.qk_unit and value_mix != "none":
            raise ValueError("scored_attention: value mixing belongs to the kernel that makes unit keys")
        self.names = {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o", "mix": "vmix", "r1": "r1", "r2": "r2",
                      "lq1": "lq1", "lk1": "lk1", "lq2": "lq2", "lk2": "lk2", **dict(names or {})}
        self.w_in = self.w_o = self.mix = self.r1 = self.r2 = None

    # -- sizes of the stacked projection's parts
    @property
    def _q(self) -> int:
        return self.num_heads * self.maps * self.head_dim

    @property
    def _k(self) -> int:
        return self.num_kv_heads * self.maps * self.head_dim if self.own_kv else 0

    @property
    def _v(self) -> int:
        return self.num_kv_heads * self.value_dim if self.own_kv else 0

    @property
    def _o(self) -> int:
        return self.num_heads * self.value_dim

    def weight_specs(self) -> dict[str, WeightSpec]:
        n, h = self.names, self.hidden_size
        specs = {n["q"]: WeightSpec((self._q, h)), n["o"]: WeightSpec((h, self._o))}
        if self.own_kv:
            specs.update({n["k"]: WeightSpec((self._k, h)), n["v"]: WeightSpec((self._v, h))})
        if self.bias:
            specs.update({n[s] + ".b": WeightSpec((size,), role="float32", init="zeros")
                          for s, size in (("q", self._q), ("k", self._k), ("v", self._v)) if size})
        if self.output_gate:
            specs[n["g"]] = WeightSpec((self._o, h))
        if self.head_gate:
            specs[n["g"]] = WeightSpec((self.num_heads, h))
        if self.maps == 2:
            specs.update({n[s]: WeightSpec((self.head_dim,), role="float32", init="zeros") for s in ("lq1", "lk1", "lq2", "lk2")})
        if self.distance_penalty:
            specs[n["r1"]] = WeightSpec((self.num_heads,), role="float32", init="norm")
            specs[n["r2"]] = WeightSpec((self.num_heads,), role="float32", init="norm")
        if self.value_mix != "none":
            # the source layer's file carries the scalar too, unused
            specs[n["mix"]] = WeightSpec((), role="float32")
        return specs

    def load_weights(self, tensors: Mapping[str, torch.Tensor]) -> None:
        n = self.names

        def by_map(t: torch.Tensor, heads: int) -> torch.Tensor:
            """Rows (or entries) laid out head by head as [map 1, map 2] become all first maps, then all second."""
            if self.maps == 1:
                return t
            return t.reshape(heads, self.maps, self.head_dim, *t.shape[1:]).transpose(0, 1).reshape(t.shape)

        kinds = [("q", self.num_heads)] + ([("k", self.num_kv_heads), ("v", 0)] if self.own_kv else [])
        stacked = [by_map(tensors[n[s]], heads) if heads else tensors[n[s]] for s, heads in kinds]
        if self.output_gate or self.head_gate:
            stacked.append(tensors[n["g"]])
        self.w_in = stack_rows(stacked)
        if self.bias:
            b = torch.cat([by_map(tensors[n[s] + ".b"], heads) if heads else tensors[n[s] + ".b"] for s, heads in kinds])
            self.b_in = torch.cat([b, b.new_zeros(self.w_in.shape[0] - b.shape[0])]).contiguous()
        if self.maps == 2:
            lq1, lk1, lq2, lk2 = (tensors[n[s]].float() for s in ("lq1", "lk1", "lq2", "lk2"))
            self.lam = float(torch.exp((lq1 * lk1).sum()) - torch.exp((lq2 * lk2).sum())) + self.diff
        self.w_o = tensors[n["o"]]
        if self.distance_penalty:
            self.r1, self.r2 = tensors[n["r1"]].contiguous(), tensors[n["r2"]].contiguous()
        if self.value_mix == "mix":
            self.mix = tensors[n["mix"]].reshape(1).contiguous()

    def sub_parts(self) -> dict:
        return {"position": self.position}

    def finalize(self) -> None:
        table = self.position.rotary_table()
        if table is not None and (table.dim > self.head_dim or table.pairing not in ("half", "interleaved")):
            raise ops.KernelArgumentError(f"scored_attention cannot rotate {table.dim} of {self.head_dim} components "
                                          f"with the pairing {table.pairing!r}")
        if table is None and type(self.position).apply is not PositionEncoding.apply:
            raise ops.KernelArgumentError("scored_attention takes a rotary table or no position encoding")

    def cache_spec(self) -> Optional[PagedKVSpec]:
        if not self.own_kv:
            return None   # the schedule hands this layer another entry's cache
        # (a window that keeps its first positions gives no page back while the request runs)
        kept = self.cache_window if self.cache_window is not None else (0 if self.keep_first else self.window)
        return PagedKVSpec(self.num_kv_heads * self.maps, self.head_dim, kept,
                           None if self.value_dim == self.head_dim else self.value_dim,
                           self.num_kv_heads if self.maps > 1 else None)

    def graph_capturable(self, page_size: int) -> bool:
        return True  # a step of single tokens is read through the context's device arrays alone

    def input_weight(self) -> Optional[torch.Tensor]:
        """The matrix of the one product that reads the rows, for whoever stacks it with others'
        (``forward`` then gets the product's result as ``proj``)."""
        return self.w_in

    def release_input_weight(self) -> None:
        self.w_in = None

    def forward(self, x: torch.Tensor, ctx: Any, cache: Any, proj: Optional[torch.Tensor] = None) -> torch.Tensor:
        if cache is None or cache.kind != "paged" or cache.writable != self.own_kv:
            raise RuntimeError("scored_attention needs a paged cache: its own, or with own_kv=False another entry's")
        grp = ctx.groups[cache.group]
        n = x.shape[0]
        if proj is None:
            proj = linear_f32(self.rt, as_operand(self.rt, x, ctx), self.w_in)
        q = self.rt.empty(n, self._q)
        first_in = first_out = None
        if self.value_mix == "source":
            first_out = ctx.memo(("value mix", self.value_mix_key),
                                 lambda: torch.empty(n, self._v, device=self.rt.device, dtype=torch.float32))
        elif self.value_mix == "mix":
            first_in = ctx._memo.get(("value mix", self.value_mix_key))
            if first_in is None or first_in.shape != (n, self._v):
                raise RuntimeError("value mixing needs an earlier layer of the step that keeps its values, of the same size")
        if self.qk_unit:
            ops.qk_unit_cache(proj, 0, self._q, self._q + self._k, q, grp.slots, cache.k_pages, cache.v_pages,
                              self.num_heads, self.norm_eps, mix=self.mix if self.value_mix == "mix" else None,
                              v_first_in=first_in, v_first_out=first_out)
        else:
            table = self.position.rotary_table()
            ops.rotary_cache(proj, 0, self._q, self._q + self._k, ctx.positions, None if table is None else table.inv_freq,
                             0 if table is None else table.dim, table is not None and table.pairing == "interleaved",
                             q, grp.slots if self.own_kv else None, cache.k_pages if self.own_kv else None,
                             cache.v_pages if self.own_kv else None, self.num_heads * self.maps, bias=self.b_in)
        g0 = self._q + self._k + self._v
        if self.maps == 2:
            # each map is a head of its own to the attention kernels; their results stay 32-bit until they are combined
            both = torch.empty(n, 2 * self._o, device=self.rt.device, dtype=torch.float32)
            paged_scored_attention(self.rt, ctx, cache, q, both, 2 * self.num_heads, self.head_dim, self.value_dim, self.scale,
                                   window=self.window, chunk=self.chunk, sink=self.sink, r1=self.r1, r2=self.r2,
                                   keep_first=self.keep_first)
            out = self.rt.empty(n, self._o)
            ops.diff_head_norm(both, self.lam, 1.0 - self.diff, self.norm_eps,
                               proj[:, g0:g0 + self.num_heads] if self.head_gate else None, out, self.num_heads, self.value_dim)
            return linear_f32(self.rt, out, self.w_o)
        out = self.rt.empty(n, self._o)
        gate = proj[:, g0:g0 + self._o] if self.output_gate else None
        paged_scored_attention(self.rt, ctx, cache, q, out, self.num_heads, self.head_dim, self.value_dim, self.scale,
                               gate=gate, window=self.window, chunk=self.chunk, sink=self.sink, r1=self.r1, r2=self.r2,
                               keep_first=self.keep_first)
        return linear_f32(self.rt, out, self.w_o)
