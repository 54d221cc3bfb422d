"""Token shift in front of any mixer: what the mixer reads is ``h + (h_prev - h) * mu`` element by element,
``h_prev`` being the row of the token before (as it was before this replacement; zeros before position 0).
The last row of a step is kept in the request's state, so the wrapper's cache is the composite of that
row and whatever the inner mixer keeps (pages, a state, nothing).

The rows are a 32-bit residual stream; the mix is 32-bit and goes out in the type that the inner mixer's
products read."""

from __future__ import annotations

from typing import Any, Mapping, Optional

import torch

from ..kernels import ops
from .base import CompositeCacheSpec, Mixer, Runtime, StateSpec
from .registry import build_part, register_part
from .spec import PartSpec, WeightSpec


@register_part("mixer", "token_shifted")
class TokenShifted(Mixer):
    def __init__(self, runtime: Runtime, *, hidden_size: int, inner: PartSpec, weight_name: str = "mu") -> None:
        """``inner``: the mixer behind the shift, with its own tensor prefix. ``weight_name``: the tensor
        (below this part's prefix) that holds ``mu``, one value per column."""
        super().__init__(runtime)
        self.hidden_size, self.weight_name = hidden_size, weight_name
        self.inner = build_part("mixer", inner, runtime)
        if isinstance(self.inner.cache_spec(), CompositeCacheSpec):
            raise ValueError("token_shifted takes an inner mixer that keeps one cache, not a composite")
        self.mu: Optional[torch.Tensor] = None

    def sub_parts(self) -> dict:
        return {"inner": self.inner}

    def weight_specs(self) -> dict[str, WeightSpec]:
        return {self.weight_name: WeightSpec((self.hidden_size,), role="float32", init="zeros")}

    def load_weights(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.mu = tensors[self.weight_name].reshape(1, self.hidden_size).contiguous()

    def cache_spec(self) -> CompositeCacheSpec:
        members = [("shift", StateSpec((self.hidden_size,), torch.float32))]
        inner = self.inner.cache_spec()
        if inner is not None:
            members.append(("inner", inner))
        return CompositeCacheSpec(tuple(members))

    def graph_capturable(self, page_size: int) -> bool:
        return self.inner.graph_capturable(page_size)

    def forward(self, x: torch.Tensor, ctx: Any, cache: Any) -> torch.Tensor:
        if cache is None or cache.kind != "composite" or not cache.writable:
            raise RuntimeError("token_shifted needs a cache of its own for the kept row")
        if x.dtype != torch.float32:
            raise RuntimeError("token_shifted shifts the rows of a float32 residual stream")
        kept = cache.members["shift"].state
        mixed = self.rt.empty(1, x.shape[0], self.hidden_size)
        ops.token_shift(x, self.mu, kept.view(kept.shape[0], -1), ctx.q_start, ctx.positions, ctx.state_slots, mixed)
        return self.inner.forward(mixed[0], ctx, cache.members.get("inner"))
