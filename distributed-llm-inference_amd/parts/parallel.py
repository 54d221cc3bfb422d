"""Mixers side by side: every branch reads the same rows, each branch's output is divided by its
root mean square over the model width and multiplied by a weight of its own (a plain weight, not
one plus it), and the result is the mean of the branches (``combine="norm_mean"``); or the result is
the sum of the branches' outputs, each times a constant of its own (``combine="weighted_sum"``, ``scales``).

The branches are mixers of any kind, given as part specs with their own tensor prefixes; each keeps
whatever it keeps per request (pages, a state, nothing), and the pair's cache is the composite of
theirs. Norms, weights and the mean are 32-bit, and so is the result (it is a residual stream's
next summand).

Branches that begin with one product of their rows (``input_weight()`` answers with its matrix, and
``forward`` takes the product's 32-bit result as ``proj``) share one product: their matrices are
stacked at load and each gets its columns of the result."""

from __future__ import annotations

from typing import Any, Mapping, Optional

import torch

from ..kernels import ops
from .base import CompositeCacheSpec, Mixer, Runtime
from .linear import as_operand, linear_f32
from .registry import build_part, register_part
from .spec import PartSpec, WeightSpec


@register_part("mixer", "parallel_mixers")
class ParallelMixers(Mixer):
    MAX_BRANCHES = 4  # what the kernel that normalises and averages takes

    COMBINE = ("norm_mean", "weighted_sum")

    def __init__(self, runtime: Runtime, *, hidden_size: int, branches: Mapping[str, PartSpec], norm_eps: float = 1e-6,
                 out_weight_names: Optional[Mapping[str, str]] = None, combine: str = "norm_mean",
                 scales: Optional[Mapping[str, float]] = None) -> None:
        """``branches``: name -> the branch's mixer. ``out_weight_names``: name -> the tensor (below
        this part's prefix) that multiplies the branch's normalised output; default ``<name>.out``.
        ``combine="weighted_sum"``: no norms and no tensors, ``scales``: name -> the branch's constant."""
        super().__init__(runtime)
        if not 1 <= len(branches) <= self.MAX_BRANCHES:
            raise ValueError(f"one to {self.MAX_BRANCHES} branches, not {len(branches)}")
        if combine not in self.COMBINE:
            raise ValueError(f"combine must be one of {self.COMBINE}")
        if combine == "weighted_sum" and set(scales or {}) != set(branches):
            raise ValueError("a weighted sum needs a scale for every branch")
        self.combine = combine
        self.scales = {n: float(v) for n, v in (scales or {}).items()}
        self.hidden_size, self.norm_eps = hidden_size, float(norm_eps)
        self.names = list(branches)
        self.branches = {name: build_part("mixer", spec, runtime) for name, spec in branches.items()}
        self.out_names = {name: (out_weight_names or {}).get(name, f"{name}.out") for name in self.names}
        self.out_w: dict[str, torch.Tensor] = {}
        self.w_in: Optional[torch.Tensor] = None      # the branches' first products as one
        self.spans: dict[str, tuple[int, int]] = {}

    def sub_parts(self) -> dict:
        return dict(self.branches)

    def weight_specs(self) -> dict[str, WeightSpec]:
        if self.combine == "weighted_sum":
            return {}
        return {self.out_names[n]: WeightSpec((self.hidden_size,), role="float32", init="norm") for n in self.names}

    def load_weights(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.out_w = {n: tensors[self.out_names[n]].contiguous() for n in self.names if self.out_names[n] in tensors}

    def finalize(self) -> None:
        weights = {n: b.input_weight() if hasattr(b, "input_weight") else None for n, b in self.branches.items()}
        if len(weights) < 2 or any(w is None for w in weights.values()):
            return
        at = 0
        for n, w in weights.items():
            self.spans[n] = (at, at + w.shape[0])
            at += w.shape[0]
        self.w_in = torch.cat(list(weights.values()), dim=0).contiguous()
        for b in self.branches.values():
            b.release_input_weight()

    def cache_spec(self) -> Optional[Any]:
        members = tuple((n, b.cache_spec()) for n, b in self.branches.items() if b.cache_spec() is not None)
        if not members:
            return None
        return CompositeCacheSpec(members)

    def graph_capturable(self, page_size: int) -> bool:
        return all(b.graph_capturable(page_size) for b in self.branches.values())

    def forward(self, x: torch.Tensor, ctx: Any, cache: Any) -> torch.Tensor:
        members = cache.members if cache is not None and cache.kind == "composite" else {}
        outs = []
        proj = linear_f32(self.rt, as_operand(self.rt, x, ctx), self.w_in) if self.w_in is not None else None
        for name in self.names:
            if proj is not None:
                a, b = self.spans[name]
                y = self.branches[name].forward(x, ctx, members.get(name), proj=proj[:, a:b])
            else:
                y = self.branches[name].forward(x, ctx, members.get(name))
            if y.dtype != torch.float32:
                wide = torch.empty(y.shape, device=y.device, dtype=torch.float32)
                ops.to_float(y, wide)
                y = wide
            outs.append(y)
        out = torch.empty(x.shape[0], self.hidden_size, device=self.rt.device, dtype=torch.float32)
        if self.combine == "weighted_sum":
            ops.branch_weighted_sum(outs, [self.scales[n] for n in self.names], out)
        else:
            ops.branch_norm_mean(outs, [self.out_w[n] for n in self.names], self.norm_eps, out)
        return out
