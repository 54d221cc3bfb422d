"""A mixture of small feed-forward experts behind a router.

Router: ``z = W_router h`` (``+ b_router`` with ``router_bias``) in 32-bit over ``experts + identity`` outputs, scores
``s = softmax(z)``. The
choice scores add a per-output ``correction`` (the weights do not). The outputs form ``groups`` equal
groups of neighbours; a group's score is its largest choice score, and only outputs of the best
``groups_kept`` groups can be chosen. The ``top`` largest choice scores are chosen; their weights are
their scores ``s`` divided by their sum (+ 1e-20), times ``scale`` (with ``scale = 1`` and without correction and
groups that is the softmax over the chosen logits alone). The last ``identity`` outputs are
identity experts: their result is the input itself; they have no tensors.

Expert ``e`` (tensors ``e<e>.gate``, ``e<e>.up``, ``e<e>.down``, no biases): ``g = min(W_gate h, limit)``,
``u = clamp(W_up h, -limit, limit)``, ``y = g sigmoid(alpha g) (u + up_shift)``, result ``W_down y`` (an infinite
limit, ``alpha = 1`` and ``up_shift = 0``: the plain ``silu(W_gate h) * (W_up h)``). A shared
expert of the same form (its own size and limit) may run for every token; it is added multiplied by
``sigmoid(W_sg h)``, one number per token, or as it is (``shared_gate=False``).

``routing="table"``: no router; an integer tensor ``table [vocabulary, top]`` names each token id's experts (the
entries of a row differ), each with the weight ``1 / top``.

Order of work: one 32-bit product for the router (and the shared expert's gate: its row is stacked
below the router's); the choice kernel; on the device the chosen (token, expert) pairs are sorted by
expert and cut into row tiles, over which two kernels run the experts' products (nothing waits
for the device, so a step of single tokens can be recorded); the shared expert's two plain products;
one kernel adds everything up in 32-bit. The expert matrices are stacked ``[experts, ...]`` at load.
"""

from __future__ import annotations

from typing import Any, Mapping

import torch

from ..kernels import ops
from .base import FeedForward, Runtime
from .linear import linear, linear_f32, stack_rows
from .registry import register_part
from .spec import WeightSpec


@register_part("feed_forward", "routed_experts")
class RoutedExperts(FeedForward):
    def __init__(self, runtime: Runtime, *, hidden_size: int, experts: int, top: int, expert_size: int,
                 limit: float, alpha: float = 1.702, identity: int = 0, groups: int = 1, groups_kept: int = 1,
                 scale: float = 1.0, correction: bool = True, shared_size: int = 0, shared_limit: float = 0.0,
                 shared_gate: bool = True, up_shift: float = 1.0, router_bias: bool = False, routing: str = "router",
                 vocab_size: int = 0) -> None:
        super().__init__(runtime)
        if routing not in ("router", "table"):
            raise ValueError(f"routing must be 'router' or 'table', not {routing!r}")
        if routing == "table" and (identity or vocab_size < 1 or shared_gate and shared_size):
            raise ValueError("a table names real experts for every id of a vocabulary; a shared expert's gate needs a router")
        self.routing, self.vocab_size, self.table = routing, int(vocab_size), None
        total = experts + identity
        if experts < 0 or identity < 0 or total < 1 or not 1 <= top <= min(total, 64):
            raise ValueError(f"{top} of {experts} experts and {identity} identity experts cannot be chosen")
        if groups < 1 or total % groups or not 1 <= groups_kept <= groups or groups_kept * (total // groups) < top:
            raise ValueError(f"{total} router outputs in {groups} groups of which {groups_kept} are kept do not give {top} choices")
        if experts and expert_size < 1:
            raise ValueError("experts need a size")
        self.hidden_size, self.experts, self.identity, self.total, self.top = hidden_size, experts, identity, total, top
        self.expert_size, self.limit, self.alpha = expert_size, float(limit), float(alpha)
        self.groups, self.groups_kept, self.scale = groups, groups_kept, float(scale)
        self.has_correction, self.has_router_bias, self.up_shift = bool(correction), bool(router_bias), float(up_shift)
        self.shared_size, self.shared_limit = int(shared_size), float(shared_limit)
        self.shared_gate = bool(shared_gate) and self.shared_size > 0
        self.w_router = self.router_bias = self.correction = self.w_gate = self.w_up = self.w_down = None
        self.ws_gate_up = self.ws_down = None

    def graph_capturable(self, page_size: int) -> bool:
        return True  # kernels on device arrays only; the rows are sorted by expert on the device

    def weight_specs(self) -> dict[str, WeightSpec]:
        h, f = self.hidden_size, self.expert_size
        if self.routing == "table":
            specs = {"table": WeightSpec((self.vocab_size, self.top), role="int32", init=f"distinct_below:{self.experts}")}
        else:
            specs = {"router": WeightSpec((self.total, h))}
        if self.routing == "router" and self.has_router_bias:
            specs["router.b"] = WeightSpec((self.total,), role="float32", init="zeros")
        if self.routing == "router" and self.has_correction:
            specs["correction"] = WeightSpec((self.total,), role="float32", init="zeros", optional=True)
        for e in range(self.experts):
            specs.update({f"e{e}.gate": WeightSpec((f, h)), f"e{e}.up": WeightSpec((f, h)), f"e{e}.down": WeightSpec((h, f))})
        if self.shared_size:
            s = self.shared_size
            specs.update({"shared.gate": WeightSpec((s, h)), "shared.up": WeightSpec((s, h)), "shared.down": WeightSpec((h, s))})
            if self.shared_gate:
                specs["shared.sg"] = WeightSpec((1, h))
        return specs

    def load_weights(self, tensors: Mapping[str, torch.Tensor]) -> None:
        if self.routing == "table":
            self.table = tensors["table"].contiguous()
            if self.table.numel() and not (0 <= int(self.table.min()) and int(self.table.max()) < self.experts):
                raise ValueError(f"{self.prefix}table names experts outside 0..{self.experts - 1}")
        else:
            rows = [tensors["router"]] + ([tensors["shared.sg"]] if self.shared_gate else [])
            self.w_router = stack_rows(rows)
            self.router_bias = tensors["router.b"].contiguous() if self.has_router_bias else None
            # (a checkpoint without the tensor: scores are chosen as they are)
            self.correction = tensors["correction"].contiguous() if self.has_correction and "correction" in tensors else None
        if self.experts:
            self.w_gate = torch.stack([tensors[f"e{e}.gate"] for e in range(self.experts)]).contiguous()
            self.w_up = torch.stack([tensors[f"e{e}.up"] for e in range(self.experts)]).contiguous()
            self.w_down = torch.stack([tensors[f"e{e}.down"] for e in range(self.experts)]).contiguous()
        if self.shared_size:
            self.ws_gate_up = torch.cat([tensors["shared.gate"], tensors["shared.up"]], dim=0).contiguous()
            self.ws_down = tensors["shared.down"]

    def forward(self, x: torch.Tensor, ctx: Any) -> torch.Tensor:
        n, dev = x.shape[0], self.rt.device
        ids = torch.empty(n, self.top, device=dev, dtype=torch.int32)
        weights = torch.empty(n, self.top, device=dev, dtype=torch.float32)
        if self.routing == "table":
            logits = None
            ops.table_choose(self.table, ctx.token_ids, ids, weights)
        else:
            logits = linear_f32(self.rt, x, self.w_router)
            ops.router_choose(logits, self.total, self.correction, self.groups, self.groups_kept, self.top, self.scale, ids,
                              weights, bias=self.router_bias)
        z = None
        if self.experts:
            z = ops.expert_products(ids, x, self.w_gate, self.w_up, self.w_down, self.limit, self.alpha, self.up_shift)
        shared = gate = None
        if self.shared_size:
            gate_up = linear(self.rt, x, self.ws_gate_up)
            act = self.rt.empty(n, self.shared_size)
            ops.clamped_glu(gate_up, act, self.shared_limit, self.alpha, self.up_shift)
            shared = linear_f32(self.rt, act, self.ws_down)
            if self.shared_gate:
                gate = logits[:, self.total:self.total + 1]
        out = torch.empty(n, self.hidden_size, device=dev, dtype=torch.float32)
        ops.expert_combine(ids, weights, z, x, self.experts, out, shared=shared, shared_gate=gate)
        return out
