"""Pre-norm arrangement: ``x + mixer(norm(x))`` then ``x + feed_forward(norm(x))``
(reference: src/dli/model/llama.py:194-213). The residual sums are made inside the norms that
follow them (32-bit sum, rounded to the activation type, then normalised). A layer may have no
feed-forward; the stream may be 32-bit in a bfloat16 runtime (an embedding that hands out float32
rows, parts that return their 32-bit sums), in which case nothing of it is ever rounded."""

from __future__ import annotations

from typing import Any, Mapping, Optional

import torch

from .base import Block, DecodeStream, Part, Runtime
from .linear import as_operand
from .registry import register_part


@register_part("block", "pre_norm")
class PreNormBlock(Block):
    roles = ("mixer_norm", "mixer")   # and, unless the layer has no feed-forward, "feed_forward_norm" and "feed_forward"

    def __init__(self, runtime: Runtime) -> None:
        super().__init__(runtime)

    def graph_capturable(self, page_size: int) -> bool:
        return True  # kernels on device arrays only

    def forward(self, x: torch.Tensor, delta: Optional[torch.Tensor], ctx: Any, cache: Any,
                parts: Mapping[str, Part]) -> tuple[torch.Tensor, Optional[torch.Tensor]]:
        h = parts["mixer_norm"].forward(x, delta)          # x <- x + delta
        a = parts["mixer"].forward(h, ctx, cache)
        if "feed_forward" not in parts:
            return x, a
        h = parts["feed_forward_norm"].forward(x, a)       # x <- x + a
        f = parts["feed_forward"].forward(h, ctx)
        return x, f

    # the arrangement of parts that the loop in C implements (``DLI_BLOCK_PRENORM_RMS_GQA_SILU``)
    NATIVE_KIND = 1
    NATIVE_PARTS = {"mixer_norm": "rms_norm", "mixer": "gqa_rotary_half", "feed_forward_norm": "rms_norm",
                    "feed_forward": "gated_silu"}

    def native_fields(self, parts: Mapping[str, Part]) -> Optional[dict]:
        """This arrangement with its parts' tensors and constants, for the loop in C that issues a
        step's launches. That loop hard-codes one order of work, so the answer is ``None`` unless
        this is exactly this class (a subclass must describe itself), each of the four parts
        names exactly the kind that the loop computes, and all agree on the width."""
        if type(self) is not PreNormBlock or any(role not in parts for role in self.NATIVE_PARTS):
            return None
        fields = {role: parts[role].native_fields() for role in self.NATIVE_PARTS}
        if any(f is None or f.get("kind") != self.NATIVE_PARTS[role] for role, f in fields.items()):
            return None
        n1, n2, mix, ff = (fields[r] for r in ("mixer_norm", "feed_forward_norm", "mixer", "feed_forward"))
        if not n1["width"] == n2["width"] == mix["hidden"] == ff["hidden"]:
            return None
        return {**mix, **ff, "kind": self.NATIVE_KIND, "norm1_w": n1["w"], "eps1": n1["eps"], "norm2_w": n2["w"],
                "eps2": n2["eps"]}

    def streams(self, ctx: Any, parts: Mapping[str, Part]) -> bool:
        if "feed_forward" not in parts:
            return False
        fused_norms = all(hasattr(parts[r], "fused_params") for r in ("mixer_norm", "feed_forward_norm"))
        return fused_norms and parts["mixer"].streams(ctx) and parts["feed_forward"].streams(ctx)

    def first_norm(self, parts: Mapping[str, Part]) -> Optional[Part]:
        return parts["mixer_norm"]

    def forward_stream(self, stream: DecodeStream, ctx: Any, cache: Any, parts: Mapping[str, Part],
                       following: Optional[Part] = None) -> None:
        """``following``: the norm that whatever comes after this block applies first (the last
        kernel of the block may apply it while it writes the stream)."""
        parts["mixer"].forward_stream(stream, parts["mixer_norm"], ctx, cache, following=parts["feed_forward_norm"])
        parts["feed_forward"].forward_stream(stream, parts["feed_forward_norm"], ctx, following=following)


@register_part("block", "output_norm")
class OutputNormBlock(Block):
    """Norms on the sublayers' outputs only, around a 32-bit residual stream:
    ``x <- x + norm1(mixer(x))``, then ``x <- x + norm2(feed_forward(x))``; the sublayers read ``x``
    itself. The feed-forward and its norm may be absent. ``x`` is float32 in both runtimes; each
    norm is applied and added into the stream by one kernel (``Norm.add_normed``). The mixer gets
    the stream as it is (what it feeds to its products it rounds itself); the feed-forward gets it
    in the type that its products read."""

    roles = ("mixer", "mixer_norm")

    def __init__(self, runtime: Runtime) -> None:
        super().__init__(runtime)

    def graph_capturable(self, page_size: int) -> bool:
        return True  # kernels on device arrays only

    def forward(self, x: torch.Tensor, delta: Optional[torch.Tensor], ctx: Any, cache: Any,
                parts: Mapping[str, Part]) -> tuple[torch.Tensor, Optional[torch.Tensor]]:
        if x.dtype != torch.float32:
            raise RuntimeError("the output_norm block keeps a float32 residual stream")
        if delta is not None:
            from ..kernels import ops
            from .linear import RoundedStream
            ops.add(x, delta, x)
            RoundedStream.offer(ctx, x, None)
        parts["mixer_norm"].add_normed(x, parts["mixer"].forward(x, ctx, cache), ctx)
        if "feed_forward" in parts:
            y = parts["feed_forward"].forward(as_operand(self.rt, x, ctx), ctx)
            parts["feed_forward_norm"].add_normed(x, y, ctx)
        return x, None


@register_part("block", "post_norm")
class PostNormBlock(Block):
    """Norms after the residual sums, around a 32-bit residual stream:
    ``x <- norm1(alpha x + r1 * mixer(x))``, then ``x <- norm2(alpha x + r2 * feed_forward(x))``; the sublayers
    read ``x`` itself. With ``gated`` each sublayer's result is multiplied element by element by
    ``r = sigmoid(W x + b)`` before the sum (tensors ``rg1``, ``rg1.b`` for the mixer and ``rg2``, ``rg2.b`` for
    the feed-forward, below this block's prefix; ``W`` reads the same ``x`` as the sublayer); without,
    ``r = 1``. The feed-forward and its norm may be absent. ``x`` is float32 in both runtimes; gate, sum and
    norm are one kernel (``Norm.post_norm``). The mixer gets the stream as it is (what it feeds to its
    products it rounds itself); the feed-forward gets it in the type that its products read."""

    roles = ("mixer", "mixer_norm")

    def __init__(self, runtime: Runtime, *, hidden_size: int, alpha: float = 1.0, gated: bool = False,
                 feed_forward: bool = True, names: Optional[Mapping[str, str]] = None) -> None:
        super().__init__(runtime)
        self.hidden_size, self.alpha, self.gated, self.has_ff = hidden_size, float(alpha), bool(gated), bool(feed_forward)
        self.names = {"mixer": "rg1", "feed_forward": "rg2", **dict(names or {})}
        self.w: dict[str, torch.Tensor] = {}
        self.b: dict[str, torch.Tensor] = {}

    def graph_capturable(self, page_size: int) -> bool:
        return True  # kernels on device arrays only

    def _gates(self) -> list[str]:
        return [] if not self.gated else ["mixer"] + (["feed_forward"] if self.has_ff else [])

    def weight_specs(self) -> dict:
        from .spec import WeightSpec

        h, specs = self.hidden_size, {}
        for role in self._gates():
            specs[self.names[role]] = WeightSpec((h, h))
            specs[self.names[role] + ".b"] = WeightSpec((h,), role="float32", init="zeros")
        return specs

    def load_weights(self, tensors: Mapping[str, torch.Tensor]) -> None:
        for role in self._gates():
            self.w[role] = tensors[self.names[role]]
            self.b[role] = tensors[self.names[role] + ".b"].contiguous()

    def _gate(self, role: str, operand: torch.Tensor) -> tuple[Optional[torch.Tensor], Optional[torch.Tensor]]:
        if not self.gated:
            return None, None
        from .linear import linear_f32

        return linear_f32(self.rt, operand, self.w[role]), self.b[role]

    def forward(self, x: torch.Tensor, delta: Optional[torch.Tensor], ctx: Any, cache: Any,
                parts: Mapping[str, Part]) -> tuple[torch.Tensor, Optional[torch.Tensor]]:
        if x.dtype != torch.float32:
            raise RuntimeError("the post_norm block keeps a float32 residual stream")
        if delta is not None:
            from ..kernels import ops
            from .linear import RoundedStream
            ops.add(x, delta, x)
            RoundedStream.offer(ctx, x, None)
        g, b = self._gate("mixer", as_operand(self.rt, x, ctx))
        y = parts["mixer"].forward(x, ctx, cache)
        parts["mixer_norm"].post_norm(x, y, self.alpha, ctx, gate=g, gate_bias=b)
        if "feed_forward" in parts:
            h = as_operand(self.rt, x, ctx)
            g, b = self._gate("feed_forward", h)
            y = parts["feed_forward"].forward(h, ctx)
            parts["feed_forward_norm"].post_norm(x, y, self.alpha, ctx, gate=g, gate_bias=b)
        return x, None


@register_part("block", "parallel_norms")
class ParallelNormsBlock(Block):
    """Mixer and feed-forward side by side, each behind a norm of its own, both reading the same stream:
    ``x <- x + (mixer(norm1(x)) + feed_forward(norm2(x)))`` around a 32-bit residual stream. The feed-forward and
    its norm may be absent. ``x`` is float32 in both runtimes; the norms round once, to the type that the
    products read; the two results are added to each other and then into the stream, in 32-bit."""

    roles = ("mixer_norm", "mixer")   # and, unless the layer has no feed-forward, "feed_forward_norm" and "feed_forward"

    def __init__(self, runtime: Runtime) -> None:
        super().__init__(runtime)

    def graph_capturable(self, page_size: int) -> bool:
        return True  # kernels on device arrays only

    def forward(self, x: torch.Tensor, delta: Optional[torch.Tensor], ctx: Any, cache: Any,
                parts: Mapping[str, Part]) -> tuple[torch.Tensor, Optional[torch.Tensor]]:
        from ..kernels import ops

        if x.dtype != torch.float32:
            raise RuntimeError("the parallel_norms block keeps a float32 residual stream")
        if delta is not None:
            ops.add(x, delta, x)
        if "feed_forward" not in parts:
            ops.add(x, _as_f32(parts["mixer"].forward(parts["mixer_norm"].forward(x), ctx, cache)), x)
            return x, None
        n1, n2 = parts["mixer_norm"], parts["feed_forward_norm"]
        pair = [getattr(n, "fused_params", None) for n in (n1, n2)]
        if all(pair) and pair[0]()[1] == pair[1]()[1]:
            # plain RMS norms that agree on eps: one pass over the rows' statistics for both
            h1, h2 = self.rt.empty(*x.shape), self.rt.empty(*x.shape)
            ops.rms_norm_pair(x, pair[0]()[0], pair[1]()[0], pair[0]()[1], h1, h2)
        else:
            h1, h2 = n1.forward(x), n2.forward(x)
        y = _as_f32(parts["mixer"].forward(h1, ctx, cache))
        f = _as_f32(parts["feed_forward"].forward(h2, ctx))
        ops.add_pair_into_stream(x, y, f)
        return x, None


def _as_f32(y: torch.Tensor) -> torch.Tensor:
    if y.dtype == torch.float32:
        return y
    from ..kernels import ops

    wide = torch.empty(y.shape, device=y.device, dtype=torch.float32)
    ops.to_float(y, wide)
    return wide
