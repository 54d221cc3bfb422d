"""RMSNorm: ``w * cast(x * rsqrt(mean(x^2) + eps))`` with 32-bit statistics; eps inside the root,
no bias, no ``1 + w`` (reference: src/dli/model/llama.py:27-44)."""

from __future__ import annotations

from typing import Mapping, Optional

import torch

from ..kernels import ops
from .base import Norm, Runtime
from .registry import register_part
from .spec import WeightSpec


@register_part("norm", "rms_norm")
class RMSNorm(Norm):
    def __init__(self, runtime: Runtime, *, width: int, eps: float, weight_name: str = "weight",
                 unit_offset: bool = False) -> None:
        """``unit_offset``: the checkpoint stores the weight around zero and the norm multiplies by one plus it
        (the sum is made once, at load, in 32-bit; every kernel then sees an ordinary weight)."""
        super().__init__(runtime)
        self.width, self.eps, self.weight_name, self.unit_offset = width, float(eps), weight_name, bool(unit_offset)
        self.weight: torch.Tensor | None = None

    def graph_capturable(self, page_size: int) -> bool:
        return True  # kernels on device arrays only

    def weight_specs(self) -> dict[str, WeightSpec]:
        return {self.weight_name: WeightSpec((self.width,), role="float32", init="zeros" if self.unit_offset else "norm")}

    def load_weights(self, tensors: Mapping[str, torch.Tensor]) -> None:
        w = tensors[self.weight_name]
        self.weight = (w + 1.0).contiguous() if self.unit_offset else w

    def forward_f32(self, x: torch.Tensor) -> torch.Tensor:
        """The norm of a float32 ``x`` as float32 whatever the runtime's type (a norm inside a 32-bit stream)."""
        out = torch.empty_like(x)
        ops.rms_norm_from_f32(x, self.weight, self.eps, out)
        return out

    def fused_params(self) -> tuple[torch.Tensor, float]:
        """Weight and eps, for a consumer that computes this norm inside its own kernel."""
        return self.weight, self.eps

    def native_fields(self) -> Optional[dict]:
        w = self.weight
        if type(self) is not RMSNorm:
            return None  # a subclass computes something else: it must describe itself
        if w is None or w.dtype != torch.float32 or not w.is_cuda or not w.is_contiguous() or w.data_ptr() % 32:
            return None
        return {"kind": "rms_norm", "w": w, "eps": self.eps, "width": self.width}

    def add_normed(self, x: torch.Tensor, y: torch.Tensor, ctx=None) -> None:
        """``x += norm(y)``: the norm on a sublayer's output, added into a 32-bit residual stream
        ``x`` in one kernel (statistics, product and sum in 32-bit; ``y`` float32 or bfloat16). In a
        bfloat16 runtime the kernel leaves the new stream once more in bfloat16 on ``ctx``, for the
        product that reads it next."""
        from .linear import RoundedStream

        rounded = self.rt.empty(*x.shape) if self.rt.is_bf16 and ctx is not None else None
        ops.norm_into_stream(y, self.weight, self.eps, x, rounded=rounded)
        RoundedStream.offer(ctx, x, rounded)

    def post_norm(self, x: torch.Tensor, y: torch.Tensor, alpha: float, ctx=None, gate: Optional[torch.Tensor] = None,
                  gate_bias: Optional[torch.Tensor] = None) -> None:
        """``x <- norm(alpha x + r y)``, ``r = sigmoid(gate + gate_bias)`` or 1: the norm after a residual sum,
        on a 32-bit residual stream ``x`` in one kernel (gate, sum, statistics and product in 32-bit; ``y``
        float32 or bfloat16, ``gate`` float32). In a bfloat16 runtime the kernel leaves the new stream once
        more in bfloat16 on ``ctx``, for the product that reads it next."""
        from .linear import RoundedStream

        rounded = self.rt.empty(*x.shape) if self.rt.is_bf16 and ctx is not None else None
        ops.post_norm_stream(x, y, self.weight, alpha, self.eps, gate=gate, gate_bias=gate_bias, rounded=rounded)
        RoundedStream.offer(ctx, x, rounded)

    def forward(self, x: torch.Tensor, delta: Optional[torch.Tensor] = None) -> torch.Tensor:
        if x.dtype == torch.float32 and self.rt.is_bf16:
            # a 32-bit residual stream in a bfloat16 runtime: normalised in 32-bit and rounded once,
            # to the type that the product after the norm reads
            if delta is not None:
                ops.add(x, delta, x)
            out = self.rt.empty(*x.shape)
            ops.rms_norm_from_f32(x, self.weight, self.eps, out)
            return out
        out = torch.empty_like(x)
        if delta is None:
            ops.rms_norm(x, self.weight, self.eps, out)
        else:
            ops.rms_norm(x, self.weight, self.eps, out, delta=delta, sum_out=x)
        return out


@register_part("norm", "group_rms_norm")
class GroupRMSNorm(Norm):
    """RMS norm in groups, on a 32-bit residual stream: a row is split into ``groups`` equal
    consecutive parts, each is divided by its own ``sqrt(mean(part^2) + eps)``, and the whole is
    multiplied by the weight. Statistics and products are 32-bit; the result is rounded once, to the
    type that the product after the norm reads. ``groups=1`` is the plain RMS norm of such a stream.
    It offers no ``fused_params``: the kernels that compute a norm inside a product compute the plain one."""

    def __init__(self, runtime: Runtime, *, width: int, eps: float, groups: int = 1, weight_name: str = "weight") -> None:
        super().__init__(runtime)
        if groups < 1 or width % groups:
            raise ValueError(f"a row of {width} does not split into {groups} equal parts")
        self.width, self.eps, self.groups, self.weight_name = width, float(eps), int(groups), weight_name
        self.weight: torch.Tensor | None = None

    def graph_capturable(self, page_size: int) -> bool:
        return True  # kernels on device arrays only

    def weight_specs(self) -> dict[str, WeightSpec]:
        return {self.weight_name: WeightSpec((self.width,), role="float32", init="norm")}

    def load_weights(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.weight = tensors[self.weight_name]

    def forward(self, x: torch.Tensor, delta: Optional[torch.Tensor] = None) -> torch.Tensor:
        if x.dtype != torch.float32:
            raise RuntimeError("group_rms_norm normalises a float32 residual stream")
        out = self.rt.empty(*x.shape)
        ops.group_norm(x, self.weight, self.groups, self.eps, out, delta=delta)
        return out
