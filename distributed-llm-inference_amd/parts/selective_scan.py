"""The selective scan as a mixer (``selective_scan``): a diagonal recurrence per channel whose step size,
input and output maps depend on the token.

From the rows ``h``: ``W_in h`` is ``x`` and ``z``, ``inner_size`` channels each. ``x`` passes a short causal
convolution per channel (``conv_taps`` taps with a bias, zeros before position 0) and silu. ``W_x x`` is
``dt_low`` (``dt_rank``), ``B`` and ``C`` (``state_size`` each); the step size of a channel is
``dt = softplus(W_dt dt_low + b_dt)``; ``A = -exp(A_log)``, ``inner_size x state_size``. Per channel ``c`` and
state ``n``: ``S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n``, ``y_c = sum_n S[c, n] C_n + D_c x_c``; the result is
``W_o (y * silu(z))``.

The request's state slot holds ``S`` and the convolution's last ``conv_taps - 1`` inputs, all 32-bit. The
products read the runtime's type and leave 32-bit sums; the convolution, the step sizes (the second half
of their low-rank projection included), the decays, the recurrence and the gate are 32-bit."""

from __future__ import annotations

from typing import Any, Mapping

import torch

from ..kernels import ops
from .base import Mixer, Runtime, StateSpec
from .linear import as_operand, linear_f32, stack_rows
from .registry import register_part
from .spec import WeightSpec


@register_part("mixer", "selective_scan")
class SelectiveScan(Mixer):
    def __init__(self, runtime: Runtime, *, hidden_size: int, inner_size: int, state_size: int, dt_rank: int,
                 conv_taps: int = 4) -> None:
        super().__init__(runtime)
        if min(hidden_size, inner_size, state_size, dt_rank) < 1 or not 1 <= conv_taps <= 16:
            raise ValueError("sizes must be positive and the convolution have 1 to 16 taps")
        if state_size > 256:
            raise ops.KernelArgumentError(f"the selective scan keeps up to 256 states a channel, not {state_size}")
        self.hidden_size, self.inner, self.states, self.dt_rank, self.taps = hidden_size, inner_size, state_size, dt_rank, conv_taps
        self.state_floats = inner_size * state_size
        self.w_in = self.w_x = self.w_dt_t = self.dt_bias = self.conv_w = self.conv_b = None
        self.a_log = self.d = self.w_o = None

    def weight_specs(self) -> dict[str, WeightSpec]:
        h, c, n, r = self.hidden_size, self.inner, self.states, self.dt_rank
        return {"in": WeightSpec((2 * c, h)), "conv": WeightSpec((c, self.taps), role="float32"),
                "conv.b": WeightSpec((c,), role="float32", init="zeros"), "x": WeightSpec((r + 2 * n, c)),
                "dt": WeightSpec((c, r), role="float32"), "dt.b": WeightSpec((c,), role="float32", init="zeros"),
                "A_log": WeightSpec((c, n), role="float32", init="zeros"), "D": WeightSpec((c,), role="float32", init="ones"),
                "o": WeightSpec((h, c))}

    def load_weights(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.w_in, self.w_x = stack_rows([tensors["in"]]), stack_rows([tensors["x"]])
        self.conv_w, self.conv_b = tensors["conv"].contiguous(), tensors["conv.b"].contiguous()
        self.w_dt_t, self.dt_bias = tensors["dt"].t().contiguous(), tensors["dt.b"].contiguous()   # [rank, channels]
        self.a_log, self.d, self.w_o = tensors["A_log"].contiguous(), tensors["D"].contiguous(), tensors["o"]

    def cache_spec(self) -> StateSpec:
        return StateSpec((self.state_floats + (self.taps - 1) * self.inner,), torch.float32)

    def graph_capturable(self, page_size: int) -> bool:
        return True  # kernels on the context's device arrays only; padding rows write the spare slot

    def forward(self, x: torch.Tensor, ctx: Any, cache: Any) -> torch.Tensor:
        if cache is None or cache.kind != "state" or not cache.writable:
            raise RuntimeError("selective_scan needs a state of its own")
        state = cache.state.view(cache.state.shape[0], -1)
        n, c, dev = x.shape[0], self.inner, self.rt.device
        proj = linear_f32(self.rt, as_operand(self.rt, x, ctx), self.w_in)          # x | z
        xc = torch.empty(n, c, device=dev, dtype=torch.float32)
        operand = self.rt.empty(n, c) if self.rt.is_bf16 else None                  # what the next product reads
        ops.causal_conv(proj, self.conv_w, self.conv_b, state, self.state_floats, ctx.q_start, ctx.positions,
                        ctx.state_slots, xc, rounded=operand, act="silu")
        low = linear_f32(self.rt, xc if operand is None else operand, self.w_x)     # dt_low | B | C
        dt = torch.empty(n, c, device=dev, dtype=torch.float32)
        ops.lowrank_out(low[:, :self.dt_rank], self.w_dt_t, self.dt_bias, dt, act="none", out_act="softplus")
        out = self.rt.empty(n, c)
        ops.selective_scan(xc, dt, low, self.dt_rank, self.dt_rank + self.states, proj[:, c:2 * c], self.a_log, self.d,
                           state, ctx.q_start, ctx.positions, ctx.state_slots, out)
        return linear_f32(self.rt, out, self.w_o)
