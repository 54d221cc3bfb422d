"""Mixers that carry a matrix state per head from token to token instead of a cache of keys:
``general_delta`` (a generalized delta rule), ``wkv`` (decayed sums with a bonus for the current
token and token shift), ``gated_delta`` (the delta rule with one decay and one write strength per
head, behind short convolutions), ``gated_linear`` (decayed sums whose forget gate also decides what
is written), ``matrix_memory`` (exponential input and forget gates, one pair a head, with a normaliser) and
``decayed_linear`` (linear attention with a constant decay per head). The state lives in 32-bit in the request's state slot
(:class:`StateSpec`), starts at zero at position 0, and is all that a step leaves for the next.

All run their projections as products of the runtime's type with 32-bit sums, and everything
after them in 32-bit: decays, rates, unit keys, the recurrence, the per-head norm of its output
and the gate (``csrc/recurrent_scan.hip``). The decay's pre-activation is a low-rank projection,
``W2 tanh(W1 h) + w0``, whose second half is 32-bit; its rank is read off the checkpoint's tensor.
"""

from __future__ import annotations

from typing import Any, Mapping, Optional

import torch

from ..kernels import ops
from .base import Mixer, Runtime, StateSpec
from .linear import as_operand, linear_f32, stack_rows
from .registry import register_part
from .spec import WeightSpec


def default_rank(hidden_size: int) -> int:
    """The rank that random-weights mode gives a low-rank projection when nothing names one."""
    return max(8, min(64, hidden_size // 16 // 8 * 8))


class _MatrixStateMixer(Mixer):
    """What the two rules share: sizes, the state, the decay's low-rank projection and the output."""

    rule = -1

    def __init__(self, runtime: Runtime, *, hidden_size: int, num_heads: int, head_dim: int, norm_eps: float = 1e-6,
                 decay_rank: Optional[int] = None) -> None:
        super().__init__(runtime)
        if num_heads < 1 or head_dim < 1:
            raise ValueError("heads and their size must be positive")
        self.hidden_size, self.num_heads, self.head_dim = hidden_size, num_heads, head_dim
        self.norm_eps, self.decay_rank = float(norm_eps), decay_rank
        self.width = num_heads * head_dim
        self.w2t = self.w0 = self.norm_w = self.w_o = None

    def _shared_specs(self) -> dict[str, WeightSpec]:
        h, c = self.hidden_size, self.width
        rank = self.decay_rank if self.decay_rank else -1
        drawn = self.decay_rank or default_rank(h)
        return {"w1": WeightSpec((rank, h), drawn_shape=(drawn, h)),
                "w2": WeightSpec((c, rank), role="float32", drawn_shape=(c, drawn)),
                "w0": WeightSpec((c,), role="float32"), "norm": WeightSpec((c,), role="float32", init="norm"),
                "o": WeightSpec((h, c))}

    def _load_shared(self, tensors: Mapping[str, torch.Tensor]) -> None:
        if tensors["w1"].shape[0] != tensors["w2"].shape[1]:
            raise ValueError(f"{self.prefix}w1 and {self.prefix}w2 disagree on the rank of the decay's projection")
        self.w2t, self.w0 = tensors["w2"].t().contiguous(), tensors["w0"]  # [rank, features]: the kernel's order
        self.norm_w, self.w_o = tensors["norm"], tensors["o"]

    def graph_capturable(self, page_size: int) -> bool:
        return True  # kernels on the context's device arrays only; padding rows write the spare slot

    def _check(self, cache: Any) -> torch.Tensor:
        if cache is None or cache.kind != "state" or not cache.writable:
            raise RuntimeError(f"{self.kind} needs a state of its own")
        if not ops.recurrent_scan_supports(self.head_dim):
            raise ops.KernelArgumentError(f"the recurrence kernel does not take heads of {self.head_dim}")
        return cache.state.view(cache.state.shape[0], -1)


@register_part("mixer", "general_delta")
class GeneralDelta(_MatrixStateMixer):
    """Per head, with ``u = k / sqrt(sum k^2 + 1e-6)``, ``w = exp(-exp(-1/2) sigmoid(W2 tanh(W1 h) + w0))`` and
    ``a = sigmoid(W_a h + b_a)`` per key channel: ``S <- diag(w) S - (a * u)(u^T S) + k v^T`` (both terms read
    the old state), ``o = S^T r``; then ``o / rms(o) * norm * sigmoid(W_g h)`` and the output product."""

    rule = ops.RULE_DELTA

    def weight_specs(self) -> dict[str, WeightSpec]:
        h, c = self.hidden_size, self.width
        specs = {n: WeightSpec((c, h)) for n in ("r", "k", "v", "g", "a")}
        specs["a.b"] = WeightSpec((c,), role="float32")
        specs.update(self._shared_specs())
        return specs

    def load_weights(self, tensors: Mapping[str, torch.Tensor]) -> None:
        # one product for everything that reads h: r, k, v, g, a, and the first half of the decay's
        self.w_in = torch.cat([tensors[n] for n in ("r", "k", "v", "g", "a", "w1")], dim=0).contiguous()
        self.rank = tensors["w1"].shape[0]
        self.a_bias = tensors["a.b"]
        self._load_shared(tensors)

    def cache_spec(self) -> StateSpec:
        return StateSpec((self.num_heads * self.head_dim * self.head_dim,), torch.float32)

    def forward(self, x: torch.Tensor, ctx: Any, cache: Any) -> torch.Tensor:
        state = self._check(cache)
        n, c = x.shape[0], self.width
        proj = linear_f32(self.rt, as_operand(self.rt, x, ctx), self.w_in)
        r, k, v, g, a = (proj[:, i * c:(i + 1) * c] for i in range(5))
        # the decay, and in the same launch the removal rate in place: sigmoid(W_a h + b_a)
        w = torch.empty(n, c, device=self.rt.device, dtype=torch.float32)
        ops.lowrank_out(proj[:, 5 * c:5 * c + self.rank], self.w2t, self.w0, w, act="tanh", out_act="delta_decay",
                        rate=a, rate_bias=self.a_bias)
        out = self.rt.empty(n, c)
        ops.recurrent_scan(r, k, v, w, g, self.norm_w, self.norm_eps, state, ctx.q_start, ctx.positions,
                           ctx.state_slots, out, self.num_heads, self.head_dim, self.rule, a=a)
        return linear_f32(self.rt, out, self.w_o)


@register_part("mixer", "wkv")
class WKV(_MatrixStateMixer):
    """Token shift, then per head ``o = (S + diag(u) k v^T)^T r`` and ``S <- diag(w) S + k v^T`` with
    ``w = exp(-exp(W2 tanh(W1 m_w) + w0))``; r, k, v, the gate and the decay each read a mix of their
    own, ``m_s = h + (h_prev - h) * mu_s``, of the row with the row before it (zeros before position
    0; the last row of a step is kept in the state beside S). Then ``o / rms(o) * norm * silu(W_g m_g)``
    and the output product."""

    rule = ops.RULE_BONUS
    MIXES = ("r", "k", "v", "g", "w")

    def weight_specs(self) -> dict[str, WeightSpec]:
        h, c = self.hidden_size, self.width
        specs = {n: WeightSpec((c, h)) for n in ("r", "k", "v", "g")}
        specs.update({f"mu.{s}": WeightSpec((h,), role="float32") for s in self.MIXES})
        specs["u"] = WeightSpec((self.num_heads, self.head_dim), role="float32")
        specs.update(self._shared_specs())
        return specs

    def load_weights(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.w = {n: tensors[n] for n in ("r", "k", "v", "g")}
        self.w1 = tensors["w1"]
        self.rank = self.w1.shape[0]
        self.mu = torch.stack([tensors[f"mu.{s}"] for s in self.MIXES], dim=0).contiguous()
        self.bonus = tensors["u"].contiguous()
        self._load_shared(tensors)

    def cache_spec(self) -> StateSpec:
        # the row before the next step's first row, then S
        return StateSpec((self.hidden_size + self.num_heads * self.head_dim * self.head_dim,), torch.float32)

    def forward(self, x: torch.Tensor, ctx: Any, cache: Any) -> torch.Tensor:
        state = self._check(cache)
        if x.dtype != torch.float32:
            raise RuntimeError("wkv shifts the rows of a float32 residual stream")
        n, c, h = x.shape[0], self.width, self.hidden_size
        mixes = self.rt.empty(len(self.MIXES), n, h)
        ops.token_shift(x, self.mu, state, ctx.q_start, ctx.positions, ctx.state_slots, mixes)
        proj = torch.empty(n, 4 * c + -(-self.rank // 8) * 8, device=self.rt.device, dtype=torch.float32)
        for i, name in enumerate(("r", "k", "v", "g")):
            linear_f32(self.rt, mixes[i], self.w[name], out=proj[:, i * c:(i + 1) * c])
        linear_f32(self.rt, mixes[4], self.w1, out=proj[:, 4 * c:4 * c + self.rank])
        r, k, v, g = (proj[:, i * c:(i + 1) * c] for i in range(4))
        w = torch.empty(n, c, device=self.rt.device, dtype=torch.float32)
        ops.lowrank_out(proj[:, 4 * c:4 * c + self.rank], self.w2t, self.w0, w, act="tanh", out_act="double_exp_decay")
        out = self.rt.empty(n, c)
        ops.recurrent_scan(r, k, v, w, g, self.norm_w, self.norm_eps, state[:, h:], ctx.q_start, ctx.positions,
                           ctx.state_slots, out, self.num_heads, self.head_dim, self.rule, bonus=self.bonus)
        return linear_f32(self.rt, out, self.w_o)


@register_part("mixer", "gated_delta")
class GatedDelta(Mixer):
    """The gated delta rule. From the rows ``h``: q and k (``num_kv_heads x head_dim``) and v (``num_heads x
    value_dim``) each pass a short causal convolution over time per channel (``conv_taps`` taps, zeros
    before position 0) and silu; q and k become unit vectors per head, ``x / sqrt(sum x^2 + 1e-6)``, q also
    times ``head_dim^-1/2``; value head ``i`` reads q/k head ``i // (num_heads / num_kv_heads)``;
    ``beta = sigmoid(W_b h)`` and ``g = exp(-exp(A_log) softplus(W_a h + dt_bias))`` per head. Per head
    ``S <- g S``, ``u = beta (v - S^T k)``, ``S <- S + k u^T``, ``o = S^T q``; then
    ``o / rms(o) * norm * silu(W_g h)`` (``norm`` of ``value_dim`` values, shared by the heads) and the
    output product. The request's state slot holds ``S`` and the last ``conv_taps - 1`` inputs of the
    convolutions, all 32-bit; everything between the projections and the output product is 32-bit."""

    def __init__(self, runtime: Runtime, *, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 value_dim: int, conv_taps: int = 4, norm_eps: float = 1e-6) -> None:
        super().__init__(runtime)
        if num_heads < 1 or num_kv_heads < 1 or num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads do not group onto {num_kv_heads} q/k heads")
        if head_dim < 1 or value_dim < 1 or not 1 <= conv_taps <= 16:
            raise ValueError("head sizes must be positive and the convolution have 1 to 16 taps")
        self.hidden_size, self.num_heads, self.num_kv_heads = hidden_size, num_heads, num_kv_heads
        self.head_dim, self.value_dim, self.conv_taps, self.norm_eps = head_dim, value_dim, conv_taps, float(norm_eps)
        self.qk, self.hv = num_kv_heads * head_dim, num_heads * value_dim
        self.channels = 2 * self.qk + self.hv
        self.state_floats = num_heads * value_dim * head_dim
        self.w_in = self.conv_w = self.a_log = self.dt_bias = self.norm_w = self.w_o = None

    def weight_specs(self) -> dict[str, WeightSpec]:
        h, t = self.hidden_size, self.conv_taps
        return {"q": WeightSpec((self.qk, h)), "k": WeightSpec((self.qk, h)), "v": WeightSpec((self.hv, h)),
                "q.conv": WeightSpec((self.qk, t), role="float32"),
                "k.conv": WeightSpec((self.qk, t), role="float32"),
                "v.conv": WeightSpec((self.hv, t), role="float32"),
                "b": WeightSpec((self.num_heads, h)), "a": WeightSpec((self.num_heads, h)),
                "A_log": WeightSpec((self.num_heads,), role="float32", init="zeros"),
                "dt_bias": WeightSpec((self.num_heads,), role="float32", init="zeros"),
                "norm": WeightSpec((self.value_dim,), role="float32", init="norm"),
                "g": WeightSpec((self.hv, h)), "o": WeightSpec((h, self.hv))}

    def load_weights(self, tensors: Mapping[str, torch.Tensor]) -> None:
        # one product for everything that reads h: q, k, v (the convolutions' channels, in this order),
        # the gate, beta and the decay
        self.w_in = stack_rows([tensors[n] for n in ("q", "k", "v", "g", "b", "a")])
        self.conv_w = torch.cat([tensors[n] for n in ("q.conv", "k.conv", "v.conv")], dim=0).contiguous()
        self.a_log, self.dt_bias = tensors["A_log"].contiguous(), tensors["dt_bias"].contiguous()
        self.norm_w = tensors["norm"].repeat(self.num_heads).contiguous()   # the kernel reads a value per head and column
        self.w_o = tensors["o"]

    def cache_spec(self) -> StateSpec:
        return StateSpec((self.state_floats + (self.conv_taps - 1) * self.channels,), torch.float32)

    def graph_capturable(self, page_size: int) -> bool:
        return True  # kernels on the context's device arrays only; padding rows write the spare slot

    def input_weight(self) -> Optional[torch.Tensor]:
        """The matrix of the one product that reads the rows, for whoever stacks it with others'
        (``forward`` then gets the product's result as ``proj``)."""
        return self.w_in

    def release_input_weight(self) -> None:
        self.w_in = None

    def forward(self, x: torch.Tensor, ctx: Any, cache: Any, proj: Optional[torch.Tensor] = None) -> torch.Tensor:
        if cache is None or cache.kind != "state" or not cache.writable:
            raise RuntimeError("gated_delta needs a state of its own")
        state = cache.state.view(cache.state.shape[0], -1)
        n, H = x.shape[0], self.num_heads
        if proj is None:
            proj = linear_f32(self.rt, as_operand(self.rt, x, ctx), self.w_in)
        g_off = self.channels
        b_off, a_off = g_off + self.hv, g_off + self.hv + H
        prep = torch.empty(n, self.channels + 2 * H, device=self.rt.device, dtype=torch.float32)
        ops.conv_prepare(proj, b_off, a_off, self.conv_w, self.a_log, self.dt_bias, state, self.state_floats,
                         ctx.q_start, ctx.positions, ctx.state_slots, prep, H, self.num_kv_heads, self.head_dim,
                         self.value_dim)
        o = torch.empty(n, self.hv, device=self.rt.device, dtype=torch.float32)
        ops.gated_delta_scan(prep, state, ctx.q_start, ctx.positions, ctx.state_slots, o, H, self.num_kv_heads,
                             self.head_dim, self.value_dim)
        out = self.rt.empty(n, self.hv)
        ops.head_norm_gate(o, proj[:, g_off:g_off + self.hv], self.norm_w, self.norm_eps, out, H, self.value_dim, gate="silu")
        return linear_f32(self.rt, out, self.w_o)


@register_part("mixer", "gated_linear")
class GatedLinear(Mixer):
    """Linear attention in which the forget gate also decides what is written. From the rows ``h``:
    ``q = silu(W_q h)`` (``num_heads x head_dim``), ``v = W_v h`` (``num_heads x value_dim``), and per head and key
    channel the forget gate ``f = lower + (1 - lower) sigmoid(W_f h + b_f)`` with a lower bound per channel. Per
    head ``S <- diag(f) S + (1 - f) v^T``, ``o = S^T q`` (no key, no scale); then each head's ``o / rms(o) * norm``
    (``norm`` of ``value_dim`` values, shared by the heads) and the output product. The request's state slot
    holds ``S`` in 32-bit; everything between the projections and the output product is 32-bit."""

    def __init__(self, runtime: Runtime, *, hidden_size: int, num_heads: int, head_dim: int, value_dim: Optional[int] = None,
                 norm_eps: float = 1e-6) -> None:
        super().__init__(runtime)
        value_dim = head_dim if value_dim is None else value_dim
        if min(hidden_size, num_heads, head_dim, value_dim) < 1:
            raise ValueError("heads and their sizes must be positive")
        self.hidden_size, self.num_heads, self.head_dim, self.value_dim = hidden_size, num_heads, head_dim, value_dim
        self.norm_eps = float(norm_eps)
        self.hd, self.hv = num_heads * head_dim, num_heads * value_dim
        self.w_in = self.f_bias = self.lower = self.norm_w = self.w_o = None

    def weight_specs(self) -> dict[str, WeightSpec]:
        h = self.hidden_size
        return {"q": WeightSpec((self.hd, h)), "f": WeightSpec((self.hd, h)),
                "f.b": WeightSpec((self.hd,), role="float32", init="zeros"),
                "lower": WeightSpec((self.hd,), role="float32", init="zeros"), "v": WeightSpec((self.hv, h)),
                "norm": WeightSpec((self.value_dim,), role="float32", init="norm"), "o": WeightSpec((h, self.hv))}

    def load_weights(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.w_in = stack_rows([tensors[n] for n in ("q", "f", "v")])   # one product for everything that reads h
        self.f_bias, self.lower = tensors["f.b"].contiguous(), tensors["lower"].contiguous()
        self.norm_w = tensors["norm"].repeat(self.num_heads).contiguous()   # the kernel reads a value per head and column
        self.w_o = tensors["o"]

    def cache_spec(self) -> StateSpec:
        return StateSpec((self.num_heads * self.value_dim * self.head_dim,), torch.float32)

    def graph_capturable(self, page_size: int) -> bool:
        return True  # kernels on the context's device arrays only; padding rows write the spare slot

    def forward(self, x: torch.Tensor, ctx: Any, cache: Any) -> torch.Tensor:
        if cache is None or cache.kind != "state" or not cache.writable:
            raise RuntimeError("gated_linear needs a state of its own")
        state = cache.state.view(cache.state.shape[0], -1)
        n = x.shape[0]
        proj = linear_f32(self.rt, as_operand(self.rt, x, ctx), self.w_in)         # q | f | v
        ops.bounded_gates(proj, 0, self.hd, self.hd, self.f_bias, self.lower)
        o = torch.empty(n, self.hv, device=self.rt.device, dtype=torch.float32)
        ops.gated_linear_scan(proj, 0, self.hd, 2 * self.hd, state, ctx.q_start, ctx.positions, ctx.state_slots, o,
                              self.num_heads, self.head_dim, self.value_dim)
        out = self.rt.empty(n, self.hv)
        ops.head_norm_gate(o, None, self.norm_w, self.norm_eps, out, self.num_heads, self.value_dim, gate="none")
        return linear_f32(self.rt, out, self.w_o)


class _ScalarGateMixer(Mixer):
    """What the recurrences under scalar gates share: ``S <- a S + b k v^T``, ``o = S^T q`` per head with one keep
    factor ``a`` and one write factor ``b`` a token and head (``csrc/scalar_gate_scan.hip``)."""

    def __init__(self, runtime: Runtime, *, hidden_size: int, num_heads: int, head_dim: int, value_dim: Optional[int] = None,
                 norm_eps: float = 1e-6) -> None:
        super().__init__(runtime)
        value_dim = head_dim if value_dim is None else value_dim
        if min(hidden_size, num_heads, head_dim, value_dim) < 1:
            raise ValueError("heads and their sizes must be positive")
        self.hidden_size, self.num_heads, self.head_dim, self.value_dim = hidden_size, num_heads, head_dim, value_dim
        self.norm_eps = float(norm_eps)
        self.hd, self.hv = num_heads * head_dim, num_heads * value_dim
        self.w_in = self.norm_w = self.w_o = None

    def graph_capturable(self, page_size: int) -> bool:
        return True  # kernels on the context's device arrays only; padding rows write the spare slot

    def input_weight(self) -> Optional[torch.Tensor]:
        """The matrix of the one product that reads the rows, for whoever stacks it with others'
        (``forward`` then gets the product's result as ``proj``)."""
        return self.w_in

    def release_input_weight(self) -> None:
        self.w_in = None

    def _state(self, cache: Any) -> torch.Tensor:
        if cache is None or cache.kind != "state" or not cache.writable:
            raise RuntimeError(f"{self.kind} needs a state of its own")
        return cache.state.view(cache.state.shape[0], -1)


@register_part("mixer", "matrix_memory")
class MatrixMemory(_ScalarGateMixer):
    """A matrix memory with exponential gates. From the rows ``h``: ``q = W_q h * head_dim^-1/2`` and ``k = W_k h``
    (``num_heads x head_dim``), ``v = W_v h`` (``num_heads x value_dim``), and per head the log input gate
    ``i = cap tanh((W_i h + b_i) / cap)`` and the log forget gate ``f = logsigmoid(cap tanh((W_f h + b_f) / cap))``
    (``gate_cap`` 0: no cap). With a running reference point ``m`` that starts at 0 (not at minus infinity):
    ``m' = max(f + m, i)``, ``S' = e^(f + m - m') S + e^(i - m') k v^T``, ``n'`` alike from ``k`` alone, and
    ``o = S'^T q / (max(|n' . q|, e^(-m')) + 1e-6)``. Each head's ``o`` is divided by its root mean square, the heads
    side by side are multiplied by ``norm`` (all heads' size) and by ``sigmoid(W_g h)``, then the output product.
    The request's state slot holds ``S`` with ``n`` as one more column a head, then ``m``, all 32-bit; everything
    between the projections and the output product is 32-bit."""

    def __init__(self, runtime: Runtime, *, hidden_size: int, num_heads: int, head_dim: int, value_dim: Optional[int] = None,
                 norm_eps: float = 1e-6, gate_cap: float = 0.0) -> None:
        super().__init__(runtime, hidden_size=hidden_size, num_heads=num_heads, head_dim=head_dim, value_dim=value_dim,
                         norm_eps=norm_eps)
        if gate_cap < 0:
            raise ValueError("the gates' cap must not be negative")
        self.gate_cap = float(gate_cap)
        self.state_floats = num_heads * (self.value_dim + 1) * head_dim
        self.i_bias = self.f_bias = None

    def weight_specs(self) -> dict[str, WeightSpec]:
        h, H = self.hidden_size, self.num_heads
        return {"q": WeightSpec((self.hd, h)), "k": WeightSpec((self.hd, h)), "v": WeightSpec((self.hv, h)),
                "g": WeightSpec((self.hv, h)), "i": WeightSpec((H, h)), "f": WeightSpec((H, h)),
                "i.b": WeightSpec((H,), role="float32", init="zeros"), "f.b": WeightSpec((H,), role="float32", init="zeros"),
                "norm": WeightSpec((self.hv,), role="float32", init="norm"), "o": WeightSpec((h, self.hv))}

    def load_weights(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.w_in = stack_rows([tensors[n] for n in ("q", "k", "v", "g", "i", "f")])   # one product for everything that reads h
        self.i_bias, self.f_bias = tensors["i.b"].contiguous(), tensors["f.b"].contiguous()
        self.norm_w, self.w_o = tensors["norm"].contiguous(), tensors["o"]

    def cache_spec(self) -> StateSpec:
        return StateSpec((self.state_floats + self.num_heads,), torch.float32)

    def forward(self, x: torch.Tensor, ctx: Any, cache: Any, proj: Optional[torch.Tensor] = None) -> torch.Tensor:
        state = self._state(cache)
        n, H = x.shape[0], self.num_heads
        if proj is None:
            proj = linear_f32(self.rt, as_operand(self.rt, x, ctx), self.w_in)
        k0, v0, g0 = self.hd, 2 * self.hd, 2 * self.hd + self.hv
        i0 = g0 + self.hv
        keep, write, floor, log_keep = ops.exp_gates(proj, i0, i0 + H, self.i_bias, self.f_bias, self.gate_cap, state, self.state_floats,
                                           ctx.q_start, ctx.positions, ctx.state_slots, H)
        o = torch.empty(n, self.hv, device=self.rt.device, dtype=torch.float32)
        den = torch.empty(n, H, device=self.rt.device, dtype=torch.float32)
        ops.scalar_gate_scan(proj[:, :k0], proj[:, k0:v0], proj[:, v0:g0], state, ctx.q_start, ctx.positions, ctx.state_slots,
                             o, H, self.head_dim, self.value_dim, keep=keep, write=write, floor=floor, den=den,
                             log_keep=log_keep, q_scale=self.head_dim ** -0.5)
        out = self.rt.empty(n, self.hv)
        ops.head_norm_gate(o, proj[:, g0:g0 + self.hv], self.norm_w, self.norm_eps, out, H, self.value_dim, gate="sigmoid",
                           den=den)
        return linear_f32(self.rt, out, self.w_o)


@register_part("mixer", "decayed_linear")
class DecayedLinear(_ScalarGateMixer):
    """Linear attention with a constant decay per head. From the rows ``h``: ``q = silu(W_q h)`` and
    ``k = silu(W_k h)`` (``num_heads x head_dim``), ``v = silu(W_v h)`` (``num_heads x value_dim``); per head
    ``S <- decay S + k v^T``, ``o = S^T q`` (no other scale). The heads side by side are divided by their root mean
    square over all of them, multiplied by ``norm`` and by ``sigmoid(W_g h)``, then the output product. The
    request's state slot holds ``S`` in 32-bit; everything between the projections and the output product is 32-bit."""

    def __init__(self, runtime: Runtime, *, hidden_size: int, num_heads: int, head_dim: int, decay: Any,
                 value_dim: Optional[int] = None, norm_eps: float = 1e-6) -> None:
        super().__init__(runtime, hidden_size=hidden_size, num_heads=num_heads, head_dim=head_dim, value_dim=value_dim,
                         norm_eps=norm_eps)
        self.decay_values = [float(d) for d in decay]
        if len(self.decay_values) != num_heads:
            raise ValueError(f"{len(self.decay_values)} decays for {num_heads} heads")
        self.decay: Optional[torch.Tensor] = None

    def weight_specs(self) -> dict[str, WeightSpec]:
        h = self.hidden_size
        return {"q": WeightSpec((self.hd, h)), "k": WeightSpec((self.hd, h)), "v": WeightSpec((self.hv, h)),
                "g": WeightSpec((self.hv, h)), "norm": WeightSpec((self.hv,), role="float32", init="norm"),
                "o": WeightSpec((h, self.hv))}

    def load_weights(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.w_in = stack_rows([tensors[n] for n in ("q", "k", "v", "g")])   # one product for everything that reads h
        self.norm_w, self.w_o = tensors["norm"].contiguous(), tensors["o"]

    def finalize(self) -> None:
        self.decay = torch.tensor(self.decay_values, dtype=torch.float32, device=self.rt.device)

    def cache_spec(self) -> StateSpec:
        return StateSpec((self.num_heads * self.value_dim * self.head_dim,), torch.float32)

    def forward(self, x: torch.Tensor, ctx: Any, cache: Any, proj: Optional[torch.Tensor] = None) -> torch.Tensor:
        state = self._state(cache)
        n = x.shape[0]
        if proj is None:
            proj = linear_f32(self.rt, as_operand(self.rt, x, ctx), self.w_in)
        if self.decay is None:
            self.finalize()
        k0, v0, g0 = self.hd, 2 * self.hd, 2 * self.hd + self.hv
        o = torch.empty(n, self.hv, device=self.rt.device, dtype=torch.float32)
        # a step of single tokens applies silu inside the scan; one with portions beforehand, all threads at once
        # (inside, it would sit on the one wave that walks a request's tokens)
        inside = ctx.num_decode == ctx.num_entries
        if not inside:
            ops.silu_columns(proj[:, :g0])
        ops.scalar_gate_scan(proj[:, :k0], proj[:, k0:v0], proj[:, v0:g0], state, ctx.q_start, ctx.positions, ctx.state_slots,
                             o, self.num_heads, self.head_dim, self.value_dim, decay=self.decay, silu=inside)
        out = self.rt.empty(n, self.hv)
        # one norm over all heads: the row as a single head
        ops.head_norm_gate(o, proj[:, g0:g0 + self.hv], self.norm_w, self.norm_eps, out, 1, self.hv, gate="sigmoid")
        return linear_f32(self.rt, out, self.w_o)
