"""Attention through a latent (``latent_attention``): per token one normalised vector ``c`` of ``kv_rank`` values
is cached, and every head's keys and values are linear maps of it.

From the rows ``h``: ``c_q = norm(W_dq h)`` (RMS norm with a weight), ``q = W_uq c_q`` (``num_heads x head_dim``);
``c = norm(W_dkv h)``. Head ``i`` has ``k = U_i c`` and ``v = V_i c`` (the rows of ``W_uk`` and ``W_uv`` that belong to
it), scores ``scale (q_i . k)`` over every earlier position and itself, an ordinary softmax, and with
``output_gate`` the concatenated heads are multiplied by ``sigmoid(W_g h)`` before the output product. There
are no positions in it.

Since ``q_i . (U_i c) = (U_i^T q_i) . c`` and ``sum_j p_j V_i c_j = V_i (sum_j p_j c_j)``, the attention runs over the
cached latents themselves, as one kv head shared by all query heads whose values are its keys, between
two small products per head: ``q'_i = U_i^T q_i`` before and ``V_i (.)`` after. The cache is a group of pages
with one kv head of ``kv_rank`` (the latent lies there as a key and, in the value pages' order, as a value);
the attention kernels are those of :mod:`dli_amd.parts.scored_attention`.

Norms, scores and weights are 32-bit; the products read the runtime's type with 32-bit sums."""

from __future__ import annotations

from typing import Any, Mapping, Optional

import torch

from ..kernels import ops
from .base import Mixer, PagedKVSpec, Runtime
from .linear import as_operand, linear, linear_f32, stack_rows
from .registry import register_part
from .scored_attention import paged_scored_attention
from .spec import WeightSpec


@register_part("mixer", "latent_attention")
class LatentAttention(Mixer):
    def __init__(self, runtime: Runtime, *, hidden_size: int, num_heads: int, head_dim: int, kv_rank: int, q_rank: int,
                 value_dim: Optional[int] = None, scale: Optional[float] = None, norm_eps: float = 1e-6,
                 output_gate: bool = False, window: int = 0) -> None:
        super().__init__(runtime)
        value_dim = head_dim if value_dim is None else value_dim
        if min(num_heads, head_dim, value_dim, kv_rank, q_rank) < 1 or window < 0:
            raise ValueError("heads, sizes and ranks must be positive, the window not negative")
        if kv_rank > 256:
            raise ops.KernelArgumentError(f"the attention kernels take a latent of at most 256 values, not {kv_rank}")
        self.hidden_size, self.num_heads, self.head_dim, self.value_dim = hidden_size, num_heads, head_dim, value_dim
        self.kv_rank, self.q_rank, self.window = kv_rank, q_rank, int(window)
        self.scale = float(scale) if scale is not None else head_dim ** -0.5
        self.norm_eps, self.output_gate = float(norm_eps), bool(output_gate)
        self.w_in = self.w_uq = self.w_uk_t = self.w_uv = self.w_o = self.q_norm = self.c_norm = None

    def weight_specs(self) -> dict[str, WeightSpec]:
        h, H, d, dv = self.hidden_size, self.num_heads, self.head_dim, self.value_dim
        specs = {"dq": WeightSpec((self.q_rank, h)), "dq.norm": WeightSpec((self.q_rank,), role="float32", init="norm"),
                 "uq": WeightSpec((H * d, self.q_rank)), "dkv": WeightSpec((self.kv_rank, h)),
                 "dkv.norm": WeightSpec((self.kv_rank,), role="float32", init="norm"),
                 "uk": WeightSpec((H * d, self.kv_rank)), "uv": WeightSpec((H * dv, self.kv_rank)),
                 "o": WeightSpec((h, H * dv))}
        if self.output_gate:
            specs["g"] = WeightSpec((H * dv, h))
        return specs

    def load_weights(self, tensors: Mapping[str, torch.Tensor]) -> None:
        H, d, dv, r = self.num_heads, self.head_dim, self.value_dim, self.kv_rank
        # one product for everything that reads h: both latents and the gate
        self.w_in = stack_rows([tensors["dq"], tensors["dkv"]] + ([tensors["g"]] if self.output_gate else []))
        self.q_norm, self.c_norm = tensors["dq.norm"].contiguous(), tensors["dkv.norm"].contiguous()
        self.w_uq = tensors["uq"]
        self.w_uk_t = tensors["uk"].view(H, d, r).transpose(1, 2).contiguous()    # per head [kv_rank, head_dim]
        self.w_uv = tensors["uv"].view(H, dv, r).contiguous()
        self.w_o = tensors["o"]

    def cache_spec(self) -> PagedKVSpec:
        return PagedKVSpec(1, self.kv_rank, self.window)

    def graph_capturable(self, page_size: int) -> bool:
        return True  # a step of single tokens is read through the context's device arrays alone

    def forward(self, x: torch.Tensor, ctx: Any, cache: Any) -> torch.Tensor:
        if cache is None or cache.kind != "paged" or not cache.writable or cache.v_pages is None:
            raise RuntimeError("latent_attention needs a paged cache of its own")
        grp = ctx.groups[cache.group]
        n, H, r = x.shape[0], self.num_heads, self.kv_rank
        proj = linear_f32(self.rt, as_operand(self.rt, x, ctx), self.w_in)
        cq = self.rt.empty(n, self.q_rank)
        ops.latent_norm_cache(proj, 0, self.q_rank, self.q_rank, r, self.q_norm, self.c_norm, self.norm_eps, cq,
                              grp.slots, cache.k_pages, cache.v_pages)
        q = linear(self.rt, cq, self.w_uq)
        q_latent = self.rt.empty(n, H * r)
        ops.head_products(q, self.w_uk_t, q_latent)
        mixed = self.rt.empty(n, H * r)
        paged_scored_attention(self.rt, ctx, cache, q_latent, mixed, H, r, r, self.scale, window=self.window)
        out = self.rt.empty(n, H * self.value_dim)
        g0 = self.q_rank + r
        ops.head_products(mixed, self.w_uv, out, gate=proj[:, g0:g0 + H * self.value_dim] if self.output_gate else None)
        return linear_f32(self.rt, out, self.w_o)
