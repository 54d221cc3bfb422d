"""Token embedding: a row gather, no scaling (reference: src/dli/model/llama.py:221,291)."""

from __future__ import annotations

from typing import Any, Mapping, Optional

import numpy as np
import torch

from ..kernels import ops
from .base import DecodeStream, Embedding, Runtime
from .registry import build_part, register_part
from .spec import PartSpec, WeightSpec


@register_part("embedding", "token_embedding")
class TokenEmbedding(Embedding):
    def __init__(self, runtime: Runtime, *, vocab_size: int, hidden_size: int, weight_name: str = "weight",
                 float32_rows: bool = False, norm: Optional[PartSpec] = None) -> None:
        """``float32_rows``: the rows go out widened to float32 whatever the runtime's type, for a
        model that keeps its residual stream in 32-bit (the table keeps the runtime's type). ``norm``: a norm
        (a part with ``forward_f32``) that the float32 rows pass before they become the stream."""
        super().__init__(runtime)
        self.vocab_size, self.hidden_size = vocab_size, hidden_size
        self.weight_name, self.float32_rows = weight_name, bool(float32_rows)
        self.weight: torch.Tensor | None = None
        if norm is not None and not self.float32_rows:
            raise ValueError("a norm on the embedded rows belongs to a float32 stream")
        self.norm = build_part("norm", norm, runtime) if norm is not None else None

    def sub_parts(self) -> dict:
        return {"norm": self.norm} if self.norm is not None else {}

    def graph_capturable(self, page_size: int) -> bool:
        return True  # kernels on device arrays only

    def weight_specs(self) -> dict[str, WeightSpec]:
        return {self.weight_name: WeightSpec((self.vocab_size, self.hidden_size))}

    def load_weights(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.weight = tensors[self.weight_name]

    def table(self) -> torch.Tensor:
        assert self.weight is not None
        return self.weight

    def forward(self, ids: torch.Tensor) -> torch.Tensor:
        if self.float32_rows:
            raise RuntimeError("this embedding hands its rows to the step: call forward_step(ctx)")
        out = self.rt.empty(ids.shape[0], self.hidden_size)
        ops.embedding(self.table(), ids, out)
        return out

    def forward_step(self, ctx: Any) -> torch.Tensor:
        if not self.float32_rows:
            return self.forward(ctx.token_ids)
        out = torch.empty(ctx.token_ids.shape[0], self.hidden_size, device=self.rt.device, dtype=torch.float32)
        ops.embed_sinusoid(self.table(), ctx.token_ids, ctx.positions, None, out)
        return out if self.norm is None else self.norm.forward_f32(out)

    def streams(self, ctx) -> bool:
        return self.rt.is_bf16 and not self.float32_rows  # the fused decode kernels keep a stream of the runtime's type

    def forward_stream(self, ids: torch.Tensor) -> DecodeStream:
        n = ids.shape[0]
        out = self.rt.empty(n, self.hidden_size)
        ssq = torch.empty(1, n, device=self.rt.device, dtype=torch.float32)
        ops.embedding_ssq(self.table(), ids, out, ssq)
        return DecodeStream(out, ssq)


@register_part("embedding", "sinusoidal_token_embedding")
class SinusoidalTokenEmbedding(TokenEmbedding):
    """Token rows plus an absolute sinusoidal position vector, into a 32-bit residual stream:
    ``x[t] = table[id] + pe(p)`` with ``pe[2i] = sin(p base^(-2i/width))`` and ``pe[2i+1]`` the cosine of
    the same angle. The frequencies are made once on the host in double precision and rounded to
    float32; angles and sums are 32-bit on the device. The rows are float32 whatever the runtime's
    type (the table itself has the runtime's type, so a tied head can read it)."""

    def __init__(self, runtime: Runtime, *, vocab_size: int, hidden_size: int, base: float = 10000.0,
                 weight_name: str = "weight") -> None:
        super().__init__(runtime, vocab_size=vocab_size, hidden_size=hidden_size, weight_name=weight_name,
                         float32_rows=True)
        self.base = float(base)
        self._inv_freq: Optional[torch.Tensor] = None

    def finalize(self) -> None:
        pairs = (self.hidden_size + 1) // 2
        inv = np.power(self.base, -2.0 * np.arange(pairs, dtype=np.float64) / self.hidden_size).astype(np.float32)
        self._inv_freq = torch.from_numpy(inv).to(self.rt.device)

    def streams(self, ctx) -> bool:
        return False  # the fused decode kernels keep a stream of the runtime's type

    def forward(self, ids: torch.Tensor) -> torch.Tensor:
        raise RuntimeError("this embedding needs the positions of the step: call forward_step(ctx)")

    def forward_step(self, ctx: Any) -> torch.Tensor:
        if self._inv_freq is None:
            self.finalize()
        from .linear import RoundedStream

        out = torch.empty(ctx.token_ids.shape[0], self.hidden_size, device=self.rt.device, dtype=torch.float32)
        rounded = self.rt.empty(*out.shape) if self.rt.is_bf16 and hasattr(ctx, "_memo") else None
        ops.embed_sinusoid(self.table(), ctx.token_ids, ctx.positions, self._inv_freq, out, rounded=rounded)
        RoundedStream.offer(ctx, out, rounded)
        return out
