"""A plain, slow Zarinex in float64: whole sequences, no cache, no batching, one function per
mechanism. It takes the configuration as the dictionary that ``config.json`` holds and the tensors by
their checkpoint names, and shares no code with the engine.

A layer is ``x <- norm1(alpha x + r1 * mixer(shift(x)))`` then ``x <- norm2(alpha x + r2 * ff(x))`` with
``r = sigmoid(W_rg x + b_rg)`` read from the unshifted ``x``; the mixers are a selective scan (``mamba1``),
attention through a latent (``latent_attention``) and a gated linear recurrence (``hgrn2``); the
feed-forward is a mixture of experts with a shared expert. ``states`` carry what a sequence keeps from
one call to the next, so that the same functions also step token by token.
"""

from __future__ import annotations

import math
from typing import Any, Mapping, Optional

import torch

F = torch.float64


def rms_norm(x: torch.Tensor, w: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if w is None else y * w


def sigmoid(x: torch.Tensor) -> torch.Tensor:
    return 1.0 / (1.0 + torch.exp(-x))


def silu(x: torch.Tensor) -> torch.Tensor:
    return x * sigmoid(x)


def softplus(x: torch.Tensor) -> torch.Tensor:
    return torch.where(x > 30.0, x, torch.log1p(torch.exp(torch.clamp(x, max=30.0))))


def position_vectors(positions: torch.Tensor, width: int) -> torch.Tensor:
    """Entry 2i is sin(p 10000^(-2i/width)), entry 2i+1 the cosine of the same angle."""
    out = torch.zeros(positions.shape[0], width, dtype=F)
    for c in range(width):
        i = c // 2
        angle = positions.to(F) * (10000.0 ** (-2.0 * i / width))
        out[:, c] = torch.cos(angle) if c % 2 else torch.sin(angle)
    return out


def token_shift(h: torch.Tensor, shift: torch.Tensor, state: dict) -> torch.Tensor:
    """``h + (h_prev - h) * shift`` with the row before (zeros before the first); ``state['prev']`` is
    the last unshifted row seen so far."""
    prev0 = state.get("prev")
    if prev0 is None:
        prev0 = torch.zeros(h.shape[1], dtype=F)
    before = torch.cat([prev0[None], h[:-1]], dim=0)
    state["prev"] = h[-1].clone()
    return h + (before - h) * shift


def causal_conv(x: torch.Tensor, w: torch.Tensor, b: Optional[torch.Tensor], state: dict) -> torch.Tensor:
    """Per channel, ``y[t] = b + sum_j w[:, taps-1-j] x[t-j]``; ``state['conv']`` holds the last ``taps-1`` inputs."""
    taps = w.shape[1]
    kept = state.get("conv")
    if kept is None:
        kept = torch.zeros(taps - 1, x.shape[1], dtype=F)
    full = torch.cat([kept, x], dim=0)
    out = torch.zeros_like(x)
    for t in range(x.shape[0]):
        window = full[t:t + taps]                    # oldest first; the last row is token t
        out[t] = (window * w.t()).sum(0)
    if b is not None:
        out = out + b
    state["conv"] = full[full.shape[0] - (taps - 1):].clone()
    return out


def selective_scan(x: torch.Tensor, dt: torch.Tensor, B: torch.Tensor, C: torch.Tensor, A_log: torch.Tensor,
                   D: torch.Tensor, S: Optional[torch.Tensor]) -> tuple:
    """``S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n``, ``y_c = sum_n S[c, n] C_n + D_c x_c`` token by token."""
    A = -torch.exp(A_log)                            # [channels, states]
    if S is None:
        S = torch.zeros(A.shape, dtype=F)
    y = torch.zeros_like(x)
    for t in range(x.shape[0]):
        S = torch.exp(dt[t][:, None] * A) * S + (dt[t] * x[t])[:, None] * B[t][None, :]
        y[t] = S @ C[t] + D * x[t]
    return y, S


def mamba1(h: torch.Tensor, p: Mapping[str, torch.Tensor], m: Mapping[str, Any], state: dict) -> torch.Tensor:
    inner, n_state, rank = m["inner"], m["state"], m["dt_rank"]
    xz = h @ p["in"].t()
    x, z = xz[:, :inner], xz[:, inner:]
    x = silu(causal_conv(x, p["conv"], p["conv.b"], state))
    low = x @ p["x"].t()
    dt, B, C = low[:, :rank], low[:, rank:rank + n_state], low[:, rank + n_state:]
    dt = softplus(dt @ p["dt"].t() + p["dt.b"])      # [tokens, inner]
    y, state["S"] = selective_scan(x, dt, B, C, p["A_log"], p["D"], state.get("S"))
    return (y * silu(z)) @ p["o"].t()


def latent_attention(h: torch.Tensor, p: Mapping[str, torch.Tensor], m: Mapping[str, Any], eps: float,
                     state: dict) -> torch.Tensor:
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    cq = rms_norm(h @ p["dq"].t(), p["dq.norm"], eps)
    q = (cq @ p["uq"].t()).view(-1, H, d)
    c = rms_norm(h @ p["dkv"].t(), p["dkv.norm"], eps)
    past = state.get("c")
    c_all = c if past is None else torch.cat([past, c], dim=0)
    state["c"] = c_all
    k = (c_all @ p["uk"].t()).view(-1, H, d)
    v = (c_all @ p["uv"].t()).view(-1, H, dv)
    n, total = h.shape[0], c_all.shape[0]
    first = total - n
    out = torch.zeros(n, H, dv, dtype=F)
    for t in range(n):
        seen = first + t + 1
        s = torch.einsum("hd,jhd->hj", q[t], k[:seen]) * m["scale"]
        w = torch.softmax(s, dim=-1)
        out[t] = torch.einsum("hj,jhd->hd", w, v[:seen])
    gate = sigmoid(h @ p["g"].t())
    return (out.reshape(n, H * dv) * gate) @ p["o"].t()


def gated_linear(q: torch.Tensor, f: torch.Tensor, v: torch.Tensor, S: Optional[torch.Tensor]) -> tuple:
    """Per head ``S <- diag(f) S + (1 - f) v^T``, ``o = S^T q``; q, f ``[n, H, d]``, v ``[n, H, dv]``, S ``[H, d, dv]``."""
    n, H, d = q.shape
    if S is None:
        S = torch.zeros(H, d, v.shape[2], dtype=F)
    out = torch.zeros(n, H, v.shape[2], dtype=F)
    for t in range(n):
        S = f[t][:, :, None] * S + (1.0 - f[t])[:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", S, q[t])
    return out, S


def hgrn2(h: torch.Tensor, p: Mapping[str, torch.Tensor], m: Mapping[str, Any], eps: float, state: dict) -> torch.Tensor:
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    n = h.shape[0]
    q = silu(h @ p["q"].t()).view(n, H, d)
    v = (h @ p["v"].t()).view(n, H, dv)
    lower = p["lower"]
    f = (lower + (1.0 - lower) * sigmoid(h @ p["f"].t() + p["f.b"])).view(n, H, d)
    out, state["S"] = gated_linear(q, f, v, state.get("S"))
    out = rms_norm(out, p["norm"], eps)
    return out.reshape(n, H * dv) @ p["o"].t()


def expert(h: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor) -> torch.Tensor:
    return (silu(h @ gate.t()) * (h @ up.t())) @ down.t()


def route(z: torch.Tensor, top: int) -> tuple:
    """The ``top`` largest logits of a token (the lower index on a tie) and the softmax over them alone."""
    order = sorted(range(z.shape[0]), key=lambda e: (-float(z[e]), e))[:top]
    return order, torch.softmax(z[order], dim=0)


def moe(h: torch.Tensor, p: Mapping[str, torch.Tensor], m: Mapping[str, Any]) -> torch.Tensor:
    top = m["router"]["top"]
    z = h @ p["router"].t() + p["router.b"]
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        order, w = route(z[t], top)
        for j, e in enumerate(order):
            out[t] += w[j] * expert(h[t:t + 1], p[f"e{e}.gate"], p[f"e{e}.up"], p[f"e{e}.down"])[0]
    if m.get("shared"):
        out = out + expert(h, p["shared.gate"], p["shared.up"], p["shared.down"])
    return out


def sub_tensors(tensors: Mapping[str, torch.Tensor], prefix: str) -> dict:
    return {k[len(prefix):]: v.to(F) for k, v in tensors.items() if k.startswith(prefix)}


class PlainZarinex:
    def __init__(self, config: Mapping[str, Any], tensors: Mapping[str, torch.Tensor]) -> None:
        self.cfg, self.t = config, {k: v.to(F) for k, v in tensors.items()}
        self.width, self.eps, self.alpha = config["width"], float(config["norm"]["eps"]), float(config["postln_alpha"])

    def new_state(self) -> list:
        return [{"shift": {}, "mixer": {}} for _ in self.cfg["layers"]]

    def layer(self, i: int, x: torch.Tensor, state: dict) -> torch.Tensor:
        entry = self.cfg["layers"][i]
        src = entry.get("weights_of", i)
        src = i if src is None else src
        own = sub_tensors(self.t, f"l{src}.")
        mix = sub_tensors(self.t, f"l{src}.mix.")
        h = x
        r = sigmoid(h @ own["rg1"].t() + own["rg1.b"])
        shifted = token_shift(h, own["shift"], state["shift"])
        kind, m = entry["type"], entry["mixer"]
        if kind == "mamba1":
            y = mamba1(shifted, mix, m, state["mixer"])
        elif kind == "latent_attention":
            y = latent_attention(shifted, mix, m, self.eps, state["mixer"])
        elif kind == "hgrn2":
            y = hgrn2(shifted, mix, m, self.eps, state["mixer"])
        else:
            raise ValueError(kind)
        x = rms_norm(self.alpha * x + r * y, own["norm1"], self.eps)
        if entry.get("mlp") is not None:
            h = x
            r = sigmoid(h @ own["rg2"].t() + own["rg2.b"])
            y = moe(h, sub_tensors(self.t, f"l{src}.mlp."), entry["mlp"])
            x = rms_norm(self.alpha * x + r * y, own["norm2"], self.eps)
        return x

    def forward(self, tokens, states: Optional[list] = None, start: int = 0, layers_out: Optional[list] = None) -> torch.Tensor:
        """Logits ``[tokens, vocab]`` of ``tokens`` at positions ``start, start+1, ...``; ``states`` (from
        :meth:`new_state`) carries the sequence from call to call."""
        states = self.new_state() if states is None else states
        ids = torch.as_tensor(tokens, dtype=torch.long)
        x = self.t["embed"][ids] + position_vectors(torch.arange(start, start + len(ids)), self.width)
        for i in range(len(self.cfg["layers"])):
            x = self.layer(i, x, states[i])
            if layers_out is not None:
                layers_out.append(x.clone())
        x = rms_norm(x, self.t["final.norm"], self.eps)
        return x @ self.t["embed"].t()


def forward_logits(cfg: Mapping[str, Any], tensors: Mapping[str, torch.Tensor], tokens) -> torch.Tensor:
    return PlainZarinex(cfg, tensors).forward(tokens)


def greedy_generate(cfg: Mapping[str, Any], tensors: Mapping[str, torch.Tensor], prompt, n_new: int) -> list:
    toks, out = list(prompt), []
    m = PlainZarinex(cfg, tensors)
    for _ in range(n_new):
        nxt = int(m.forward(toks)[-1].argmax())
        out.append(nxt)
        toks.append(nxt)
    return out


# ------------------------------------------------------------------------------ weights of a test model

def tensor_shapes(cfg: Mapping[str, Any]) -> dict:
    """Name -> shape of every tensor of a model of this configuration."""
    w = cfg["width"]
    out = {"embed": (cfg["vocab"], w), "final.norm": (w,)}
    for i, layer in enumerate(cfg["layers"]):
        if layer.get("weights_of") is not None:
            continue
        p, m = f"l{i}.", layer["mixer"]
        out.update({p + "norm1": (w,), p + "shift": (w,), p + "rg1": (w, w), p + "rg1.b": (w,)})
        if layer["type"] == "mamba1":
            c, n, r = m["inner"], m["state"], m["dt_rank"]
            out.update({p + "mix.in": (2 * c, w), p + "mix.conv": (c, m["conv"]), p + "mix.conv.b": (c,),
                        p + "mix.x": (r + 2 * n, c), p + "mix.dt": (c, r), p + "mix.dt.b": (c,), p + "mix.A_log": (c, n),
                        p + "mix.D": (c,), p + "mix.o": (w, c)})
        elif layer["type"] == "latent_attention":
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            out.update({p + "mix.dq": (m["q_rank"], w), p + "mix.dq.norm": (m["q_rank"],), p + "mix.uq": (H * d, m["q_rank"]),
                        p + "mix.dkv": (m["kv_rank"], w), p + "mix.dkv.norm": (m["kv_rank"],), p + "mix.uk": (H * d, m["kv_rank"]),
                        p + "mix.uv": (H * dv, m["kv_rank"]), p + "mix.g": (H * dv, w), p + "mix.o": (w, H * dv)})
        else:
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            out.update({p + "mix.q": (H * d, w), p + "mix.f": (H * d, w), p + "mix.f.b": (H * d,), p + "mix.lower": (H * d,),
                        p + "mix.v": (H * dv, w), p + "mix.norm": (dv,), p + "mix.o": (w, H * dv)})
        f = layer.get("mlp")
        if f is not None:
            out.update({p + "norm2": (w,), p + "rg2": (w, w), p + "rg2.b": (w,), p + "mlp.router": (f["router"]["experts"], w),
                        p + "mlp.router.b": (f["router"]["experts"],)})
            for e in range(f["router"]["experts"]):
                out.update({p + f"mlp.e{e}.gate": (f["expert"]["ff"], w), p + f"mlp.e{e}.up": (f["expert"]["ff"], w),
                            p + f"mlp.e{e}.down": (w, f["expert"]["ff"])})
            if f.get("shared"):
                s = f["shared"]["ff"]
                out.update({p + "mlp.shared.gate": (s, w), p + "mlp.shared.up": (s, w), p + "mlp.shared.down": (w, s)})
    return out


def random_weights(cfg: Mapping[str, Any], seed: int) -> dict:
    """Random tensors whose values are exactly representable in bfloat16 (float64 here), drawn so that every
    mechanism matters: projections of unit-size outputs, norm weights near one, shifts spread over (0, 1),
    gates that are neither open nor shut, a router that prefers some experts clearly, decays spread out."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.split(".", 1)[1] if name.startswith("l") and "." in name else name
        if leaf in ("norm1", "norm2", "final.norm", "mix.norm", "mix.dq.norm", "mix.dkv.norm"):
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif leaf == "shift":
            t = torch.rand(shape, generator=g)
        elif leaf in ("rg1.b", "rg2.b", "mix.f.b", "mix.conv.b", "mlp.router.b"):
            t = 0.5 * torch.randn(shape, generator=g)
        elif leaf == "mix.conv":
            t = 0.6 * torch.randn(shape, generator=g)
        elif leaf == "mix.A_log":
            t = torch.rand(shape, generator=g) * 2.5 - 1.5
        elif leaf == "mix.dt.b":
            t = torch.randn(shape, generator=g) - 1.0
        elif leaf == "mix.D":
            t = 1.0 + 0.3 * torch.randn(shape, generator=g)
        elif leaf == "mix.lower":
            t = 0.9 * torch.rand(shape, generator=g)
        elif leaf == "mlp.router":
            t = 3.0 * torch.randn(shape, generator=g) / math.sqrt(shape[-1])
        elif name == "embed":
            t = 0.5 * torch.randn(shape, generator=g)
        else:
            t = torch.randn(shape, generator=g) / math.sqrt(shape[-1]) * (2.0 if leaf in ("mix.uq", "mix.uk", "mix.f") else 1.0)
        out[name] = t.to(torch.bfloat16).to(F)
    return out


def jittered(tensors: Mapping[str, torch.Tensor], seed: int = 0, size: float = 2.0 ** -8) -> dict:
    """Every matrix with relative noise of the size of bfloat16's rounding: how far the logits of a position
    move under it says how far rounding may move them. Routers are left alone."""
    g = torch.Generator().manual_seed(seed)
    return {n: t * (1 + size * torch.randn(t.shape, generator=g, dtype=F)) if t.dim() == 2 and not n.endswith("router") else t
            for n, t in tensors.items()}


def write_folder(folder, cfg: Mapping[str, Any], tensors: Mapping[str, torch.Tensor]):
    """``config.json`` and ``model.safetensors`` (bfloat16) of ``tensors``, written byte by byte here."""
    import json
    import struct

    import numpy as np

    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(cfg))
    header, blobs, at = {}, [], 0
    for name in sorted(tensors):
        bits = (tensors[name].to(torch.float32).contiguous().view(torch.int32).numpy().astype(np.uint32) >> 16).astype("<u2")
        raw = bits.tobytes()
        header[name] = {"dtype": "BF16", "shape": list(tensors[name].shape), "data_offsets": [at, at + len(raw)]}
        blobs.append(raw)
        at += len(raw)
    head = json.dumps(header).encode()
    head += b" " * (-len(head) % 8)
    with open(folder / "model.safetensors", "wb") as f:
        f.write(struct.pack("<Q", len(head)))
        f.write(head)
        for raw in blobs:
            f.write(raw)
    return folder
