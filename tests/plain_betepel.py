"""A plain, slow Betepel in float64: whole sequences, no cache, no batching, one function per
mechanism. It takes the configuration as the dictionary that ``config.json`` holds and the tensors by
their checkpoint names, and shares no code with the engine.

The embedding is normalised; a layer is ``x <- x + mixer(norm1(x)) + ff(norm2(x))`` (both norms of the same
``x``, weights stored as ``w`` and applied as ``1 + w``); the mixers are a matrix memory with exponential
gates (``mlstm``), differential attention under a sliding window that keeps the first positions
(``attention``; a layer may read another layer's keys and values), and a pair side by side: windowed
rotary attention and a linear attention with a constant decay per head (``parallel``). The feed-forward
is a mixture of experts that a table chooses by token id, plus a shared expert. ``states`` carry what a
sequence keeps from one call to the next, so that the same functions also step token by token.
"""

from __future__ import annotations

import math
from typing import Any, Mapping, Optional

import torch

F = torch.float64


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def offset_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return rms(x, eps) * (1.0 + w)


def sigmoid(x: torch.Tensor) -> torch.Tensor:
    return 1.0 / (1.0 + torch.exp(-x))


def silu(x: torch.Tensor) -> torch.Tensor:
    return x * sigmoid(x)


def log_sigmoid(x: torch.Tensor) -> torch.Tensor:
    return -(torch.clamp(-x, min=0.0) + torch.log1p(torch.exp(-x.abs())))


def rotary_frequencies(rot: Mapping[str, Any]) -> torch.Tensor:
    """``base^(-2i/dims)``, and with ``scaling`` the three bands by wavelength: short ones kept, long ones
    divided by ``factor``, a linear blend between."""
    dims = rot["dims"]
    f = torch.tensor([float(rot["base"]) ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F)
    sc = rot.get("scaling")
    if sc:
        factor, low, high, orig = float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"])
        out = f.clone()
        for i in range(f.shape[0]):
            wavelength = 2.0 * math.pi / float(f[i])
            if wavelength < orig / high:
                continue
            if wavelength > orig / low:
                out[i] = f[i] / factor
            else:
                s = (orig / wavelength - low) / (high - low)
                out[i] = (1.0 - s) * f[i] / factor + s * f[i]
        f = out
    return f


def rotate(x: torch.Tensor, positions: torch.Tensor, rot: Optional[Mapping[str, Any]]) -> torch.Tensor:
    """``x [n, ..., dim]``: component ``i`` turns with component ``i + dims/2`` for ``i < dims/2``; the rest stays."""
    if not rot:
        return x
    dims = rot["dims"]
    half = dims // 2
    angle = positions.to(F)[:, None] * rotary_frequencies(rot)[None, :]           # [n, half]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    c, s = torch.cos(angle).view(shape), torch.sin(angle).view(shape)
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def visible(i: int, j: int, mask: Optional[Mapping[str, Any]]) -> bool:
    if j > i:
        return False
    if not mask or mask.get("size") is None:
        return True
    return i - j < mask["size"] or j < (mask.get("keep_first") or 0)


def masked_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, first: int, scale: float,
                     mask: Optional[Mapping[str, Any]]) -> torch.Tensor:
    """``q [n, heads, d]`` at positions ``first ..``; ``k [total, kv, d]``, ``v [total, kv, dv]`` from position 0;
    query head ``h`` reads kv head ``h // (heads / kv)``. Returns ``[n, heads, dv]``."""
    n, H, _ = q.shape
    per = H // k.shape[1]
    out = torch.zeros(n, H, v.shape[2], dtype=F)
    for t in range(n):
        i = first + t
        seen = [j for j in range(i + 1) if visible(i, j, mask)]
        for h in range(H):
            g = h // per
            s = (k[seen, g] @ q[t, h]) * scale
            w = torch.softmax(s, dim=0)
            out[t, h] = w @ v[seen, g]
    return out


def attention_sizes(m: Mapping[str, Any]) -> tuple:
    """heads, kv heads (absent: as many), key size, value size (absent: the key's), scale (absent: dim^-1/2)."""
    H, d = m["heads"], m["dim"]
    scale = m.get("scale")
    return H, m.get("kv_heads") or H, d, m.get("vdim") or d, float(scale) if scale is not None else d ** -0.5


def project(h: torch.Tensor, p: Mapping[str, torch.Tensor], name: str) -> torch.Tensor:
    y = h @ p[name].t()
    return y + p[name + ".b"] if name + ".b" in p else y


def keys_values(h: torch.Tensor, p: Mapping[str, torch.Tensor], m: Mapping[str, Any], maps: int, first: int,
                state: dict) -> tuple:
    """This call's rotated keys and values appended to what ``state`` holds; keys ``[total, kv * maps, d]``."""
    n = h.shape[0]
    _, G, d, dv, _ = attention_sizes(m)
    pos = torch.arange(first, first + n)
    k = rotate(project(h, p, "k").view(n, G * maps, d), pos, m.get("rot"))
    v = project(h, p, "v").view(n, G, dv)
    if "k" in state:
        k, v = torch.cat([state["k"], k]), torch.cat([state["v"], v])
    state["k"], state["v"] = k, v
    return k, v


def differential_attention(h: torch.Tensor, p: Mapping[str, torch.Tensor], m: Mapping[str, Any], eps: float,
                           first: int, state: dict, borrowed: Optional[dict] = None) -> torch.Tensor:
    """Two score maps per head over the same values: ``o = a1 - lam a2``, normalised per head without a
    weight, times ``1 - diff``, times one gate per head. ``borrowed``: another layer's state with keys and
    values (this layer then has none of its own)."""
    n = h.shape[0]
    H, G, d, dv, scale = attention_sizes(m)
    pos = torch.arange(first, first + n)
    q = rotate(project(h, p, "q").view(n, H * 2, d), pos, m.get("rot")).view(n, H, 2, d)
    if borrowed is None:
        k, v = keys_values(h, p, m, 2, first, state)
    else:
        k, v = borrowed["k"], borrowed["v"]
    k = k.view(-1, G, 2, d)
    a1 = masked_attention(q[:, :, 0], k[:, :, 0], v, first, scale, m.get("mask"))
    a2 = masked_attention(q[:, :, 1], k[:, :, 1], v, first, scale, m.get("mask"))
    diff = float(m["diff"])
    lam = torch.exp((p["lq1"] * p["lk1"]).sum()) - torch.exp((p["lq2"] * p["lk2"]).sum()) + diff
    o = rms(a1 - lam * a2, eps) * (1.0 - diff)
    o = o * sigmoid(h @ p["g"].t())[:, :, None]
    return o.reshape(n, H * dv) @ p["o"].t()


def windowed_attention(h: torch.Tensor, p: Mapping[str, torch.Tensor], m: Mapping[str, Any], first: int,
                       state: dict) -> torch.Tensor:
    n = h.shape[0]
    H, _, d, _, scale = attention_sizes(m)
    pos = torch.arange(first, first + n)
    q = rotate(project(h, p, "q").view(n, H, d), pos, m.get("rot"))
    k, v = keys_values(h, p, m, 1, first, state)
    o = masked_attention(q, k, v, first, scale, m.get("mask"))
    return o.reshape(n, -1) @ p["o"].t()


def decayed_linear_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: torch.Tensor,
                             S: Optional[torch.Tensor]) -> tuple:
    """Per head ``S <- decay S + k v^T``, ``o = S^T q``; q, k ``[n, H, d]``, v ``[n, H, dv]``, S ``[H, d, dv]``."""
    n, H, d = q.shape
    if S is None:
        S = torch.zeros(H, d, v.shape[2], dtype=F)
    out = torch.zeros(n, H, v.shape[2], dtype=F)
    for t in range(n):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", S, q[t])
    return out, S


def lightning(h: torch.Tensor, p: Mapping[str, torch.Tensor], m: Mapping[str, Any], eps: float, state: dict) -> torch.Tensor:
    n, H, d = h.shape[0], m["heads"], m["dim"]
    dv = m.get("vdim") or d
    q, k = silu(h @ p["q"].t()).view(n, H, d), silu(h @ p["k"].t()).view(n, H, d)
    v = silu(h @ p["v"].t()).view(n, H, dv)
    o, state["S"] = decayed_linear_attention(q, k, v, torch.tensor(m["decay"], dtype=F), state.get("S"))
    o = rms(o.reshape(n, H * dv), eps) * p["norm"]
    return (o * sigmoid(h @ p["g"].t())) @ p["o"].t()


def side_by_side(h: torch.Tensor, p: Mapping[str, torch.Tensor], m: Mapping[str, Any], eps: float, first: int,
                 state: dict) -> torch.Tensor:
    left = windowed_attention(h, sub_tensors(p, "left."), m["left"], first, state.setdefault("left", {}))
    right = lightning(h, sub_tensors(p, "right."), m["right"], eps, state.setdefault("right", {}))
    return float(m.get("left_scale", 1.0)) * left + float(m.get("right_scale", 1.0)) * right


def matrix_memory(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, i: torch.Tensor, f: torch.Tensor, state: dict) -> torch.Tensor:
    """Per head, with log gates ``i`` and ``f`` ``[n, H]`` and a running reference point ``m`` that starts at 0:
    ``m' = max(f + m, i)``, ``S' = e^(f + m - m') S + e^(i - m') k v^T``, ``n'`` the same with ``k`` alone,
    ``o = S'^T q / (max(|n' . q|, e^(-m')) + 1e-6)``."""
    n, H, d = q.shape
    dv = v.shape[2]
    S = state.get("S", torch.zeros(H, d, dv, dtype=F))
    nrm = state.get("n", torch.zeros(H, d, dtype=F))
    m = state.get("m", torch.zeros(H, dtype=F))
    out = torch.zeros(n, H, dv, dtype=F)
    for t in range(n):
        m_new = torch.maximum(f[t] + m, i[t])
        keep, write = torch.exp(f[t] + m - m_new), torch.exp(i[t] - m_new)
        S = keep[:, None, None] * S + write[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        nrm = keep[:, None] * nrm + write[:, None] * k[t]
        m = m_new
        den = torch.maximum((nrm * q[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
        out[t] = torch.einsum("hdv,hd->hv", S, q[t]) / den[:, None]
    state["S"], state["n"], state["m"] = S, nrm, m
    return out


def mlstm(h: torch.Tensor, p: Mapping[str, torch.Tensor], m: Mapping[str, Any], eps: float, state: dict) -> torch.Tensor:
    n, H, d, cap = h.shape[0], m["heads"], m["dim"], float(m.get("gate_cap") or 0.0)
    dv = m.get("vdim") or d
    q = (h @ p["q"].t()).view(n, H, d) * d ** -0.5
    k, v = (h @ p["k"].t()).view(n, H, d), (h @ p["v"].t()).view(n, H, dv)
    i, f = h @ p["i"].t() + p["i.b"], h @ p["f"].t() + p["f.b"]
    if cap:                                          # (no cap: the gates' pre-activations as they are)
        i, f = cap * torch.tanh(i / cap), cap * torch.tanh(f / cap)
    f = log_sigmoid(f)
    o = rms(matrix_memory(q, k, v, i, f, state), eps).reshape(n, H * dv) * p["norm"]
    return (o * sigmoid(h @ p["g"].t())) @ p["o"].t()


def expert(h: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor) -> torch.Tensor:
    return (silu(h @ gate.t()) * (h @ up.t())) @ down.t()


def table_experts(h: torch.Tensor, ids: torch.Tensor, p: Mapping[str, torch.Tensor], f: Mapping[str, Any]) -> torch.Tensor:
    """Each token's experts are the row of ``table`` at its token id, each weighted ``1 / top``."""
    top = f["router"]["top"]
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e in p["table"][int(ids[t])].tolist():
            e = int(e)
            out[t] += expert(h[t:t + 1], p[f"e{e}.gate"], p[f"e{e}.up"], p[f"e{e}.down"])[0] / top
    if f.get("shared"):
        out = out + expert(h, p["shared.gate"], p["shared.up"], p["shared.down"])
    return out


def sub_tensors(tensors: Mapping[str, torch.Tensor], prefix: str) -> dict:
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


class PlainBetepel:
    def __init__(self, config: Mapping[str, Any], tensors: Mapping[str, torch.Tensor]) -> None:
        self.cfg = config
        self.t = {k: (v.to(F) if v.is_floating_point() else v.to(torch.long)) for k, v in tensors.items()}
        self.width, self.eps = config["width"], float(config["norm"]["eps"])

    def new_state(self) -> list:
        return [{} for _ in self.cfg["layers"]]

    def layer(self, i: int, x: torch.Tensor, ids: torch.Tensor, first: int, states: list) -> torch.Tensor:
        entry = self.cfg["layers"][i]
        own, mix = sub_tensors(self.t, f"l{i}."), sub_tensors(self.t, f"l{i}.mix.")
        h = offset_norm(x, own["norm1"], self.eps)
        kind, m = entry["type"], entry["mixer"]
        if kind == "mlstm":
            y = mlstm(h, mix, m, self.eps, states[i])
        elif kind == "attention":
            src = m.get("kv_from")
            y = differential_attention(h, mix, m, self.eps, first, states[i], None if src is None else states[src])
        elif kind == "parallel":
            y = side_by_side(h, mix, m, self.eps, first, states[i])
        else:
            raise ValueError(kind)
        if entry.get("mlp") is not None:
            y = y + table_experts(offset_norm(x, own["norm2"], self.eps), ids, sub_tensors(self.t, f"l{i}.mlp."), entry["mlp"])
        return x + y

    def forward(self, tokens, states: Optional[list] = None, start: int = 0, layers_out: Optional[list] = None) -> torch.Tensor:
        """Logits ``[tokens, vocab]`` of ``tokens`` at positions ``start, start+1, ...``; ``states`` (from
        :meth:`new_state`) carries the sequence from call to call."""
        states = self.new_state() if states is None else states
        ids = torch.as_tensor(tokens, dtype=torch.long)
        x = offset_norm(self.t["embed"][ids], self.t["embed.norm"], self.eps)
        for i in range(len(self.cfg["layers"])):
            x = self.layer(i, x, ids, start, states)
            if layers_out is not None:
                layers_out.append(x.clone())
        x = offset_norm(x, self.t["final.norm"], self.eps)
        return (x @ self.t["embed"].t()) * float(self.cfg.get("logit_scale", 1.0))


def forward_logits(cfg: Mapping[str, Any], tensors: Mapping[str, torch.Tensor], tokens) -> torch.Tensor:
    return PlainBetepel(cfg, tensors).forward(tokens)


def greedy_generate(cfg: Mapping[str, Any], tensors: Mapping[str, torch.Tensor], prompt, n_new: int) -> list:
    m = PlainBetepel(cfg, tensors)
    states = m.new_state()
    logits = m.forward(list(prompt), states)
    out, at = [], len(prompt)
    for _ in range(n_new):
        nxt = int(logits[-1].argmax())
        out.append(nxt)
        logits = m.forward([nxt], states, start=at)
        at += 1
    return out


# ------------------------------------------------------------------------------ weights of a test model

def attention_shapes(p: str, m: Mapping[str, Any], w: int, maps: int, own_kv: bool) -> dict:
    H, G, d, dv, _ = attention_sizes(m)
    out = {p + "q": (H * maps * d, w), p + "q.b": (H * maps * d,), p + "o": (w, H * dv)}
    if own_kv:
        out.update({p + "k": (G * maps * d, w), p + "k.b": (G * maps * d,), p + "v": (G * dv, w), p + "v.b": (G * dv,)})
    return out


def tensor_shapes(cfg: Mapping[str, Any]) -> dict:
    """Name -> shape of every tensor of a model of this configuration."""
    w = cfg["width"]
    out = {"embed": (cfg["vocab"], w), "embed.norm": (w,), "final.norm": (w,)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = (w,)
        if layer["type"] == "mlstm":
            H, d = m["heads"], m["dim"]
            dv = m.get("vdim") or d
            out.update({p + "mix.q": (H * d, w), p + "mix.k": (H * d, w), p + "mix.v": (H * dv, w), p + "mix.g": (H * dv, w),
                        p + "mix.o": (w, H * dv), p + "mix.norm": (H * dv,), p + "mix.i": (H, w), p + "mix.i.b": (H,),
                        p + "mix.f": (H, w), p + "mix.f.b": (H,)})
        elif layer["type"] == "attention":
            out.update(attention_shapes(p + "mix.", m, w, 2, m.get("kv_from") is None))
            d = m["dim"]
            out.update({p + "mix.lq1": (d,), p + "mix.lk1": (d,), p + "mix.lq2": (d,), p + "mix.lk2": (d,),
                        p + "mix.g": (m["heads"], w)})
        else:
            out.update(attention_shapes(p + "mix.left.", m["left"], w, 1, True))
            r = m["right"]
            H, d = r["heads"], r["dim"]
            dv = r.get("vdim") or d
            out.update({p + "mix.right.q": (H * d, w), p + "mix.right.k": (H * d, w), p + "mix.right.v": (H * dv, w),
                        p + "mix.right.g": (H * dv, w), p + "mix.right.o": (w, H * dv), p + "mix.right.norm": (H * dv,)})
        f = layer.get("mlp")
        if f is not None:
            out[p + "norm2"] = (w,)
            out[p + "mlp.table"] = (cfg["vocab"], f["router"]["top"])
            for e in range(f["router"]["experts"]):
                out.update({p + f"mlp.e{e}.gate": (f["expert"]["ff"], w), p + f"mlp.e{e}.up": (f["expert"]["ff"], w),
                            p + f"mlp.e{e}.down": (w, f["expert"]["ff"])})
            if f.get("shared"):
                s = f["shared"]["ff"]
                out.update({p + "mlp.shared.gate": (s, w), p + "mlp.shared.up": (s, w), p + "mlp.shared.down": (w, s)})
    return out


def random_weights(cfg: Mapping[str, Any], seed: int) -> dict:
    """Random tensors whose values are exactly representable in bfloat16 (float64 here; the experts' table
    int32), drawn so that every mechanism matters: projections of unit-size outputs, offset norm weights
    around zero, plain ones around one, input and forget gates that move, biases that count, a table whose
    rows name different experts."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.split(".")[-1] if not name.endswith(".b") else ".".join(name.split(".")[-2:])
        if leaf == "table":
            experts = int(name and cfg["layers"][int(name[1:name.index(".")])]["mlp"]["router"]["experts"])
            rows = [torch.randperm(experts, generator=g)[:shape[1]] for _ in range(shape[0])]
            out[name] = torch.stack(rows).to(torch.int32)
            continue
        if leaf in ("norm1", "norm2") or name in ("embed.norm", "final.norm"):
            t = 0.2 * torch.randn(shape, generator=g)
        elif leaf == "norm":
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif leaf in ("lq1", "lk1", "lq2", "lk2"):
            t = 0.3 * torch.randn(shape, generator=g)
        elif leaf in ("i.b", "f.b"):
            t = torch.randn(shape, generator=g) + (2.0 if leaf == "f.b" else 0.0)
        elif leaf.endswith(".b"):
            t = 0.3 * torch.randn(shape, generator=g)
        elif name == "embed":
            t = 0.5 * torch.randn(shape, generator=g)
        elif leaf in ("i", "f"):
            t = 3.0 * torch.randn(shape, generator=g) / math.sqrt(shape[-1])
        else:
            t = torch.randn(shape, generator=g) / math.sqrt(shape[-1]) * (2.0 if leaf in ("q", "k") else 1.0)
        out[name] = t.to(torch.bfloat16).to(F)
    return out


def jittered(tensors: Mapping[str, torch.Tensor], seed: int = 0, size: float = 2.0 ** -8) -> dict:
    """Every matrix with relative noise of the size of bfloat16's rounding: how far the logits of a position
    move under it says how far rounding may move them. Integer tables are left alone."""
    g = torch.Generator().manual_seed(seed)
    return {n: t * (1 + size * torch.randn(t.shape, generator=g, dtype=F)) if t.is_floating_point() and t.dim() == 2 else t
            for n, t in tensors.items()}


def write_folder(folder, cfg: Mapping[str, Any], tensors: Mapping[str, torch.Tensor]):
    """``config.json`` and ``model.safetensors`` (bfloat16; integer tables int32) of ``tensors``, written byte by
    byte here."""
    import json
    import struct

    import numpy as np

    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(cfg))
    header, blobs, at = {}, [], 0
    for name in sorted(tensors):
        t = tensors[name]
        if t.is_floating_point():
            bits = (t.to(torch.float32).contiguous().view(torch.int32).numpy().astype(np.uint32) >> 16).astype("<u2")
            raw, kind = bits.tobytes(), "BF16"
        else:
            raw, kind = t.to(torch.int32).contiguous().numpy().astype("<i4").tobytes(), "I32"
        header[name] = {"dtype": kind, "shape": list(t.shape), "data_offsets": [at, at + len(raw)]}
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
