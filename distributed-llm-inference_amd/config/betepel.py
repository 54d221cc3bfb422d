"""Typed configuration of the Betepel decoder: a normalised embedding, then a list of layers in each of
which a mixer and a feed-forward read the same stream behind norms of their own (norm weights stored
around zero), a 32-bit residual stream, and a head tied to the embedding whose logits are scaled. The
mixer is a matrix memory with exponential gates (``mlstm``), differential attention under a sliding window
that keeps the first positions (``attention``, which may read another layer's keys and values), or a pair
side by side (``parallel``): windowed rotary attention and linear attention with a constant decay per head.
The feed-forward is a mixture of experts that a table chooses by token id, plus a shared expert.

``config.json`` keys: ``vocab``, ``width``, ``norm.eps``, ``logit_scale`` (absent: 1) and ``layers``: a list of
``{"type", "mixer": {...}, "mlp": {...} | null}``. Mixer keys by type:
``mlstm``: ``heads``, ``dim``, ``vdim``, ``gate_cap``;
``attention``: ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``, ``diff``, ``mask.{size, keep_first}``,
``rot.{dims, base, scaling.{factor, low, high, original}}``, ``kv_from`` (an earlier attention layer of the same
head counts and rotation that has keys and values of its own);
``parallel``: ``left`` (``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``, ``mask.size``, ``rot``), ``right`` (``heads``,
``dim``, ``vdim``, ``decay``: a number per head), ``left_scale``, ``right_scale``.
Absent ``mask`` (or ``mask.size``): every earlier position is seen; absent ``rot``: no rotation; absent
``rot.scaling``: the plain frequencies; absent ``kv_heads``: as many as heads; absent ``vdim``: ``dim``.
``mlp``: ``{"kind": "moe", "expert": {ff}, "router": {experts, top}, "shared": {ff} | absent}``.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional

from .errors import UnsupportedModelError
from .makodra import _need, _positive

LAYER_TYPES = ("mlstm", "attention", "parallel")
MLP_KINDS = ("moe",)


def _number(value: Any, name: str) -> float:
    if isinstance(value, bool) or not isinstance(value, (int, float)):
        raise UnsupportedModelError(f"{name}={value!r} must be a number")
    return float(value)


def _unknown(d: Mapping[str, Any], known: tuple, where: str) -> None:
    extra = sorted(set(d) - set(known))
    if extra:
        raise UnsupportedModelError(f"{where} has keys that are not implemented: {extra}")


@dataclass(frozen=True)
class BetepelRotation:
    dims: int
    base: float
    factor: float = 1.0        # 1: the plain frequencies
    low: float = 1.0
    high: float = 4.0
    original: int = 0

    @staticmethod
    def parse(rot: Optional[Mapping[str, Any]], dim: int, where: str) -> Optional["BetepelRotation"]:
        if not rot:
            return None
        _unknown(rot, ("dims", "base", "scaling"), where)
        dims = _positive(_need(rot, "dims", where), where + ".dims")
        if dims % 2 or dims > dim:
            raise UnsupportedModelError(f"{where}.dims={dims} must be even and at most dim={dim}")
        base = _number(_need(rot, "base", where), where + ".base")
        sc = rot.get("scaling")
        if not sc:
            return BetepelRotation(dims, base)
        _unknown(sc, ("factor", "low", "high", "original"), where + ".scaling")
        factor = _number(_need(sc, "factor", where + ".scaling"), where + ".scaling.factor")
        low, high = _number(sc.get("low", 1.0), where + ".scaling.low"), _number(sc.get("high", 4.0), where + ".scaling.high")
        if not factor > 0 or not high > low:
            raise UnsupportedModelError(f"{where}.scaling: factor must be positive and high above low")
        return BetepelRotation(dims, base, factor, low, high,
                               _positive(_need(sc, "original", where + ".scaling"), where + ".scaling.original"))


@dataclass(frozen=True)
class BetepelAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int = 0            # mask.size (0: every earlier position is seen)
    keep_first: int = 0        # mask.keep_first
    rot: Optional[BetepelRotation] = None
    diff: Optional[float] = None     # differential attention's constant; None: one score map a head
    kv_from: Optional[int] = None

    @staticmethod
    def parse(m: Mapping[str, Any], where: str, differential: bool) -> "BetepelAttention":
        heads = _positive(_need(m, "heads", where), where + ".heads")
        kv = _positive(m.get("kv_heads") or heads, where + ".kv_heads")
        if heads % kv:
            raise UnsupportedModelError(f"{where}: {heads} heads do not group onto {kv} kv_heads")
        dim = _positive(_need(m, "dim", where), where + ".dim")
        mask = dict(m.get("mask") or {})
        _unknown(mask, ("size", "keep_first") if differential else ("size",), where + ".mask")
        window = _positive(mask["size"], where + ".mask.size") if mask.get("size") is not None else 0
        keep = int(mask.get("keep_first") or 0)
        if keep < 0:
            raise UnsupportedModelError(f"{where}.mask.keep_first={keep} must not be negative")
        kv_from = m.get("kv_from")
        if kv_from is not None and (isinstance(kv_from, bool) or not isinstance(kv_from, int) or kv_from < 0):
            raise UnsupportedModelError(f"{where}.kv_from={kv_from!r} must name a layer")
        return BetepelAttention(
            heads=heads, kv_heads=kv, dim=dim, vdim=_positive(m.get("vdim") or dim, where + ".vdim"),
            scale=_number(m["scale"], where + ".scale") if m.get("scale") is not None else dim ** -0.5,
            window=window, keep_first=keep if window else 0, rot=BetepelRotation.parse(m.get("rot"), dim, where + ".rot"),
            diff=_number(_need(m, "diff", where), where + ".diff") if differential else None,
            kv_from=kv_from if differential else None)


@dataclass(frozen=True)
class BetepelMemory:
    """``mlstm`` and the right side of ``parallel``: heads with keys of ``dim`` and values of ``vdim``."""
    heads: int
    dim: int
    vdim: int
    gate_cap: float = 0.0
    decay: tuple = ()

    @staticmethod
    def parse(m: Mapping[str, Any], where: str, decayed: bool) -> "BetepelMemory":
        heads = _positive(_need(m, "heads", where), where + ".heads")
        dim = _positive(_need(m, "dim", where), where + ".dim")
        vdim = _positive(m.get("vdim") or dim, where + ".vdim")
        if not decayed:
            return BetepelMemory(heads, dim, vdim, gate_cap=_number(m.get("gate_cap") or 0.0, where + ".gate_cap"))
        decay = _need(m, "decay", where)
        if not isinstance(decay, (list, tuple)) or len(decay) != heads:
            raise UnsupportedModelError(f"{where}.decay must hold a number for each of the {heads} heads")
        return BetepelMemory(heads, dim, vdim, decay=tuple(_number(d, where + ".decay") for d in decay))


@dataclass(frozen=True)
class BetepelMLP:
    experts: int
    top: int
    ff: int
    shared_ff: int = 0         # 0: no shared expert

    @staticmethod
    def parse(raw: Mapping[str, Any], where: str) -> "BetepelMLP":
        kind = raw.get("kind", "moe")
        if kind not in MLP_KINDS:
            raise UnsupportedModelError(f"{where}.kind={kind!r}; known: {MLP_KINDS}")
        expert, router = _need(raw, "expert", where), _need(raw, "router", where)
        experts = _positive(_need(router, "experts", where + ".router"), where + ".router.experts")
        top = _positive(_need(router, "top", where + ".router"), where + ".router.top")
        if top > min(experts, 64):
            raise UnsupportedModelError(f"{where}.router: {top} of {experts} experts cannot be chosen (at most 64)")
        shared = raw.get("shared")
        return BetepelMLP(experts=experts, top=top, ff=_positive(_need(expert, "ff", where + ".expert"), where + ".expert.ff"),
                          shared_ff=_positive(_need(shared, "ff", where + ".shared"), where + ".shared.ff") if shared else 0)


@dataclass(frozen=True)
class BetepelLayer:
    type: str
    attention: Optional[BetepelAttention] = None     # attention; parallel: the left side
    memory: Optional[BetepelMemory] = None           # mlstm; parallel: the right side
    left_scale: float = 1.0
    right_scale: float = 1.0
    mlp: Optional[BetepelMLP] = None

    @staticmethod
    def parse(raw: Mapping[str, Any], index: int) -> "BetepelLayer":
        where = f"layers[{index}]"
        kind = _need(raw, "type", where)
        if kind not in LAYER_TYPES:
            raise UnsupportedModelError(f"{where}.type={kind!r}; known: {LAYER_TYPES}")
        m = _need(raw, "mixer", where)
        mlp = BetepelMLP.parse(raw["mlp"], where + ".mlp") if raw.get("mlp") is not None else None
        w = where + ".mixer"
        if kind == "mlstm":
            return BetepelLayer(kind, memory=BetepelMemory.parse(m, w, False), mlp=mlp)
        if kind == "attention":
            return BetepelLayer(kind, attention=BetepelAttention.parse(m, w, True), mlp=mlp)
        return BetepelLayer(kind, attention=BetepelAttention.parse(_need(m, "left", w), w + ".left", False),
                            memory=BetepelMemory.parse(_need(m, "right", w), w + ".right", True),
                            left_scale=_number(m.get("left_scale", 1.0), w + ".left_scale"),
                            right_scale=_number(m.get("right_scale", 1.0), w + ".right_scale"), mlp=mlp)


@dataclass(frozen=True)
class BetepelConfig:
    vocab: int
    width: int
    norm_eps: float
    logit_scale: float
    layers: tuple[BetepelLayer, ...]

    architecture = "Betepel"

    # the names under which the engine's tools ask any configuration for its common sizes
    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "BetepelConfig":
        layers = _need(raw, "layers", "")
        if not isinstance(layers, list) or not layers:
            raise UnsupportedModelError("layers must be a list with at least one layer")
        parsed = tuple(BetepelLayer.parse(l, i) for i, l in enumerate(layers))
        for i, layer in enumerate(parsed):
            a = layer.attention
            if layer.type != "attention" or a.kv_from is None:
                continue
            src = parsed[a.kv_from] if a.kv_from < i else None
            if src is None or src.type != "attention" or src.attention.kv_from is not None:
                raise UnsupportedModelError(f"layers[{i}].mixer.kv_from={a.kv_from} must name an earlier attention layer "
                                            "with keys and values of its own")
            b = src.attention
            if (a.heads, a.kv_heads, a.dim, a.vdim, a.rot) != (b.heads, b.kv_heads, b.dim, b.vdim, b.rot):
                raise UnsupportedModelError(f"layers[{i}] reads the keys of layers[{a.kv_from}], whose head counts, sizes "
                                            "or rotation differ")
        return cls(vocab=_positive(_need(raw, "vocab", ""), "vocab"), width=_positive(_need(raw, "width", ""), "width"),
                   norm_eps=_number(_need(_need(raw, "norm", ""), "eps", "norm"), "norm.eps"),
                   logit_scale=_number(raw.get("logit_scale", 1.0), "logit_scale"), layers=parsed)
