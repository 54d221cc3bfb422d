"""Typed configuration of the Zarinex decoder: a list of layers, each ``x <- norm1(alpha x + r1 * mixer(shift(x)))``
then ``x <- norm2(alpha x + r2 * ff(x))`` (norms after the sums, token shift in front of the mixer, a sigmoid
gate on every sublayer's result), with one of three mixers (a selective scan, attention through a latent, a
gated linear recurrence) and a mixture of experts with a shared expert, or no feed-forward. Sinusoidal
positions are added to the embedding; the head is the embedding table. A layer may run another layer's
weights with a cache and state of its own.

``config.json`` keys: ``vocab``, ``width``, ``norm.eps``, ``postln_alpha`` and ``layers``: a list of
``{"type", "mixer": {...}, "mlp": {...} | null, "weights_of": j (optional)}``. Mixer keys by type:
``mamba1``: ``inner``, ``state``, ``dt_rank``, ``conv``;
``latent_attention``: ``heads``, ``dim``, ``vdim``, ``kv_rank``, ``q_rank``, ``scale`` (absent: ``dim ** -0.5``);
``hgrn2``: ``heads``, ``dim``, ``vdim``.
``mlp``: ``{"kind": "moe", "expert": {ff}, "router": {experts, top}, "shared": {ff} | absent}``.
"""

from __future__ import annotations

from dataclasses import dataclass, replace
from typing import Any, Mapping, Optional

from .errors import UnsupportedModelError
from .makodra import _need, _positive

MIXER_TYPES = ("mamba1", "latent_attention", "hgrn2")


@dataclass(frozen=True)
class ZarinexMLP:
    ff: int
    experts: int
    top: int
    shared_ff: int = 0          # 0: no shared expert

    @staticmethod
    def parse(raw: Mapping[str, Any], where: str) -> "ZarinexMLP":
        kind = raw.get("kind", "moe")
        if kind != "moe":
            raise UnsupportedModelError(f"{where}.kind={kind!r}; known: 'moe'")
        expert, router = _need(raw, "expert", where), _need(raw, "router", where)
        experts = _positive(_need(router, "experts", where + ".router"), where + ".router.experts")
        top = _positive(_need(router, "top", where + ".router"), where + ".router.top")
        if top > experts:
            raise UnsupportedModelError(f"{where}.router: {top} of {experts} experts cannot be chosen")
        shared = raw.get("shared")
        return ZarinexMLP(ff=_positive(_need(expert, "ff", where + ".expert"), where + ".expert.ff"), experts=experts, top=top,
                          shared_ff=_positive(_need(shared, "ff", where + ".shared"), where + ".shared.ff") if shared else 0)


@dataclass(frozen=True)
class ZarinexLayer:
    type: str
    mixer: Mapping[str, Any]        # the mixer's sizes and constants, checked for its type
    mlp: Optional[ZarinexMLP]
    weights_of: Optional[int] = None

    @staticmethod
    def parse(raw: Mapping[str, Any], index: int) -> "ZarinexLayer":
        where = f"layers[{index}]"
        kind = _need(raw, "type", where)
        if kind not in MIXER_TYPES:
            raise UnsupportedModelError(f"{where}.type={kind!r}; known: {MIXER_TYPES}")
        m = dict(_need(raw, "mixer", where))
        w = where + ".mixer"
        if kind == "mamba1":
            sizes = {k: _positive(_need(m, k, w), f"{w}.{k}") for k in ("inner", "state", "dt_rank", "conv")}
        elif kind == "latent_attention":
            sizes = {k: _positive(_need(m, k, w), f"{w}.{k}") for k in ("heads", "dim", "kv_rank", "q_rank")}
            sizes["vdim"] = _positive(m.get("vdim") or sizes["dim"], w + ".vdim")
            sizes["scale"] = float(m["scale"]) if m.get("scale") is not None else sizes["dim"] ** -0.5
        else:
            sizes = {k: _positive(_need(m, k, w), f"{w}.{k}") for k in ("heads", "dim")}
            sizes["vdim"] = _positive(m.get("vdim") or sizes["dim"], w + ".vdim")
        mlp = raw.get("mlp")
        source = raw.get("weights_of")
        if source is not None and (isinstance(source, bool) or not isinstance(source, int)):
            raise UnsupportedModelError(f"{where}.weights_of={source!r} must name a layer by its number")
        return ZarinexLayer(type=kind, mixer=sizes, mlp=ZarinexMLP.parse(mlp, where + ".mlp") if mlp is not None else None,
                            weights_of=source)


@dataclass(frozen=True)
class ZarinexConfig:
    vocab: int
    width: int
    norm_eps: float
    postln_alpha: float
    layers: tuple[ZarinexLayer, ...]

    architecture = "Zarinex"

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
    def from_dict(cls, raw: Mapping[str, Any]) -> "ZarinexConfig":
        layers = _need(raw, "layers", "")
        if not isinstance(layers, list) or not layers:
            raise UnsupportedModelError("layers must be a list with at least one layer")
        norm = _need(raw, "norm", "")
        parsed = [ZarinexLayer.parse(l, i) for i, l in enumerate(layers)]
        for i, layer in enumerate(parsed):
            j = layer.weights_of
            if j is None:
                continue
            # a layer that names one which itself runs another's tensors runs those: follow to the owner
            seen = {i}
            while isinstance(j, int) and 0 <= j < len(parsed) and j not in seen and parsed[j].weights_of is not None:
                seen.add(j)
                j = parsed[j].weights_of
            if not 0 <= j < len(parsed) or j in seen:
                raise UnsupportedModelError(f"layers[{i}].weights_of={layer.weights_of} must lead to another layer that has tensors of its own")
            if (parsed[j].type, dict(parsed[j].mixer), parsed[j].mlp) != (layer.type, dict(layer.mixer), layer.mlp):
                raise UnsupportedModelError(f"layers[{i}] runs the weights of layers[{j}] but differs from it in its sizes")
            if j != layer.weights_of:
                parsed[i] = replace(layer, weights_of=j)
        parsed = tuple(parsed)
        return cls(vocab=_positive(_need(raw, "vocab", ""), "vocab"), width=_positive(_need(raw, "width", ""), "width"),
                   norm_eps=float(_need(norm, "eps", "norm")), postln_alpha=float(raw.get("postln_alpha", 1.0)),
                   layers=parsed)
