"""``Betepel`` as a list of parts. Tensor names: ``embed``, ``embed.norm``, ``final.norm``, and per layer ``i``
``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.<name>`` (``l<i>.mix.{left,right}.<name>`` for a pair) and ``l<i>.mlp.<name>``;
the head is the embedding table. Every layer is the ``parallel_norms`` arrangement around a 32-bit residual
stream (mixer and feed-forward side by side behind norms whose weights are stored around zero); its mixer is
a matrix memory, differential attention (which may read an earlier layer's cache) or a pair of windowed
attention and decayed linear attention; its feed-forward a mixture of experts chosen by a table, or absent."""

from __future__ import annotations

from typing import Optional

from ..config.betepel import BetepelAttention, BetepelConfig, BetepelMemory
from ..config.registry import register_architecture
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry


def build_betepel_spec(cfg: BetepelConfig) -> ModelSpec:
    w, eps = cfg.width, cfg.norm_eps

    def norm(name: str, prefix: str) -> PartSpec:
        return PartSpec("rms_norm", dict(width=w, eps=eps, weight_name=name, unit_offset=True), prefix)

    def position(a: BetepelAttention) -> Optional[PartSpec]:
        r = a.rot
        if r is None:
            return None
        if r.factor == 1.0 and not r.original:
            return PartSpec("rotary", dict(dim=r.dims, theta=r.base, pairing="half"))
        return PartSpec("rotary", dict(dim=r.dims, theta=r.base, pairing="half", rope_type="llama3", factor=r.factor,
                                       low_freq_factor=r.low, high_freq_factor=r.high,
                                       original_max_position_embeddings=r.original))

    def kept_keys(i: int) -> Optional[int]:
        """What layer ``i``'s pages must keep for itself and for the layers that read them: every key (0) if one of
        them sees every earlier position or keeps first positions, else the longest of their windows."""
        readers = [cfg.layers[i].attention] + [l.attention for l in cfg.layers if l.type == "attention" and l.attention.kv_from == i]
        if len(readers) == 1:
            return None
        return 0 if any(not a.window or a.keep_first for a in readers) else max(a.window for a in readers)

    def attention(a: BetepelAttention, prefix: str, cache_window: Optional[int] = None) -> PartSpec:
        params = dict(hidden_size=w, num_heads=a.heads, num_kv_heads=a.kv_heads, head_dim=a.dim, value_dim=a.vdim,
                      scale=a.scale, qk_unit=False, position=position(a), window=a.window, keep_first=a.keep_first,
                      bias=True, norm_eps=eps)
        if a.diff is not None:
            params.update(maps=2, diff=a.diff, head_gate=True, own_kv=a.kv_from is None, cache_window=cache_window)
        return PartSpec("scored_attention", params, prefix)

    def memory(m: BetepelMemory, prefix: str) -> PartSpec:
        if m.decay:
            return PartSpec("decayed_linear", dict(hidden_size=w, num_heads=m.heads, head_dim=m.dim, value_dim=m.vdim,
                                                   decay=m.decay, norm_eps=eps), prefix)
        return PartSpec("matrix_memory", dict(hidden_size=w, num_heads=m.heads, head_dim=m.dim, value_dim=m.vdim,
                                              gate_cap=m.gate_cap, norm_eps=eps), prefix)

    layers, schedule = [], []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        if layer.type == "mlstm":
            mixer = memory(layer.memory, p + "mix.")
        elif layer.type == "attention":
            mixer = attention(layer.attention, p + "mix.", kept_keys(i) if layer.attention.kv_from is None else None)
        else:
            mixer = PartSpec("parallel_mixers", dict(
                hidden_size=w, combine="weighted_sum", scales={"left": layer.left_scale, "right": layer.right_scale},
                branches={"left": attention(layer.attention, p + "mix.left."), "right": memory(layer.memory, p + "mix.right.")}),
                p + "mix.")
        parts = {"mixer": ("mixer", mixer), "mixer_norm": ("norm", norm("norm1", p))}
        f = layer.mlp
        if f is not None:
            parts["feed_forward"] = ("feed_forward", PartSpec("routed_experts", dict(
                hidden_size=w, experts=f.experts, top=f.top, expert_size=f.ff, limit=float("inf"), alpha=1.0, up_shift=0.0,
                correction=False, routing="table", vocab_size=cfg.vocab, shared_size=f.shared_ff,
                shared_limit=float("inf"), shared_gate=False), p + "mlp."))
            parts["feed_forward_norm"] = ("norm", norm("norm2", p))
        layers.append(LayerSpec(block=PartSpec("parallel_norms"), parts=parts))
        kv_from = layer.attention.kv_from if layer.type == "attention" else None
        schedule.append(ScheduleEntry(i, cache_of=kv_from))
    return ModelSpec(
        architecture=cfg.architecture, vocab_size=cfg.vocab, hidden_size=w,
        embedding=PartSpec("token_embedding", dict(vocab_size=cfg.vocab, hidden_size=w, weight_name="embed",
                                                   float32_rows=True, norm=norm("norm", "embed."))),
        layers=tuple(layers), schedule=tuple(schedule), final_norm=norm("norm", "final."),
        head=PartSpec("linear_head", dict(vocab_size=cfg.vocab, hidden_size=w, tied=True, scale=cfg.logit_scale)))


register_architecture("Betepel", BetepelConfig.from_dict, build_betepel_spec, model_types=("betepel",), replace=True)
