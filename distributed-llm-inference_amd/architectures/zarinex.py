"""``Zarinex`` as a list of parts. Tensor names: ``embed``, ``final.norm``, and per layer ``i`` that has tensors
of its own ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.shift``, ``l<i>.rg1`` (+ ``.b``), ``l<i>.rg2`` (+ ``.b``),
``l<i>.mix.<name>`` and ``l<i>.mlp.<name>``; the head is the embedding table. Every layer is the
``post_norm`` arrangement around a 32-bit residual stream, its mixer behind a token shift. A layer that
runs another's weights is that layer once more in the schedule, with a cache and state of its own."""

from __future__ import annotations

from ..config.registry import register_architecture
from ..config.zarinex import ZarinexConfig
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry


def build_zarinex_spec(cfg: ZarinexConfig) -> ModelSpec:
    w, eps = cfg.width, cfg.norm_eps
    layers: list[LayerSpec] = []
    built: dict[int, int] = {}     # the configuration's layer -> its place among the layers that have tensors
    schedule: list[ScheduleEntry] = []
    for i, layer in enumerate(cfg.layers):
        if layer.weights_of is not None:
            continue
        p, m = f"l{i}.", layer.mixer
        if layer.type == "mamba1":
            inner = PartSpec("selective_scan", dict(hidden_size=w, inner_size=m["inner"], state_size=m["state"],
                                                    dt_rank=m["dt_rank"], conv_taps=m["conv"]), p + "mix.")
        elif layer.type == "latent_attention":
            inner = PartSpec("latent_attention", dict(hidden_size=w, num_heads=m["heads"], head_dim=m["dim"],
                                                      value_dim=m["vdim"], kv_rank=m["kv_rank"], q_rank=m["q_rank"],
                                                      scale=m["scale"], norm_eps=eps, output_gate=True), p + "mix.")
        else:
            inner = PartSpec("gated_linear", dict(hidden_size=w, num_heads=m["heads"], head_dim=m["dim"],
                                                  value_dim=m["vdim"], norm_eps=eps), p + "mix.")
        mixer = PartSpec("token_shifted", dict(hidden_size=w, inner=inner, weight_name="shift"), p)
        parts = {"mixer": ("mixer", mixer),
                 "mixer_norm": ("norm", PartSpec("rms_norm", dict(width=w, eps=eps, weight_name="norm1"), p))}
        f = layer.mlp
        if f is not None:
            parts["feed_forward"] = ("feed_forward", PartSpec("routed_experts", dict(
                hidden_size=w, experts=f.experts, top=f.top, expert_size=f.ff, limit=float("inf"), alpha=1.0, up_shift=0.0,
                correction=False, router_bias=True, shared_size=f.shared_ff, shared_limit=float("inf"), shared_gate=False),
                p + "mlp."))
            parts["feed_forward_norm"] = ("norm", PartSpec("rms_norm", dict(width=w, eps=eps, weight_name="norm2"), p))
        block = PartSpec("post_norm", dict(hidden_size=w, alpha=cfg.postln_alpha, gated=True,
                                           feed_forward=f is not None), p)
        built[i] = len(layers)
        layers.append(LayerSpec(block=block, parts=parts))
    for i, layer in enumerate(cfg.layers):
        schedule.append(ScheduleEntry(built[i if layer.weights_of is None else layer.weights_of]))
    return ModelSpec(
        architecture=cfg.architecture, vocab_size=cfg.vocab, hidden_size=w,
        embedding=PartSpec("sinusoidal_token_embedding", dict(vocab_size=cfg.vocab, hidden_size=w, weight_name="embed")),
        layers=tuple(layers), schedule=tuple(schedule),
        final_norm=PartSpec("rms_norm", dict(width=w, eps=eps, weight_name="norm"), "final."),
        head=PartSpec("linear_head", dict(vocab_size=cfg.vocab, hidden_size=w, tied=True)))


register_architecture("Zarinex", ZarinexConfig.from_dict, build_zarinex_spec, model_types=("zarinex",), replace=True)
