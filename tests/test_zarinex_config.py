"""Zarinex without a GPU: the configuration's reader, the list of parts it becomes, tensor names and
shapes against the plain implementation's own table, layers that run another layer's weights, and the
plain implementation's mechanisms against their definitions."""

from __future__ import annotations

import copy

import pytest
import torch

import plain_zarinex as P

F = torch.float64


def cfg_dict():
    moe = {"kind": "moe", "expert": {"ff": 20}, "router": {"experts": 7, "top": 2}, "shared": {"ff": 28}}
    bare = {"kind": "moe", "expert": {"ff": 12}, "router": {"experts": 3, "top": 3}}
    att = {"heads": 3, "dim": 8, "vdim": 12, "kv_rank": 20, "q_rank": 24, "scale": 0.3}
    scan = {"inner": 40, "state": 5, "dt_rank": 3, "conv": 4}
    lin = {"heads": 2, "dim": 8, "vdim": 6}
    return {"architecture": "Zarinex", "vocab": 50, "width": 48, "norm": {"eps": 1e-5}, "postln_alpha": 1.5,
            "layers": [{"type": "mamba1", "mixer": scan, "mlp": moe},
                       {"type": "latent_attention", "mixer": att, "mlp": None},
                       {"type": "hgrn2", "mixer": lin, "mlp": bare},
                       {"type": "latent_attention", "mixer": att, "mlp": None, "weights_of": 1},
                       {"type": "mamba1", "mixer": scan, "mlp": moe, "weights_of": 0}]}


def build(raw):
    from dli_amd.config.registry import resolve_architecture
    from dli_amd.parts import Runtime
    from dli_amd.parts.model import Model
    import dli_amd.architectures  # noqa: F401

    arch = resolve_architecture(raw)
    cfg = arch.parse_config(raw)
    return cfg, Model(arch.build_spec(cfg), Runtime(torch.device("cpu"), torch.float32))


def test_a_layer_that_names_a_borrower_runs_the_owners_tensors():
    raw = cfg_dict()
    raw["layers"].append({"type": "mamba1", "mixer": raw["layers"][0]["mixer"], "mlp": raw["layers"][0]["mlp"], "weights_of": 4})
    cfg, model = build(raw)
    assert [l.weights_of for l in cfg.layers] == [None, None, None, 1, 0, 0]
    assert [e.layer for e in model.spec.schedule] == [0, 1, 2, 1, 0, 0]


def test_config_is_read_and_becomes_parts():
    from dli_amd.parts import CompositeCacheSpec, PagedKVSpec, StateSpec

    cfg, model = build(cfg_dict())
    assert cfg.architecture == "Zarinex" and (cfg.vocab, cfg.width, cfg.norm_eps, cfg.postln_alpha) == (50, 48, 1e-5, 1.5)
    assert [l.type for l in cfg.layers] == ["mamba1", "latent_attention", "hgrn2", "latent_attention", "mamba1"]
    assert [l.weights_of for l in cfg.layers] == [None, None, None, 1, 0]
    m = cfg.layers[0].mlp
    assert (m.experts, m.top, m.ff, m.shared_ff) == (7, 2, 20, 28) and cfg.layers[2].mlp.shared_ff == 0
    assert cfg.layers[1].mlp is None
    # three layers have tensors; the schedule runs five
    assert len(model.layers) == 3 and [e.layer for e in model.spec.schedule] == [0, 1, 2, 1, 0]
    mixers = [l.parts["mixer"] for l in model.layers]
    assert all(x.kind == "token_shifted" for x in mixers)
    assert [x.inner.kind for x in mixers] == ["selective_scan", "latent_attention", "gated_linear"]
    att = mixers[1].inner
    assert (att.num_heads, att.head_dim, att.value_dim, att.kv_rank, att.q_rank, att.scale, att.output_gate) == \
        (3, 8, 12, 20, 24, 0.3, True)
    scan = mixers[0].inner
    assert (scan.inner, scan.states, scan.dt_rank, scan.taps) == (40, 5, 3, 4)
    assert [type(l.parts.get("feed_forward")).__name__ for l in model.layers] == ["RoutedExperts", "NoneType", "RoutedExperts"]
    assert all(l.block.kind == "post_norm" and l.block.alpha == 1.5 and l.block.gated for l in model.layers)
    shift = ("shift", StateSpec((48,), torch.float32))
    specs = model.cache_specs()
    assert len(specs) == 5
    assert specs[0] == specs[4] == CompositeCacheSpec((shift, ("inner", StateSpec((40 * 5 + 3 * 40,), torch.float32))))
    assert specs[1] == specs[3] == CompositeCacheSpec((shift, ("inner", PagedKVSpec(1, 20, 0))))
    assert specs[2] == CompositeCacheSpec((shift, ("inner", StateSpec((2 * 6 * 8,), torch.float32))))
    assert model.head.tied and model.embedding.float32_rows


def test_a_scale_left_out_is_the_usual_one():
    raw = cfg_dict()
    for l in raw["layers"]:
        l["mixer"] = dict(l["mixer"])
        l["mixer"].pop("scale", None)
    cfg, _ = build(raw)
    assert cfg.layers[1].mixer["scale"] == 8 ** -0.5


def test_tensor_names_and_shapes_are_the_plain_table():
    raw = cfg_dict()
    _, model = build(raw)
    table = P.tensor_shapes(raw)
    specs = model.weight_specs()
    assert set(specs) == set(table)
    assert not any(n.startswith(("l3.", "l4.")) for n in specs)
    for name, shape in table.items():
        assert specs[name].fits(tuple(shape)), (name, shape, specs[name].shape)


def test_what_is_not_implemented_is_refused():
    from dli_amd.config.errors import ConfigError

    def broken(change):
        raw = copy.deepcopy(cfg_dict())
        change(raw)
        with pytest.raises(ConfigError):
            build(raw)

    broken(lambda r: r["layers"][0].__setitem__("type", "mamba2"))
    broken(lambda r: r["layers"][0]["mixer"].pop("state"))
    broken(lambda r: r["layers"][1]["mixer"].__setitem__("kv_rank", 0))
    broken(lambda r: r["layers"][0]["mlp"].__setitem__("kind", "dense"))
    broken(lambda r: r["layers"][0]["mlp"]["router"].__setitem__("top", 8))          # more than there are experts
    broken(lambda r: r["layers"][3].__setitem__("weights_of", 3))                     # itself
    broken(lambda r: r["layers"][3].__setitem__("weights_of", 4))                     # leads to a layer of another kind
    broken(lambda r: (r["layers"][0].__setitem__("weights_of", 4), None))             # 0 -> 4 -> 0: nobody has the tensors
    broken(lambda r: r["layers"][3].__setitem__("weights_of", 2))                     # a layer of another kind
    broken(lambda r: r["layers"][3].__setitem__("weights_of", "1"))
    broken(lambda r: r["layers"][4].__setitem__("mixer", dict(r["layers"][4]["mixer"], inner=44)))               # other sizes than its source
    broken(lambda r: r.pop("width"))
    broken(lambda r: r.pop("norm"))


def test_plain_mechanisms_agree_with_their_definitions():
    torch.manual_seed(0)
    # token shift: the first row mixes with zeros, a later one with the row before as it was
    h, mu = torch.randn(3, 4, dtype=F), torch.rand(4, dtype=F)
    st = {}
    out = P.token_shift(h, mu, st)
    assert torch.allclose(out[0], h[0] * (1 - mu)) and torch.allclose(out[2], h[2] + (h[1] - h[2]) * mu)
    assert torch.equal(st["prev"], h[2])
    more = P.token_shift(h[:1], mu, st)
    assert torch.allclose(more[0], h[0] + (h[2] - h[0]) * mu)
    # the convolution's last column belongs to the current token, zeros before the start
    x, w = torch.randn(4, 2, dtype=F), torch.randn(2, 3, dtype=F)
    st = {}
    y = P.causal_conv(x, w, None, st)
    assert torch.allclose(y[0], w[:, 2] * x[0]) and torch.allclose(y[2], w[:, 2] * x[2] + w[:, 1] * x[1] + w[:, 0] * x[0])
    assert torch.equal(st["conv"], x[2:])
    # one token of the selective scan from a zero state: y = dt x (B . C) + D x
    xs, dt = torch.randn(1, 3, dtype=F), torch.rand(1, 3, dtype=F)
    B, C = torch.randn(1, 5, dtype=F), torch.randn(1, 5, dtype=F)
    ys, S = P.selective_scan(xs, dt, B, C, torch.randn(3, 5, dtype=F), torch.ones(3, dtype=F) * 2, None)
    assert torch.allclose(ys[0], dt[0] * xs[0] * (B[0] @ C[0]) + 2 * xs[0])
    # the gated linear recurrence writes (1 - f) v: with f = 0 the state is the last token's alone
    q, v = torch.randn(2, 1, 4, dtype=F), torch.randn(2, 1, 3, dtype=F)
    o, S = P.gated_linear(q, torch.zeros(2, 1, 4, dtype=F), v, None)
    assert torch.allclose(o[1, 0], v[1, 0] * q[1, 0].sum())
    # the router's weights are the softmax over the chosen logits alone, the lower index first on a tie
    order, wts = P.route(torch.tensor([0.5, 2.0, 2.0, -1.0], dtype=F), 2)
    assert order == [1, 2] and torch.allclose(wts, torch.tensor([0.5, 0.5], dtype=F))
    # positions: pairs of sine and cosine of one angle
    pv = P.position_vectors(torch.tensor([0, 3]), 6)
    assert torch.allclose(pv[0], torch.tensor([0, 1, 0, 1, 0, 1], dtype=F))
    assert torch.allclose(pv[1, 2], torch.sin(torch.tensor(3 * 10000.0 ** (-2 / 6), dtype=F)))


def test_the_plain_model_stepped_is_the_plain_model_whole():
    raw = cfg_dict()
    W = P.random_weights(raw, 3)
    toks = [(7 * i + 3) % 50 for i in range(23)]
    m = P.PlainZarinex(raw, W)
    whole = m.forward(toks)
    st = m.new_state()
    parts, at = [], 0
    for n in (1, 2, 5, 1, 1, 13):
        parts.append(m.forward(toks[at:at + n], st, start=at))
        at += n
    assert (torch.cat(parts) - whole).abs().max() < 1e-9
