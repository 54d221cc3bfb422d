"""Betepel without a GPU: the configuration's reader and its refusals, the list of parts it becomes, tensor
names and shapes against the plain implementation's own table, the layer that reads another's cache, and
the plain implementation's mechanisms against their definitions."""

from __future__ import annotations

import copy
import math

import pytest
import torch

import plain_betepel as P

F = torch.float64


def cfg_dict():
    moe = {"kind": "moe", "expert": {"ff": 20}, "router": {"experts": 5, "top": 2}, "shared": {"ff": 28}}
    bare = {"kind": "moe", "expert": {"ff": 12}, "router": {"experts": 3, "top": 3}}
    rot = {"dims": 4, "base": 300.0, "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 40}}
    att = {"heads": 4, "kv_heads": 2, "dim": 8, "vdim": 12, "scale": 0.4, "diff": 0.3, "mask": {"size": 11, "keep_first": 3}, "rot": rot}
    left = {"heads": 3, "kv_heads": 1, "dim": 8, "vdim": 6, "scale": 0.35, "mask": {"size": 9}, "rot": {"dims": 8, "base": 100.0}}
    right = {"heads": 2, "dim": 8, "vdim": 10, "decay": [0.7, 0.98]}
    mem = {"heads": 3, "dim": 8, "vdim": 6, "gate_cap": 6.0}
    return {"architecture": "Betepel", "vocab": 50, "width": 48, "norm": {"eps": 1e-5}, "logit_scale": 0.5,
            "layers": [{"type": "mlstm", "mixer": mem, "mlp": moe},
                       {"type": "attention", "mixer": att, "mlp": None},
                       {"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": 0.7, "right_scale": 1.3}, "mlp": bare},
                       {"type": "attention", "mixer": dict(att, kv_from=1, mask={"size": 5}), "mlp": moe}]}


def build(raw):
    from dli_amd.config.registry import resolve_architecture
    from dli_amd.parts import Runtime
    from dli_amd.parts.model import Model
    import dli_amd.architectures  # noqa: F401

    arch = resolve_architecture(raw)
    cfg = arch.parse_config(raw)
    return cfg, Model(arch.build_spec(cfg), Runtime(torch.device("cpu"), torch.float32))


def test_config_is_read_and_becomes_parts():
    from dli_amd.parts import CompositeCacheSpec, PagedKVSpec, StateSpec

    cfg, model = build(cfg_dict())
    assert cfg.architecture == "Betepel" and (cfg.vocab, cfg.width, cfg.norm_eps, cfg.logit_scale) == (50, 48, 1e-5, 0.5)
    assert [l.type for l in cfg.layers] == ["mlstm", "attention", "parallel", "attention"]
    a = cfg.layers[1].attention
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.scale, a.diff, a.window, a.keep_first, a.kv_from) == (4, 2, 8, 12, 0.4, 0.3, 11, 3, None)
    assert (a.rot.dims, a.rot.base, a.rot.factor, a.rot.low, a.rot.high, a.rot.original) == (4, 300.0, 4.0, 1.0, 4.0, 40)
    b = cfg.layers[3].attention
    assert (b.kv_from, b.window, b.keep_first) == (1, 5, 0)
    l = cfg.layers[2]
    assert (l.left_scale, l.right_scale, l.attention.diff, l.attention.window, l.memory.decay) == (0.7, 1.3, None, 9, (0.7, 0.98))
    assert cfg.layers[0].memory.gate_cap == 6.0 and cfg.layers[1].mlp is None
    m = cfg.layers[0].mlp
    assert (m.experts, m.top, m.ff, m.shared_ff) == (5, 2, 20, 28) and cfg.layers[2].mlp.shared_ff == 0
    # the borrowing layer is a schedule entry that reads the other's cache and keeps none
    assert [(e.layer, e.cache_of) for e in model.spec.schedule] == [(0, None), (1, None), (2, None), (3, 1)]
    specs = model.cache_specs()
    assert isinstance(specs[0], StateSpec) and specs[0].shape == (3 * (6 + 1) * 8 + 3,)
    # two maps a head: twice the key heads, one value head per kv head; kept positions give no page back
    assert specs[1] == PagedKVSpec(4, 8, 0, 12, 2)
    assert isinstance(specs[2], CompositeCacheSpec)
    assert dict(specs[2].members)["left"] == PagedKVSpec(1, 8, 9, 6) and dict(specs[2].members)["right"].shape == (2 * 10 * 8,)
    assert specs[3] is None
    assert model.layers[3].parts["mixer"].window == 5 and model.layers[1].parts["mixer"].keep_first == 3
    assert model.layers[1].parts["feed_forward"] if "feed_forward" in model.layers[1].parts else True
    assert "feed_forward" not in model.layers[1].parts and model.head.scale == 0.5
    assert model.graph_capturable(16)


def test_tensor_names_and_shapes_match_the_plain_table():
    raw = cfg_dict()
    _, model = build(raw)
    specs = model.weight_specs()
    want = P.tensor_shapes(raw)
    assert set(specs) == set(want)
    for name, shape in want.items():
        assert tuple(specs[name].shape) == tuple(shape), name
    assert specs["l0.mlp.table"].role == "int32" and specs["l1.mix.lq1"].role == "float32"
    assert "l3.mix.k" not in specs and "l3.mix.v.b" not in specs and "l1.norm2" not in specs


def test_absent_keys_have_their_plain_meaning():
    raw = cfg_dict()
    att = raw["layers"][1]["mixer"]
    for key in ("kv_heads", "vdim", "scale", "mask", "rot"):
        att.pop(key)
    raw["layers"][3]["mixer"] = dict(att, kv_from=1)
    raw.pop("logit_scale")
    raw["layers"][0]["mixer"].pop("gate_cap")
    raw["layers"][2]["mixer"].pop("left_scale")
    cfg, model = build(raw)
    a = cfg.layers[1].attention
    assert (a.kv_heads, a.vdim, a.window, a.keep_first, a.rot) == (4, 8, 0, 0, None) and abs(a.scale - 8 ** -0.5) < 1e-12
    assert cfg.logit_scale == 1.0 and cfg.layers[0].memory.gate_cap == 0.0 and cfg.layers[2].left_scale == 1.0
    assert model.layers[1].parts["mixer"].position.rotary_table() is None
    plain = dict(cfg_dict()["layers"][2]["mixer"]["left"]["rot"])
    assert model.layers[2].parts["mixer"].branches["left"].position.dim == plain["dims"]


@pytest.mark.parametrize("change,error", [
    (lambda r: r["layers"][0].update(type="gru"), "type"),
    (lambda r: r["layers"][1]["mixer"].update(heads=3), "group"),
    (lambda r: r["layers"][1]["mixer"]["mask"].update(chunk=4), "mask"),
    (lambda r: r["layers"][1]["mixer"]["rot"].update(dims=10), "dims"),
    (lambda r: r["layers"][1]["mixer"]["rot"]["scaling"].update(kind="yarn"), "scaling"),
    (lambda r: r["layers"][1]["mixer"].pop("diff"), "diff"),
    (lambda r: r["layers"][3]["mixer"].update(kv_from=3), "kv_from"),
    (lambda r: r["layers"][3]["mixer"].update(kv_from=0), "kv_from"),
    (lambda r: r["layers"][3]["mixer"].update(vdim=16), "differ"),
    (lambda r: r["layers"][2]["mixer"]["right"].update(decay=[0.5]), "decay"),
    (lambda r: r["layers"][2]["mixer"]["left"]["mask"].update(keep_first=2), "mask"),
    (lambda r: r["layers"][0]["mlp"].update(kind="dense"), "kind"),
    (lambda r: r["layers"][0]["mlp"]["router"].update(top=6), "chosen"),
    (lambda r: r.pop("width"), "width"),
])
def test_what_is_not_implemented_is_refused(change, error):
    from dli_amd.config.errors import ConfigError

    raw = copy.deepcopy(cfg_dict())
    change(raw)
    with pytest.raises((ConfigError, KeyError)) as exc:
        build(raw)
    assert error in str(exc.value)


def test_a_chain_of_borrowers_is_refused():
    from dli_amd.config.errors import ConfigError

    raw = cfg_dict()
    raw["layers"].append(copy.deepcopy(raw["layers"][3]))
    raw["layers"][4]["mixer"]["kv_from"] = 3
    with pytest.raises(ConfigError):
        build(raw)


def test_random_weights_mode_draws_a_table_of_distinct_experts(tmp_path):
    from dli_amd.weights import write_random_model
    from dli_amd.weights.safetensors_io import SafetensorsFile

    folder = write_random_model(tmp_path / "m", cfg_dict(), seed=3)
    f = SafetensorsFile(folder / "model.safetensors")
    import numpy as np
    table = np.array(f.get("l2.mlp.table").bits)
    f.close()
    assert table.shape == (50, 3) and table.min() == 0 and table.max() == 2
    assert all(len(set(row)) == 3 for row in table.tolist())


# ------------------------------------------------------------------------------ the plain mechanisms

def test_plain_window_keeps_the_first_positions():
    mask = {"size": 4, "keep_first": 2}
    assert [j for j in range(12) if P.visible(9, j, mask)] == [0, 1, 6, 7, 8, 9]
    assert [j for j in range(12) if P.visible(9, j, {"size": 4})] == [6, 7, 8, 9]
    assert [j for j in range(5) if P.visible(3, j, None)] == [0, 1, 2, 3]


def test_plain_rotation_turns_pairs_half_apart_and_leaves_the_rest():
    rot = {"dims": 4, "base": 100.0}
    x = torch.arange(1, 7, dtype=F).view(1, 1, 6).repeat(2, 1, 1)
    y = P.rotate(x, torch.tensor([0, 3]), rot)
    assert torch.equal(y[0], x[0]) and torch.equal(y[1, 0, 4:], x[1, 0, 4:])
    f = [1.0, 100.0 ** -0.5]
    for i in range(2):
        a = 3 * f[i]
        assert abs(float(y[1, 0, i]) - (x[1, 0, i] * math.cos(a) - x[1, 0, i + 2] * math.sin(a))) < 1e-12
        assert abs(float(y[1, 0, i + 2]) - (x[1, 0, i + 2] * math.cos(a) + x[1, 0, i] * math.sin(a))) < 1e-12


def test_plain_matrix_memory_equals_its_sums_written_out():
    """Without the reference point: S_t = sum_s (prod_(r>s) sigma(f_r)) e^(i_s) k_s v_s^T, and the same for n."""
    torch.manual_seed(0)
    n, H, D, V = 7, 2, 3, 4
    q, k, v = torch.randn(n, H, D, dtype=F), torch.randn(n, H, D, dtype=F), torch.randn(n, H, V, dtype=F)
    i, fpre = torch.randn(n, H, dtype=F), torch.randn(n, H, dtype=F)
    f = P.log_sigmoid(fpre)
    got = P.matrix_memory(q, k, v, i, f, {})
    for t in range(n):
        for h in range(H):
            S, nn, m = torch.zeros(D, V, dtype=F), torch.zeros(D, dtype=F), 0.0
            logs = []
            for s in range(t + 1):
                logs.append(float(i[s, h] + f[s + 1:t + 1, h].sum()))
            m = max(max(logs), float(f[:t + 1, h].sum()))       # the reference point started at 0
            for s in range(t + 1):
                S += math.exp(logs[s] - m) * torch.outer(k[s, h], v[s, h])
                nn += math.exp(logs[s] - m) * k[s, h]
            den = max(abs(float(nn @ q[t, h])), math.exp(-m)) + 1e-6
            assert ((S.t() @ q[t, h]) / den - got[t, h]).abs().max() < 1e-10


def test_plain_model_steps_like_it_runs_whole():
    raw = cfg_dict()
    W = P.random_weights(raw, 3)
    m = P.PlainBetepel(raw, W)
    toks = [int(t) for t in torch.randint(0, 50, (30,))]
    whole = m.forward(toks)
    states, rows, at = m.new_state(), [], 0
    for n in (1, 1, 5, 2, 13, 1, 7):
        rows.append(m.forward(toks[at:at + n], states, start=at))
        at += n
    assert (torch.cat(rows) - whole).abs().max() < 1e-9
