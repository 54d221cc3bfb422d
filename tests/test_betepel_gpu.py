"""Betepel on the GPU against the plain float64 implementation of ``plain_betepel.py``: every
mechanism's kernel alone, then whole models of several small shapes through the engine's step
function, cache manager, scheduler and entry points, however the requests are cut and batched.
"""

from __future__ import annotations

import math
import random

import pytest
import torch

import plain_betepel as P

pytestmark = pytest.mark.gpu
F = torch.float64


def i32(values):
    return torch.tensor(list(values), dtype=torch.int32).cuda()


@pytest.fixture(scope="module")
def ops():
    from dli_amd.kernels import ops as o

    o.library()
    return o


def step_arrays(entries):
    """``entries``: (slot, first position, rows) of a step -> q_start, positions, state_slots on the device."""
    starts, pos = [0], []
    for _, p0, n in entries:
        starts.append(starts[-1] + n)
        pos += list(range(p0, p0 + n))
    return i32(starts), i32(pos), i32([e[0] for e in entries])


def in_steps(requests, plan, run):
    """Walks ``plan`` (steps of (request, rows)) over ``requests`` (name -> (slot, rows tensor)): ``run(rows,
    q_start, positions, slots)`` gets the step's stacked rows and returns the step's results, which are
    handed back request by request, in order."""
    at = {r: 0 for r in requests}
    got = {r: [] for r in requests}
    for step in plan:
        entries, rows = [], []
        for r, n in step:
            slot, x = requests[r]
            entries.append((slot, at[r], n))
            rows.append(x[at[r]:at[r] + n])
        out = run(torch.cat(rows).cuda(), *step_arrays(entries))
        r0 = 0
        for r, n in step:
            got[r].append(out[r0:r0 + n].cpu())
            r0 += n
            at[r] += n
    assert all(at[r] == requests[r][1].shape[0] for r in requests)
    return {r: torch.cat(v) for r, v in got.items()}


# a plan over three requests through two slots: "c" starts in "a"'s slot once "a" has ended
PLAN = [[("a", 3), ("b", 1)], [("a", 1), ("b", 4)], [("b", 1), ("a", 2)], [("a", 17), ("b", 2)], [("a", 1)], [("a", 40), ("b", 30)],
        [("c", 1), ("b", 1)], [("c", 1)], [("c", 2), ("b", 35)], [("c", 60)]]
LENGTHS = {"a": 64, "b": 74, "c": 64}
SLOTS = {"a": 1, "b": 0, "c": 1}


# ------------------------------------------------------------------------------ small kernels

def test_norm_with_a_weight_stored_around_zero(ops):
    from dli_amd.parts.base import Runtime
    from dli_amd.parts.norm import RMSNorm

    torch.manual_seed(0)
    for width in (40, 200, 1030):
        for dtype in (torch.float32, torch.bfloat16):
            norm = RMSNorm(Runtime(torch.device("cuda"), dtype), width=width, eps=1e-4, weight_name="w", unit_offset=True)
            w = (0.3 * torch.randn(width)).to(torch.bfloat16).float()
            norm.load_weights({"w": w.cuda()})
            x = 3 * torch.randn(7, width)
            ref = P.offset_norm(x.double(), w.double(), 1e-4)
            assert (norm.forward_f32(x.cuda()).cpu().double() - ref).abs().max() < 5e-6 * ref.abs().max()
            tol = 5e-6 if dtype == torch.float32 else 6e-3
            assert (norm.forward(x.cuda()).cpu().double() - ref).abs().max() < tol * ref.abs().max()


def test_two_maps_become_one_head_by_head(ops):
    torch.manual_seed(1)
    for heads, vdim in ((3, 24), (1, 70), (5, 1), (2, 130)):
        a = torch.randn(6, 2 * heads * vdim)
        gate = torch.randn(6, heads + 3)
        lam, diff, eps = 0.37, 0.3, 1e-4
        a1, a2 = a.double()[:, :heads * vdim].view(6, heads, vdim), a.double()[:, heads * vdim:].view(6, heads, vdim)
        ref = P.rms(a1 - lam * a2, eps) * (1 - diff) * P.sigmoid(gate.double()[:, 2:2 + heads])[:, :, None]
        for dtype, tol in ((torch.float32, 5e-6), (torch.bfloat16, 6e-3)):
            out = torch.empty(6, heads * vdim, dtype=dtype).cuda()
            ops.diff_head_norm(a.cuda(), lam, 1 - diff, eps, gate.cuda()[:, 2:2 + heads], out, heads, vdim)
            assert (out.cpu().double().view(6, heads, vdim) - ref).abs().max() < tol * ref.abs().max()
        out = torch.empty(6, heads * vdim).cuda()
        ops.diff_head_norm(a.cuda(), lam, 1.0, eps, None, out, heads, vdim)
        assert (out.cpu().double().view(6, heads, vdim) - P.rms(a1 - lam * a2, eps)).abs().max() < 5e-6 * ref.abs().max() * 4


def test_sum_of_branches_with_constants(ops):
    torch.manual_seed(2)
    ys = [torch.randn(9, 70) for _ in range(3)]
    wide = torch.randn(9, 100)
    out = torch.empty(9, 70).cuda()
    ops.branch_weighted_sum([ys[0].cuda(), wide.cuda()[:, 30:], ys[2].cuda()], [0.8, -0.5, 2.0], out)
    ref = 0.8 * ys[0].double() - 0.5 * wide.double()[:, 30:] + 2.0 * ys[2].double()
    assert (out.cpu().double() - ref).abs().max() < 1e-5


def test_a_table_names_each_tokens_experts(ops):
    table = torch.stack([torch.randperm(7)[:3] for _ in range(50)]).to(torch.int32)
    toks = torch.randint(0, 50, (40,), dtype=torch.int32)
    ids, w = torch.empty(40, 3, dtype=torch.int32).cuda(), torch.empty(40, 3).cuda()
    ops.table_choose(table.cuda(), toks.cuda(), ids, w)
    assert torch.equal(ids.cpu(), table[toks.long()])
    assert torch.allclose(w.cpu(), torch.full((40, 3), 1 / 3))


def test_scaled_frequencies_in_three_bands():
    """The part's table against the plain frequencies: wavelengths below, between and above the two bounds."""
    from dli_amd.parts.position import rotary_inverse_frequencies

    rot = {"dims": 32, "base": 50000.0, "scaling": {"factor": 6.0, "low": 1.5, "high": 3.0, "original": 200}}
    ref = P.rotary_frequencies(rot)
    got = rotary_inverse_frequencies(32, 50000.0, "llama3", 6.0, 1.5, 3.0, 200)
    assert (torch.from_numpy(got).double() - ref).abs().max() < 1e-7 * ref.max()
    kinds = {("kept" if 2 * math.pi / f < 200 / 3.0 else "divided" if 2 * math.pi / f > 200 / 1.5 else "blended") for f in
             P.rotary_frequencies({"dims": 32, "base": 50000.0}).tolist()}
    assert kinds == {"kept", "divided", "blended"}
    plain = rotary_inverse_frequencies(10, 777.0)
    assert (torch.from_numpy(plain).double() - P.rotary_frequencies({"dims": 10, "base": 777.0})).abs().max() < 1e-7


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rotation_with_biases_writes_fewer_value_heads_than_key_heads(ops, dtype):
    torch.manual_seed(3)
    n, qh, kh, vh, d, dv, ps, rot_dims = 9, 6, 4, 2, 24, 10, 4, 16
    cols = qh * d + kh * d + vh * dv
    proj, bias = torch.randn(n, cols + 5), torch.randn(cols + 5)
    rot = {"dims": rot_dims, "base": 100.0}
    pos = torch.tensor([0, 1, 2, 700, 701, 5, 9000, 3, 4])
    slots = torch.tensor([4, 5, 6, 20, 21, 9, 13, -1, 2])
    kp, vp = torch.zeros(8, kh, ps, d, dtype=dtype).cuda(), torch.zeros(8, vh, dv, ps, dtype=dtype).cuda()
    q = torch.empty(n, qh * d, dtype=dtype).cuda()
    inv = P.rotary_frequencies(rot).float().cuda()
    ops.rotary_cache(proj.cuda(), 0, qh * d, (qh + kh) * d, i32(pos.tolist()), inv, rot_dims, False, q, i32(slots.tolist()), kp, vp,
                     qh, bias=bias.cuda())
    full = proj.double() + bias.double()
    q_ref = P.rotate(full[:, :qh * d].view(n, qh, d), pos, rot)
    k_ref = P.rotate(full[:, qh * d:(qh + kh) * d].view(n, kh, d), pos, rot)
    v_ref = full[:, (qh + kh) * d:cols].view(n, vh, dv)
    tol = 1e-4 if dtype == torch.float32 else 2e-2    # (32-bit frequencies: an angle at position 9000 is good to 1e-3)
    assert (q.cpu().double().view(n, qh, d) - q_ref).abs().max() < tol * q_ref.abs().max()
    for t in range(n):
        s = int(slots[t])
        if s < 0:
            continue
        assert (kp[s // ps, :, s % ps].cpu().double() - k_ref[t]).abs().max() < tol * k_ref.abs().max()
        assert (vp[s // ps, :, :, s % ps].cpu().double() - v_ref[t]).abs().max() < tol * v_ref.abs().max()
    # without pages only the queries are made
    q2 = torch.empty(n, qh * d, dtype=dtype).cuda()
    ops.rotary_cache(proj.cuda(), 0, 0, 0, i32(pos.tolist()), inv, rot_dims, False, q2, None, None, None, qh, bias=bias.cuda())
    assert torch.equal(q2, q)


# ------------------------------------------------------------------------------ recurrences under scalar gates

def plain_memory(q, k, v, gi, gf, ib, fb, cap, dim):
    i = cap * torch.tanh((gi + ib) / cap) if cap else gi + ib
    f = cap * torch.tanh((gf + fb) / cap) if cap else gf + fb
    return P.matrix_memory(q * dim ** -0.5, k, v, i, P.log_sigmoid(f), {})


@pytest.mark.parametrize("chunked", [True, False])
@pytest.mark.parametrize("H,D,V,cap", [(2, 8, 6, 15.0), (4, 32, 48, 4.0), (1, 64, 16, 0.0), (3, 20, 70, 8.0), (2, 128, 3, 15.0),
                                       (1, 16, 130, 2.0), (2, 48, 1, 30.0), (2, 64, 37, 15.0)])
def test_matrix_memory_in_steps_against_whole(ops, H, D, V, cap, chunked):
    """``chunked``: steps with portions run 64 tokens at a time on the matrix cores where the head's size allows."""
    g = torch.Generator().manual_seed(H * 100 + D)
    ib, fb = torch.randn(H, generator=g), torch.randn(H, generator=g) + 2.0
    width = 2 * H * D + H * V + 2 * H
    reqs = {r: (SLOTS[r], torch.cat([torch.randn(n, 2 * H * D + H * V, generator=g), 3 * torch.randn(n, 2 * H, generator=g)], 1))
            for r, n in LENGTHS.items()}
    floats = H * (V + 1) * D
    state = torch.full((3, floats + H + 4), 55.0).cuda()                        # rubbish where a slot was never used

    def run(rows, q_start, positions, slots):
        n = rows.shape[0]
        keep, write, floor, log_keep = ops.exp_gates(rows, width - 2 * H, width - H, ib.cuda(), fb.cuda(), cap, state, floats,
                                                     q_start, positions, slots, H)
        o, den = torch.empty(n, H * V).cuda(), torch.empty(n, H).cuda()
        ops.scalar_gate_scan(rows[:, :H * D], rows[:, H * D:2 * H * D], rows[:, 2 * H * D:2 * H * D + H * V], state, q_start,
                             positions, slots, o, H, D, V, keep=keep, write=write, floor=floor, den=den, log_keep=log_keep,
                             q_scale=D ** -0.5, chunked=chunked)
        return o.view(n, H, V) / den[:, :, None]

    got = in_steps(reqs, PLAN, run)
    for r, (_, x) in reqs.items():
        x = x.double()
        n = x.shape[0]
        ref = plain_memory(x[:, :H * D].view(n, H, D), x[:, H * D:2 * H * D].view(n, H, D),
                           x[:, 2 * H * D:2 * H * D + H * V].view(n, H, V), x[:, width - 2 * H:width - H], x[:, width - H:],
                           ib.double(), fb.double(), cap, D)
        # (a denominator |n . q| is a sum that cancels: its last bits are worth 1e-4 of a result)
        assert (got[r].double() - ref).abs().max() < 1e-4 * max(1.0, ref.abs().max()), (r, (got[r].double() - ref).abs().max())
    assert (state[:, floats + H:] == 55.0).all()


def test_the_reference_point_starts_at_zero_and_the_floor_holds_early(ops):
    """Strongly negative input gates at the first tokens: the result is bounded by exp(-m) with m from 0, not by |n . q|."""
    H, D, V = 1, 16, 4
    torch.manual_seed(5)
    n = 6
    q, k, v = torch.randn(n, H * D), torch.randn(n, H * D), torch.randn(n, H * V)
    gi, gf = torch.full((n, H), -9.0), torch.full((n, H), 3.0)
    rows = torch.cat([q, k, v, gi, gf], 1).cuda()
    state = torch.zeros(1, H * (V + 1) * D + H).cuda()
    qs, pos, sl = step_arrays([(0, 0, n)])
    keep, write, floor, log_keep = ops.exp_gates(rows, 2 * H * D + H * V, 2 * H * D + H * V + H, None, None, 0.0, state,
                                                 H * (V + 1) * D, qs, pos, sl, H)
    o, den = torch.empty(n, H * V).cuda(), torch.empty(n, H).cuda()
    ops.scalar_gate_scan(rows[:, :D], rows[:, D:2 * D], rows[:, 2 * D:2 * D + V], state, qs, pos, sl, o, H, D, V, keep=keep,
                         write=write, floor=floor, den=den, log_keep=log_keep, q_scale=D ** -0.5)
    ref = plain_memory(q.double().view(n, H, D), k.double().view(n, H, D), v.double().view(n, H, V), gi.double(), gf.double(),
                       torch.zeros(H, dtype=F), torch.zeros(H, dtype=F), 0.0, D)
    got = (o.view(n, H, V) / den[:, :, None]).cpu().double()
    assert (got - ref).abs().max() < 1e-6 * ref.abs().max() + 1e-9
    assert ref.abs().max() < 1e-2          # the floor, not the normaliser, decided


@pytest.mark.parametrize("inside", [True, False])
@pytest.mark.parametrize("H,D,V", [(2, 8, 6), (3, 64, 32), (1, 16, 130), (2, 20, 7), (2, 96, 1), (3, 48, 21)])
def test_decayed_linear_attention_in_steps_against_whole(ops, H, D, V, inside):
    """``inside``: silu inside the scan, token by token; else beforehand, and portions in chunks on the matrix cores."""
    g = torch.Generator().manual_seed(H * 10 + V)
    decay = torch.tensor([0.6, 0.97, 1.0][:H])
    reqs = {r: (SLOTS[r], torch.randn(n, 2 * H * D + H * V + 8, generator=g)) for r, n in LENGTHS.items()}
    state = torch.full((3, H * V * D + 3), -7.0).cuda()

    def run(rows, q_start, positions, slots):
        o = torch.empty(rows.shape[0], H * V).cuda()
        if not inside:
            rows = rows.clone()
            ops.silu_columns(rows[:, 8:])
        ops.scalar_gate_scan(rows[:, 8:8 + H * D], rows[:, 8 + H * D:8 + 2 * H * D], rows[:, 8 + 2 * H * D:], state, q_start, positions,
                             slots, o, H, D, V, decay=decay.cuda(), silu=inside)
        return o

    got = in_steps(reqs, PLAN, run)
    for r, (_, x) in reqs.items():
        x = P.silu(x.double()[:, 8:])
        n = x.shape[0]
        ref, _ = P.decayed_linear_attention(x[:, :H * D].view(n, H, D), x[:, H * D:2 * H * D].view(n, H, D),
                                            x[:, 2 * H * D:].view(n, H, V), decay.double(), None)
        assert (got[r].double().view(n, H, V) - ref).abs().max() < 2e-5 * max(1.0, ref.abs().max()), r
    assert (state[:, H * V * D:] == -7.0).all()


def test_a_state_written_long_ago_is_still_there(ops):
    """A head that never decays: what the first token wrote answers a query 400 single-token steps later."""
    H, D, V = 2, 16, 8
    decay = torch.tensor([0.5, 1.0]).cuda()
    state = torch.zeros(2, H * V * D).cuda()
    n = 400
    rows = torch.zeros(n, 2 * H * D + H * V)
    rows[0, H * D + D + 3] = 1.0                    # key 3 of head 1
    rows[0, 2 * H * D + V + 5] = 2.0                # value 5 of head 1
    rows[0, H * D + 3] = 1.0                        # the same on the decaying head 0
    rows[0, 2 * H * D + 5] = 2.0
    rows[n - 1, D + 3] = 1.0                        # the last query asks for key 3 on head 1
    rows[n - 1, 3] = 1.0
    rows = rows.cuda()
    o = torch.empty(n, H * V).cuda()
    qs, pos, sl = step_arrays([(1, 0, 37)])
    ops.scalar_gate_scan(rows[:37, :H * D], rows[:37, H * D:2 * H * D], rows[:37, 2 * H * D:], state, qs, pos, sl, o[:37], H, D, V,
                         decay=decay)
    for t in range(37, n):
        qs, pos, sl = step_arrays([(1, t, 1)])
        ops.scalar_gate_scan(rows[t:t + 1, :H * D], rows[t:t + 1, H * D:2 * H * D], rows[t:t + 1, 2 * H * D:], state, qs, pos, sl,
                             o[t:t + 1], H, D, V, decay=decay)
    assert abs(float(o[n - 1, V + 5]) - 2.0) < 1e-6 and abs(float(o[n - 1, 5])) < 1e-30
    assert float(o[n - 1].abs().sum()) - 2.0 < 1e-6


# ------------------------------------------------------------------------------ attention: windows, kept positions, shared values

def paged(x, page_size, dtype, order, transposed):
    """``x [tokens, heads, dim]`` into pages in the order of ``order`` (a shuffled list of page numbers)."""
    n, heads, dim = x.shape
    pages = max(order) + 1
    if transposed:
        out = torch.zeros(pages, heads, dim, page_size, dtype=dtype)
        for t in range(n):
            out[order[t // page_size], :, :, t % page_size] = x[t].to(dtype)
    else:
        out = torch.zeros(pages, heads, page_size, dim, dtype=dtype)
        for t in range(n):
            out[order[t // page_size], :, t % page_size] = x[t].to(dtype)
    return out.cuda()


def plain_maps(q, k, v, first, scale, mask, v_heads):
    """Key head ``g`` reads value head ``g % v_heads``."""
    kv = k.shape[1]
    vv = torch.stack([v[:, g % v_heads] for g in range(kv)], dim=1)
    return P.masked_attention(q, k, vv, first, scale, mask)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("qh,kh,vh,d,dv,window,keep", [(4, 2, 2, 16, 32, 24, 5), (8, 4, 2, 48, 16, 40, 20), (2, 2, 1, 32, 32, 9, 1),
                                                        (3, 1, 1, 20, 12, 30, 0), (4, 4, 2, 16, 96, 60, 66)])
def test_planted_keys_at_the_edges_of_window_and_kept_positions(ops, dtype, qh, kh, vh, d, dv, window, keep):
    """One key stands out for one query: the query must find it exactly where the mask lets it (inside the
    window, among the kept first positions) and nowhere else; through the tile kernel, the matrix-core kernel and
    the single-token kernel, with pages in shuffled order."""
    n, ps = 150, 4
    g = torch.Generator().manual_seed(qh * 31 + window)
    order = torch.randperm(n // ps + 3, generator=g).tolist()
    mask = {"size": window, "keep_first": keep}
    scale = 0.5
    k = 0.3 * torch.randn(n, kh, d, generator=g)
    v = torch.randn(n, vh, dv, generator=g)
    q = 0.3 * torch.randn(n, qh, d, generator=g)
    i = 130                                                 # the query that looks for planted keys
    planted = [i - window + 1, i - window, i - 1]           # just inside, just outside, near
    if keep:
        planted += [keep - 1, keep, 0]                      # the last kept, the first not kept, the first of all
    direction = torch.randn(d, generator=g)
    direction /= direction.norm()
    q[i] = 6.0 * direction
    for j in planted:
        k[j] = 3.0 * direction * (1 + 0.1 * planted.index(j))
        v[j] = 5.0 + planted.index(j)
    q, k, v = (t.to(torch.bfloat16).double() for t in (q, k, v))
    ref = plain_maps(q, k, v, 0, scale, mask, vh)
    # what the query at i finds: visible planted keys dominate, invisible ones leave no trace
    seen = [j for j in planted if P.visible(i, j, mask)]
    assert i - window not in seen and (not keep or keep not in seen) and i - window + 1 in seen
    kp, vp = paged(k, ps, dtype, order, False), paged(v, ps, dtype, order, True)
    table = i32(order + [0, 0]).view(1, -1)
    tol = 2e-5 if dtype == torch.float32 else 3e-2

    def check(out, rows, what):
        err = (out.cpu().double().view(-1, qh, dv) - ref[rows]).abs().max()
        assert err < tol * ref.abs().max(), (what, float(err))

    for out_dtype in {dtype, torch.float32}:
        qd = q.reshape(n, qh * d).to(dtype).cuda()
        # portions: the whole sequence at once, then its last 30 rows on top of the first 120
        for first in (0, 120):
            rows = slice(first, n)
            m = n - first
            tile_rows = ops.attention_generic_tile_rows(max(d, dv))
            ent, q0 = i32([0] * len(range(0, m, tile_rows))), i32(range(0, m, tile_rows))
            out = torch.empty(m, qh * dv, dtype=out_dtype).cuda()
            ops.attention_scored(qd[rows], kp, vp, out, i32([0, m]), i32([n]), table, ent, q0, qh, scale, window=window,
                                 keep_first=keep)
            check(out, rows, ("tiles", first, out_dtype))
            if dtype == torch.bfloat16 and ops.attention_scored_mfma_supports(d, dv, ps, dtype):
                ent, q0 = i32([0] * len(range(0, m, 64))), i32(range(0, m, 64))
                out = torch.empty(m, qh * dv, dtype=out_dtype).cuda()
                ops.attention_scored_mfma(qd[rows], kp, vp, out, i32([0, m]), i32([n]), table, ent, q0, qh, scale, window=window,
                                          keep_first=keep)
                check(out, rows, ("matrix cores", first, out_dtype))
        # single tokens: every position from 100 on as a step of its own, three at a time
        for t in range(100, n, 3):
            out = torch.empty(3, qh * dv, dtype=out_dtype).cuda()
            rows = [t, min(t + 1, n - 1), min(t + 2, n - 1)]
            ops.attention_scored(qd[rows], kp, vp, out, i32([0, 1, 2, 3]), i32([r + 1 for r in rows]), table.repeat(3, 1).contiguous(),
                                 None, None, qh, scale, window=window, keep_first=keep)
            check(out, rows, ("single", t, out_dtype))


# ------------------------------------------------------------------------------ whole models

def moe(experts, top, ff, shared=None):
    m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def config(width, vocab, scale, layers, eps=1e-5):
    return {"architecture": "Betepel", "vocab": vocab, "width": width, "norm": {"eps": eps}, "logit_scale": scale, "layers": layers}


def layer(kind, mixer, mlp):
    return {"type": kind, "mixer": dict(mixer), "mlp": mlp}


def _varied():
    rot = {"dims": 4, "base": 300.0, "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 40}}
    att = {"heads": 4, "kv_heads": 2, "dim": 8, "vdim": 12, "scale": 0.4, "diff": 0.3, "mask": {"size": 11, "keep_first": 3}, "rot": rot}
    left = {"heads": 3, "kv_heads": 1, "dim": 8, "vdim": 6, "scale": 0.35, "mask": {"size": 9}, "rot": {"dims": 8, "base": 100.0}}
    right = {"heads": 2, "dim": 8, "vdim": 10, "decay": [0.7, 0.98]}
    mem = {"heads": 3, "dim": 8, "vdim": 6, "gate_cap": 6.0}
    m = moe(5, 2, 20, 28)
    return config(48, 50, 0.5, [layer("mlstm", mem, m), layer("attention", att, m),
                                layer("parallel", {"left": left, "right": right, "left_scale": 0.7, "right_scale": 1.3}, m),
                                layer("attention", dict(att, kv_from=1, mask={"size": 5, "keep_first": 7}), moe(3, 3, 12)),
                                layer("mlstm", mem, m)])


def _aligned():
    """Sizes that the matrix-core kernels take; windows longer than a tile of keys; one expert a token."""
    rot = {"dims": 16, "base": 10000.0}
    att = {"heads": 2, "kv_heads": 1, "dim": 16, "vdim": 32, "scale": 0.25, "diff": 0.6, "mask": {"size": 70, "keep_first": 66}, "rot": rot}
    left = {"heads": 4, "kv_heads": 2, "dim": 32, "vdim": 16, "scale": 0.18, "mask": {"size": 130}, "rot": {"dims": 16, "base": 5000.0}}
    right = {"heads": 2, "dim": 32, "vdim": 32, "decay": [0.9, 0.999]}
    mem = {"heads": 2, "dim": 16, "vdim": 32, "gate_cap": 12.0}
    m = moe(4, 1, 32, 64)
    return config(64, 90, 1.0, [layer("attention", att, m),
                                layer("parallel", {"left": left, "right": right, "left_scale": 1.0, "right_scale": 0.25}, m),
                                layer("mlstm", mem, m), layer("attention", dict(att, kv_from=0), m)])


def _odd():
    """Sizes that nothing aligns, one head, as many kv heads as heads, no mask, no rotation, no cap, no shared expert, a layer
    without feed-forward, all experts chosen."""
    att = {"heads": 1, "dim": 12, "vdim": 5, "scale": 1.0, "diff": 0.1}
    att2 = {"heads": 3, "kv_heads": 3, "dim": 6, "vdim": 7, "diff": 0.8, "mask": {"size": 200}, "rot": {"dims": 2, "base": 3.0}}
    left = {"heads": 2, "dim": 10, "scale": 0.3}
    right = {"heads": 1, "dim": 20, "vdim": 70, "decay": [1.0]}
    mem = {"heads": 1, "dim": 20, "vdim": 3}
    return config(40, 33, 2.0, [layer("parallel", {"left": left, "right": right}, None), layer("attention", att, moe(2, 2, 10)),
                                layer("mlstm", mem, None), layer("attention", att2, moe(6, 1, 8, 8)),
                                layer("attention", dict(att, kv_from=1), None)], eps=1e-3)


CONFIGS = {"varied": _varied(), "aligned": _aligned()}
MORE_CONFIGS = {"odd": _odd()}
CONFIGS_ALL = {**CONFIGS, **MORE_CONFIGS}
_MODELS: dict = {}


def model(name: str, tmp_root):
    if name not in _MODELS:
        cfg = CONFIGS_ALL[name]
        W = P.random_weights(cfg, seed=len(name) * 7 + 1)
        if name == "aligned":                                   # sharp attention: a query's weight lies on few keys, near or far
            W = {k: (v * 3).to(torch.bfloat16).double() if k.endswith((".q", ".k")) and ".mix." in k and "right" not in k else v
                 for k, v in W.items()}
        _MODELS[name] = (cfg, W, P.write_folder(tmp_root / name, cfg, W))
    return _MODELS[name]


@pytest.fixture(scope="module")
def tmp_root(tmp_path_factory):
    return tmp_path_factory.mktemp("betepel")


def session(folder, dtype, pages=40, page_size=16, max_seqs=4, graphs=False):
    from dli_amd.engine.core import build_core
    from dli_amd.trace import TraceSession

    class Session(TraceSession):
        """Logits of a replayed graph are a view of its output buffer, good until the next step:
        the tests keep every step's rows, so they take copies."""

        def step(self, entries, end=()):
            return super().step(entries, end).clone()

    core = build_core(folder, num_pages=pages, page_size=page_size, max_seqs=max_seqs, dtype=dtype,
                      enable_prefix_caching=False, watermark=0.0)
    if graphs:
        core.step.enable_decode_graphs(max_seqs, pages * page_size)
    return Session(core)


_REFS: dict = {}


def reference(name, W, cfg, toks, dtype):
    """The plain logits, and how far each row moves when the matrices are jittered by bfloat16's rounding (the larger of
    two draws): what rounding of that size may do to the row. A difference of two attention maps, or a denominator
    that is a sum which cancels, makes a row here and there a hundred times more sensitive than its neighbours."""
    key = (name, tuple(toks))
    if key not in _REFS:
        ref = P.forward_logits(cfg, W, toks)
        moved = [(P.forward_logits(cfg, P.jittered(W, seed=j), toks) - ref).abs().max(dim=-1, keepdim=True).values for j in (0, 5)]
        _REFS[key] = (ref, torch.maximum(*moved))
    return _REFS[key]


def rows_of(ref, rows):
    return tuple(r[rows] for r in ref)


def close(got: torch.Tensor, ref, dtype: str, what) -> None:
    """In 32-bit every row is held, and that is where a fault of the cache, the state, a window or the table
    shows (it moves rows by 1e-2 and more); a row that a jitter of bfloat16's size moves by a tenth of its largest
    logit may be off by a thousandth of that. In bfloat16 a row may be off by bfloat16's usual share of its
    largest logit and a few times what such a jitter does to it."""
    ref, moved = ref
    got, ref = got.double().cpu(), ref.double()
    assert got.shape == ref.shape, what
    err = (got - ref).abs()
    top = ref.abs().max(dim=-1, keepdim=True).values.clamp(min=1.0)
    if dtype == "bfloat16":
        bad = (err > 8e-2 * top + 8 * moved).any(dim=-1)
        assert not bad.any(), (what, bad.nonzero().flatten().tolist())
        assert (err / top).max(dim=-1).values.median() < 4e-2, (what, (err / top).max(dim=-1).values.median())
        return
    assert (err <= 2e-4 * top + 1e-3 * moved).all(), (what, (err / top).max())
    assert (err / top).max(dim=-1).values.median() < 2e-5, (what, (err / top).max(dim=-1).values.median())


def prompt(cfg, n, seed):
    return [random.Random(seed * 1000 + i).randrange(cfg["vocab"]) for i in range(n)]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(CONFIGS_ALL))
def test_whole_prompt_and_the_first_tokens_alone(name, dtype, tmp_root):
    cfg, W, folder = model(name, tmp_root)
    toks = prompt(cfg, 70, 1)
    ref = reference(name, W, cfg, toks, dtype)
    s = session(folder, dtype)
    got = s.step([{"id": "a", "tokens": toks, "want": list(range(len(toks)))}], end=["a"])
    close(got, ref, dtype, name)
    one = s.step([{"id": "b", "tokens": toks[:1], "want": [0]}], end=["b"])   # the first token alone, in a's slot
    close(one, rows_of(ref, slice(0, 1)), dtype, name)
    two = s.step([{"id": "c", "tokens": toks[:2], "want": [0, 1]}], end=["c"])
    close(two, rows_of(ref, slice(0, 2)), dtype, name)
    s.core.manager.check_invariants()


def test_every_layer_against_the_plain_model(tmp_root):
    """The residual stream after each layer, in 32-bit, through a step of two portions."""
    cfg, W, folder = model("varied", tmp_root)
    toks = prompt(cfg, 40, 4)
    plain, layers = P.PlainBetepel(cfg, W), []
    plain.forward(toks, layers_out=layers)
    s = session(folder, "float32")
    seen = []
    m = s.core.model
    for built in m.layers:
        fwd = built.block.forward

        def spy(x, delta, ctx, cache, parts, fwd=fwd):
            out = fwd(x, delta, ctx, cache, parts)
            seen.append(out[0].clone())
            return out

        built.block.forward = spy
    s.step([{"id": "a", "tokens": toks[:25], "want": []}])
    s.step([{"id": "a", "tokens": toks[25:], "want": []}], end=["a"])
    n = len(cfg["layers"])
    for i in range(n):
        got = torch.cat([seen[i], seen[n + i]]).cpu().double()
        assert (got - layers[i]).abs().max() < 2e-5 * layers[i].abs().max(), i


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_long_prompt_whose_queries_look_far_back(dtype, tmp_root):
    """Sharp attention over 330 positions and twenty pages, windows that pass over kept positions and page
    borders, whole and with its last tokens one by one."""
    cfg, W, folder = model("aligned", tmp_root)
    toks = prompt(cfg, 330, 5)
    ref = reference("aligned", W, cfg, toks, dtype)
    s = session(folder, dtype, pages=48)
    got = s.step([{"id": "a", "tokens": toks, "want": list(range(len(toks)))}], end=["a"])
    close(got, ref, dtype, "whole")
    rows = [s.step([{"id": "b", "tokens": toks[:101], "want": [100]}])]
    for t in range(101, len(toks)):
        rows.append(s.step([{"id": "b", "tokens": toks[t:t + 1], "want": [0]}]))
    close(torch.cat(rows), rows_of(ref, slice(100, None)), dtype, "decoded")


@pytest.mark.parametrize("graphs", [False, True])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(CONFIGS))
def test_prefill_then_long_decoding_token_by_token(name, dtype, graphs, tmp_root):
    """A long run of single tokens crosses pages and windows; with graphs they are replayed."""
    if graphs and dtype == "float32":
        pytest.skip("decode graphs are recorded in bfloat16")
    cfg, W, folder = model(name, tmp_root)
    toks = prompt(cfg, 150, 2)
    ref = reference(name, W, cfg, toks, dtype)
    s = session(folder, dtype, graphs=graphs)
    rows = [s.step([{"id": "a", "tokens": toks[:19], "want": [0, 18]}])]
    for t in range(19, len(toks)):
        rows.append(s.step([{"id": "a", "tokens": toks[t:t + 1], "want": [0]}], end=["a"] if t + 1 == len(toks) else []))
    close(torch.cat(rows), rows_of(ref, [0] + list(range(18, len(toks)))), dtype, name)
    if graphs:
        assert s.core.step.graphs is not None and s.core.step.graphs.replays > 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(CONFIGS_ALL))
def test_decoding_from_the_first_token_on(name, dtype, tmp_root):
    """No prompt to speak of: one token, then single tokens across the kept positions and the first windows."""
    cfg, W, folder = model(name, tmp_root)
    toks = prompt(cfg, 90, 6)
    ref = reference(name, W, cfg, toks, dtype)
    s = session(folder, dtype, graphs=dtype == "bfloat16")
    rows = [s.step([{"id": "a", "tokens": toks[t:t + 1], "want": [0]}]) for t in range(len(toks))]
    close(torch.cat(rows), ref, dtype, name)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(CONFIGS_ALL))
def test_portions_of_every_size(name, dtype, tmp_root):
    cfg, W, folder = model(name, tmp_root)
    toks = prompt(cfg, 131, 3)
    ref = reference(name, W, cfg, toks, dtype)
    for sizes in ([2, 2, 3, 17, 2, 40, 1, 1, 5, 33, 2, 23], [64, 64, 3], [1] * 9 + [2] * 5 + [112]):
        assert sum(sizes) == len(toks)
        s = session(folder, dtype, pages=12, page_size=16, max_seqs=1)
        at, rows = 0, []
        for n in sizes:
            rows.append(s.step([{"id": 7, "tokens": toks[at:at + n], "want": list(range(n))}]))
            at += n
        close(torch.cat(rows), ref, dtype, (name, sizes))


@pytest.mark.parametrize("page_size", [16, 4])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(CONFIGS_ALL))
def test_mixed_batches_with_pages_and_slots_used_again(name, dtype, page_size, tmp_root):
    """Five unequal requests through two state slots and a pool that holds two of them at a time:
    portions of some beside single tokens of others, a request left out of steps; every request against
    itself alone."""
    cfg, W, folder = model(name, tmp_root)
    reqs = {i: prompt(cfg, n, 10 + i) for i, n in enumerate([90, 37, 1, 64, 55])}
    refs = {i: reference(name, W, cfg, t, dtype) for i, t in reqs.items()}
    s = session(folder, dtype, pages=192 // page_size, page_size=page_size, max_seqs=2, graphs=dtype == "bfloat16")
    plan = [[(0, 30), (1, 5)], [(0, 1), (1, 30)], [(0, 2), (1, 1)], [(1, 1), (0, 40)], [(0, 1)], [(0, 16), (2, 1)],
            [(3, 33)], [(3, 1)], [(3, 30), (4, 2)], [(4, 1)], [(4, 1)], [(4, 50)], [(4, 1)]]
    at = {i: 0 for i in reqs}
    got = {i: [] for i in reqs}
    for step in plan:
        entries, end = [], []
        for i, n in step:
            entries.append({"id": f"r{i}", "tokens": reqs[i][at[i]:at[i] + n], "want": list(range(n))})
            at[i] += n
            if at[i] == len(reqs[i]):
                end.append(f"r{i}")
        out = s.step(entries, end=end)
        r0 = 0
        for i, n in step:
            got[i].append(out[r0:r0 + n])
            r0 += n
        s.core.manager.check_invariants()
    for i in reqs:
        assert at[i] == len(reqs[i])
        close(torch.cat(got[i]), refs[i], dtype, (name, i))


def drawn_config(seed: int) -> dict:
    """A model whose sizes, order of layers, windows and constants are drawn from ``seed``."""
    rng = random.Random(seed)
    width, vocab = rng.choice([96, 128, 160, 192, 256]), rng.randrange(150, 700)

    def rotation(dim):
        if rng.random() < 0.15:
            return None
        rot = {"dims": rng.choice([d for d in (2, 4, 8, 12, 16, 24, 32, 48, 64) if d <= dim]), "base": rng.choice([100.0, 1e4, 5e5])}
        if rng.random() < 0.5:
            rot["scaling"] = {"factor": rng.choice([2.0, 8.0]), "low": 1.0, "high": rng.choice([2.0, 4.0]), "original": rng.choice([32, 64, 256])}
        return rot

    def heads_pair():
        kv = rng.choice([1, 2, 3])
        return kv * rng.choice([1, 2, 3]), kv

    def mlp():
        if rng.random() < 0.15:
            return None
        experts = rng.randrange(1, 9)
        return moe(experts, rng.randrange(1, min(experts, 3) + 1), rng.choice([16, 24, 32, 64]), rng.choice([None, 32, 48]))

    layers, lenders = [], []
    for i in range(rng.randrange(3, 7)):
        kind = rng.choice(["attention", "attention", "parallel", "mlstm"])
        if kind == "attention":
            if lenders and rng.random() < 0.5:
                mixer = dict(layers[rng.choice(lenders)]["mixer"], kv_from=None)
                mixer["kv_from"] = layers.index(next(l for l in layers if l["mixer"] is not mixer and l["type"] == "attention"
                                                        and l["mixer"].get("kv_from") is None and l["mixer"]["heads"] == mixer["heads"]
                                                        and l["mixer"]["dim"] == mixer["dim"] and l["mixer"]["vdim"] == mixer["vdim"]
                                                        and l["mixer"]["kv_heads"] == mixer["kv_heads"] and l["mixer"].get("rot") == mixer.get("rot")))
            else:
                h, kv = heads_pair()
                dim = rng.choice([16, 24, 32, 48, 64])
                mixer = {"heads": h, "kv_heads": kv, "dim": dim, "vdim": rng.choice([16, 32, 40, 64, 96]), "scale": dim ** -0.5 * rng.choice([1.0, 1.5]),
                         "diff": rng.choice([0.2, 0.5, 0.7]), "rot": rotation(dim)}
                if mixer["rot"] is None:
                    del mixer["rot"]
                lenders.append(i)
            mixer["mask"] = {"size": rng.randrange(5, 120), "keep_first": rng.choice([0, 1, 7, 20, 70])}
            if rng.random() < 0.1:
                del mixer["mask"]
        elif kind == "parallel":
            h, kv = heads_pair()
            dim = rng.choice([16, 32, 48, 64])
            left = {"heads": h, "kv_heads": kv, "dim": dim, "vdim": rng.choice([16, 32, 48]), "scale": dim ** -0.5, "mask": {"size": rng.randrange(5, 150)},
                    "rot": rotation(dim)}
            if left["rot"] is None:
                del left["rot"]
            rh = rng.randrange(1, 5)
            right = {"heads": rh, "dim": rng.choice([16, 24, 32, 64]), "vdim": rng.choice([8, 16, 32, 40]),
                     "decay": [rng.choice([0.6, 0.9, 0.97, 0.999, 1.0]) for _ in range(rh)]}
            mixer = {"left": left, "right": right, "left_scale": rng.choice([0.5, 1.0]), "right_scale": rng.choice([0.3, 1.2])}
        else:
            mixer = {"heads": rng.randrange(1, 5), "dim": rng.choice([16, 24, 32, 64]), "vdim": rng.choice([16, 32, 40, 64]),
                     "gate_cap": rng.choice([5.0, 15.0, 30.0])}
        layers.append(layer(kind, mixer, mlp()))
        layers[-1]["mixer"] = mixer          # (the same dictionary, so that a borrower finds its lender)
    return config(width, vocab, rng.choice([0.25, 1.0, 2.0]), layers, eps=rng.choice([1e-5, 1e-6]))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(8))
def test_models_of_drawn_sizes_whole_in_portions_decoded_and_mixed(seed, dtype, tmp_root):
    """Sizes, order of layers, windows, kept positions, rotations, tables and constants drawn at random: whole prompts, portions
    that change in size, a decoded tail, and two requests beside each other, each against the plain model."""
    name = f"drawn{seed}"
    if name not in _MODELS:
        cfg = drawn_config(seed)
        W = P.random_weights(cfg, seed=100 + seed)
        _MODELS[name] = (cfg, W, P.write_folder(tmp_root / name, cfg, W))
    cfg, W, folder = _MODELS[name]
    a, b = prompt(cfg, 170, 40 + seed), prompt(cfg, 61, 60 + seed)
    ra, rb = reference(name, W, cfg, a, dtype), reference(name, W, cfg, b, dtype)
    s = session(folder, dtype, pages=24, graphs=dtype == "bfloat16")
    close(s.step([{"id": "w", "tokens": a, "want": list(range(len(a)))}], end=["w"]), ra, dtype, (name, "whole"))
    rows, at = {"a": [], "b": []}, {"a": 0, "b": 0}
    toks = {"a": a, "b": b}
    plan = [[("a", 37)], [("a", 2), ("b", 30)], [("b", 1), ("a", 64)], [("a", 3), ("b", 1)], [("a", 40), ("b", 2)], [("b", 27)]]
    plan += [[("a", 1)]] * 24
    for step in plan:
        entries, end = [], []
        for r, n in step:
            entries.append({"id": r, "tokens": toks[r][at[r]:at[r] + n], "want": list(range(n))})
            at[r] += n
            if at[r] == len(toks[r]):
                end.append(r)
        out = s.step(entries, end=end)
        r0 = 0
        for r, n in step:
            rows[r].append(out[r0:r0 + n])
            r0 += n
    assert at == {"a": len(a), "b": len(b)}
    close(torch.cat(rows["a"]), ra, dtype, (name, "a"))
    close(torch.cat(rows["b"]), rb, dtype, (name, "b"))
    s.core.manager.check_invariants()


def test_a_row_does_not_depend_on_its_batch(tmp_root):
    """In 32-bit the logits of a request's rows are the same bits alone and beside others."""
    cfg, W, folder = model("varied", tmp_root)
    a, b, c = prompt(cfg, 40, 31), prompt(cfg, 23, 32), prompt(cfg, 9, 33)
    s = session(folder, "float32")
    alone = s.step([{"id": "a", "tokens": a, "want": list(range(40))}], end=["a"])
    s.step([{"id": "b", "tokens": b[:20], "want": []}])
    both = s.step([{"id": "b", "tokens": b[20:21], "want": [0]}, {"id": "a2", "tokens": a, "want": list(range(40))},
                   {"id": "c", "tokens": c, "want": [8]}], end=["a2", "b", "c"])
    assert torch.equal(alone, both[1:41])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_engine(dtype, tmp_root):
    """The engine's own entry points and scheduler: one request, then several at once."""
    from dli_amd.engine.generate import generate, greedy_generate
    from dli_amd.sampling import SamplingParams

    cfg, W, folder = model("varied", tmp_root)
    prompts = [prompt(cfg, n, 20 + n) for n in (9, 30, 3)]
    want = [P.greedy_generate(cfg, W, p, 12) for p in prompts]

    def same(got, ref, p):
        if got == ref:
            return
        # tokens may part only where the plain logits of the engine's own tokens are close
        logits = P.forward_logits(cfg, W, list(p) + got[:-1])
        for j, g in enumerate(got):
            row = logits[len(p) - 1 + j]
            assert (row.max() - row[g]).item() < (1e-3 if dtype == "float32" else 0.05) * row.abs().max().item(), (j, got, ref)

    same(greedy_generate(str(folder), prompts[0], 12, dtype=dtype, block_size=16), want[0], prompts[0])
    outs = generate(str(folder), prompts, SamplingParams(max_tokens=12), dtype=dtype, num_blocks=24, block_size=8,
                    max_num_seqs=2, max_num_batched_tokens=16, enable_prefix_caching=False)
    for got, ref, p in zip(outs, want, prompts):
        assert len(got) == 12
        same(got, ref, p)
