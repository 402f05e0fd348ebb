"""Lefisun on the GPU: each new mechanism's kernel alone against the plain implementation's function of
that mechanism, then the engine (cache, state slots, batches, portions, chunks, captured graphs, the entry
point) against the plain forward pass, in float32 and bfloat16."""
import copy
import json
import math
import os
import subprocess
import sys

import pytest
import torch

from helpers import max_live_tokens, replay_and_collect, trace_mixed, trace_portions, trace_tail, trace_whole
from lefisun_helpers import (CONFIGS, compare_rows, compare_with_rounding, middling_config, plain_logits, random_config, read_folder, requests_for,
                             rounding_noise, write_folder)
from plain import lefisun_plain as plain
from wllm_amd.engine import LLM, ModelRunner
from wllm_amd.engine.replay import TraceReplayer, pages_for_max_tokens
from wllm_amd.kernels import ops
from wllm_amd.parts import load_model

pytestmark = pytest.mark.gpu
DEV = "cuda"
DTYPES = [torch.float32, torch.bfloat16]
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LENGTHS = {"duo": [70, 45, 150, 33, 58], "odd": [40, 66, 25, 151], "sharp": [80, 137, 64, 50]}
FAMILIES = {"whole": trace_whole, "tail": trace_tail, "portions": trace_portions, "mixed": trace_mixed}
# a row's distance from the exact row, as a share of the row's own size or as a multiple of what rounding alone does to
# that row in the plain implementation (`rounding_noise`), whichever is larger: float32 sums in another order; bfloat16
# activations through some ten roundings a layer, and now and then a router or a key that the engine's rounding makes
# win where the plain implementation's does not (a row in some ten is then far off though nothing is wrong)
BOUND = {torch.float32: dict(relative=1e-4, times=6.0), torch.bfloat16: dict(relative=0.04, outliers=0.1)}
# (a long request: what a router's other choice changes stays in the memories' states and reaches every later row)
LONG_BOUND = {torch.float32: dict(relative=1e-4, times=6.0), torch.bfloat16: dict(relative=0.04, outliers=0.25)}
# the sharp model multiplies every rounding by some hundred (in float32 a lost key still moves a row by far more than
# this; in bfloat16 single keys and experts change places, and only the bulk of the rows says anything)
SHARP_BOUND = {torch.float32: dict(relative=6e-4), torch.bfloat16: dict(relative=0.3, outliers=0.25)}


def check_rows(got, folder, requests, exact, dtype, sharp=False, bound=None):
    bound = bound or (SHARP_BOUND if sharp else BOUND)
    return compare_with_rounding(got, exact, rounding_noise(folder, requests, dtype, exact), **bound[dtype])


def close(got, ref, dtype, what="", scale=1.0):
    atol, rtol = (3e-5 * scale, 3e-5) if dtype == torch.float32 else (1.5e-2 * scale, 1e-2)
    got, ref = got.double().cpu(), ref.double().cpu()
    err = ((got - ref).abs() / (atol + rtol * ref.abs())).max().item()
    assert err <= 1.0, f"{what}: worst error {err:.2f} x tolerance, max abs diff {(got - ref).abs().max().item():.3e}"


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("lefisun_gpu")
    return {name: write_folder(name, str(root / name)) for name in CONFIGS}


def _segments(lengths, generator, slots_total):
    q_len = torch.tensor(lengths, dtype=torch.int32)
    q_start = (torch.cumsum(q_len, 0) - q_len).to(torch.int32)
    slots = torch.randperm(slots_total, generator=generator)[:len(lengths)].to(torch.int32)
    return q_len, q_start, slots


# ---- mechanisms alone ---------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
def test_a_bias_in_front_of_the_norm_over_a_whole_projection(dtype):
    g = torch.Generator().manual_seed(3)
    n, q_cols, k_cols = 37, 44, 20
    row = torch.randn(n, q_cols + k_cols + 9, generator=g).to(dtype)
    wq, wk = 1.0 + 0.3 * torch.randn(q_cols, generator=g), 1.0 + 0.3 * torch.randn(k_cols, generator=g)
    bq, bk = torch.randn(q_cols, generator=g), torch.randn(k_cols, generator=g)
    dev = row.to(DEV)
    ops.band_norm([(dev[:, :q_cols], wq.to(DEV), q_cols, dev[:, :q_cols], bq.to(DEV)),
                   (dev[:, q_cols:q_cols + k_cols], wk.to(DEV), k_cols, dev[:, q_cols:q_cols + k_cols], bk.to(DEV))], 1e-5)
    r = row.double()
    close(dev[:, :q_cols], plain.rms_norm(r[:, :q_cols] + bq.double(), wq.double(), 1e-5), dtype, "queries")
    close(dev[:, q_cols:q_cols + k_cols], plain.rms_norm(r[:, q_cols:q_cols + k_cols] + bk.double(), wk.double(), 1e-5), dtype, "keys")
    assert torch.equal(dev[:, q_cols + k_cols:].cpu(), row[:, q_cols + k_cols:])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,d,dims,base,factor", [(3, 20, 6, 777.0, 1.0), (2, 64, 64, 1e6, 1.0), (1, 33, 2, 5.0, 8.0),
                                                      (5, 8, 0, 1.0, 1.0)])
def test_queries_and_keys_of_a_memory_are_turned_in_float32(dtype, heads, d, dims, base, factor):
    g = torch.Generator().manual_seed(d)
    n = 50
    row = torch.randn(n, 2 * heads * d + 5, generator=g).to(dtype)
    positions = torch.randint(0, 5000, (n,), generator=g).to(torch.int32)
    inv_freq = None
    if dims:
        inv_freq = (float(base) ** (-2.0 * torch.arange(dims // 2, dtype=torch.float64) / dims) / factor).float()
    qk = torch.zeros(2, n, heads * d, dtype=torch.float32, device=DEV)
    ops.memory_inputs(row.to(DEV), positions.to(DEV), inv_freq.to(DEV) if dims else None, qk, heads=heads, head_dim=d,
                      q_scale=0.5, k_scale=d ** -0.5)
    x = row[:, :2 * heads * d].double().view(n, 2 * heads, d)
    want = plain.rotate_half_split(x, positions, dims, base, factor) if dims else x
    want = want.reshape(n, 2, heads * d)
    # the angle is a float32 product of a position of some thousands: 1e-4 of a radian
    close(qk[0], want[:, 0] * 0.5, torch.float32, "queries", scale=30.0)
    close(qk[1], want[:, 1] * d ** -0.5, torch.float32, "keys", scale=30.0)


def _memory_weights(kind, heads, d, dv, g):
    """Weights that pick the columns of a row out again: the plain mixer, fed the projected row as its input,
    computes from exactly what the kernels read."""
    width = 2 * heads * d + 2 * heads * dv + (2 * heads if kind == "exponential" else 0)
    eye = torch.eye(width, dtype=torch.float64)
    qk, vw = heads * d, heads * dv
    w = {"m.q": eye[:qk], "m.k": eye[qk:2 * qk], "m.v": eye[2 * qk:2 * qk + vw], "m.g": eye[2 * qk + vw:2 * qk + 2 * vw],
         "m.o": torch.eye(vw, dtype=torch.float64)}
    if kind == "exponential":
        w["m.i"], w["m.f"] = eye[2 * qk + 2 * vw:2 * qk + 2 * vw + heads], eye[2 * qk + 2 * vw + heads:]
        w["m.i.b"], w["m.f.b"] = torch.randn(heads, generator=g).double(), 1.0 + torch.randn(heads, generator=g).double()
        w["m.norm"] = 1.0 + 0.3 * torch.randn(vw, generator=g).double()
    return width, w


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind,heads,d,dv,cap", [
    ("exponential", 2, 16, 32, 8.0), ("exponential", 3, 10, 12, 1.5), ("exponential", 1, 130, 5, 40.0),
    ("exponential", 4, 64, 72, 15.0), ("decay", 3, 10, 12, None), ("decay", 2, 32, 16, None), ("decay", 1, 256, 40, None),
    ("decay", 5, 4, 130, None)])
def test_a_matrix_memory_whole_and_token_by_token(dtype, kind, heads, d, dv, cap):
    """The recurrence over a prompt, over the same prompt cut into pieces down to single tokens (through state rows
    that held other values before and lie beside rows that must not change), against the plain mixer."""
    g = torch.Generator().manual_seed(heads * d + dv)
    T, eps = 90, 1e-5
    width, w = _memory_weights(kind, heads, d, dv, g)
    row = torch.randn(T, width, generator=g)
    if kind == "exponential":
        row[:, -2 * heads:] *= 3.0                      # log gates of some units: the cap bends them, the maximum moves
        want = plain.matrix_memory(row.to(dtype).double(), w, "m.", {"heads": heads, "dim": d, "vdim": dv, "gate_cap": cap}, eps)
        decays = None
    else:
        decay = [0.5 + 0.5 * i / heads for i in range(heads)]
        want = plain.retention(row.to(dtype).double(), w, "m.", {"heads": heads, "dim": d, "vdim": dv, "decay": decay,
                                                                  "rot": {"dims": 0, "base": 1.0}}, eps)
        decays = torch.tensor(decay, dtype=torch.float32, device=DEV)
    row = row.to(dtype).to(DEV)
    qk_w, v_w = heads * d, heads * dv
    memory = heads * d * dv
    state_w = memory + (heads * d + heads if kind == "exponential" else 0)

    def run(pieces, slot_count=5):
        state = torch.randn(slot_count, state_w, generator=g).to(DEV)
        q_len, q_start, slots = _segments(pieces, g, slot_count)
        slot = int(slots[0])
        state[slot] = 0.0
        before = state.clone()
        out = torch.zeros(T, v_w, dtype=dtype, device=DEV)
        for start, length in zip(q_start.tolist(), q_len.tolist()):
            part = row[start:start + length].contiguous()
            seg = (torch.zeros(1, dtype=torch.int32, device=DEV), torch.tensor([length], dtype=torch.int32, device=DEV),
                   torch.tensor([slot], dtype=torch.int32, device=DEV))
            qk = torch.zeros(2, length, qk_w, dtype=torch.float32, device=DEV)
            positions = torch.arange(start, start + length, dtype=torch.int32, device=DEV)
            ops.memory_inputs(part, positions, None, qk, heads=heads, head_dim=d,
                              q_scale=d ** -0.5 if kind == "exponential" else 1.0, k_scale=1.0 if kind == "exponential" else d ** -0.5)
            steps = nq = None
            if kind == "exponential":
                steps = torch.zeros(3, length, heads, dtype=torch.float32, device=DEV)
                nq = torch.zeros(length, heads, dtype=torch.float32, device=DEV)
                ops.memory_gates(part[:, 2 * qk_w + 2 * v_w:], w["m.i.b"].float().to(DEV), w["m.f.b"].float().to(DEV), state,
                                 memory + qk_w, *seg, steps, heads=heads, cap=cap)
            y = torch.zeros(length, v_w, dtype=torch.float32, device=DEV)
            ops.memory_scan(qk, part[:, 2 * qk_w:2 * qk_w + v_w], steps, decays, state, *seg, y, heads=heads, head_dim=d,
                            value_dim=dv, nq=nq, n_offset=memory if kind == "exponential" else 0)
            ops.head_norm_gate(y, part[:, 2 * qk_w + v_w:2 * qk_w + 2 * v_w],
                               w["m.norm"].float().to(DEV) if kind == "exponential" else None, out[start:start + length],
                               heads=heads, eps=eps, activation="sigmoid" if kind == "exponential" else "silu", scale=1.0,
                               nq=nq, floor=steps[2] if kind == "exponential" else None, den_eps=1e-6 if kind == "exponential" else 0.0)
        others = [i for i in range(slot_count) if i != slot]
        assert torch.equal(state[others], before[others]), "a state row of another request changed"
        return out, state[slot].clone()

    whole, state_whole = run([T])
    close(whole, want, dtype, "whole")
    cut, state_cut = run([17, 1, 1, 30, 2, 16, 1, 22])
    close(cut, want, dtype, "cut")
    # the recurrence adds in the same order however the prompt is cut
    assert (state_cut - state_whole).abs().max().item() <= 1e-5 * max(1.0, state_whole.abs().max().item())


@pytest.mark.parametrize("dtype", DTYPES)
def test_segments_of_a_batch_keep_their_own_memories(dtype):
    """Three requests of unequal length in one launch, slots in any order, against each alone."""
    g = torch.Generator().manual_seed(8)
    heads, d, dv = 2, 24, 20
    lengths = [1, 40, 7]
    n = sum(lengths)
    row = torch.randn(n, 2 * heads * d + heads * dv + 2 * heads, generator=g).to(dtype).to(DEV)
    q_len, q_start, slots = _segments(lengths, g, 6)
    state = torch.zeros(6, heads * d * dv + heads * d + heads, device=DEV)
    positions = torch.cat([torch.arange(x) for x in lengths]).to(torch.int32).to(DEV)
    qk_w = heads * d

    def run(rows, pos, seg, st):
        qk = torch.zeros(2, rows.shape[0], qk_w, dtype=torch.float32, device=DEV)
        ops.memory_inputs(rows, pos, None, qk, heads=heads, head_dim=d)
        steps = torch.zeros(3, rows.shape[0], heads, dtype=torch.float32, device=DEV)
        nq = torch.zeros(rows.shape[0], heads, dtype=torch.float32, device=DEV)
        ops.memory_gates(rows[:, 2 * qk_w + heads * dv:], None, None, st, heads * d * dv + qk_w, *seg, steps, heads=heads, cap=None)
        y = torch.zeros(rows.shape[0], heads * dv, dtype=torch.float32, device=DEV)
        ops.memory_scan(qk, rows[:, 2 * qk_w:2 * qk_w + heads * dv], steps, None, st, *seg, y, heads=heads, head_dim=d, value_dim=dv,
                        nq=nq, n_offset=heads * d * dv)
        return torch.cat([y, nq, steps[2]], dim=1)

    together = run(row, positions, (q_start.to(DEV), q_len.to(DEV), slots.to(DEV)), state)
    for s, (start, length) in enumerate(zip(q_start.tolist(), q_len.tolist())):
        alone_state = torch.zeros(1, state.shape[1], device=DEV)
        one = (torch.zeros(1, dtype=torch.int32, device=DEV), torch.tensor([length], dtype=torch.int32, device=DEV),
               torch.zeros(1, dtype=torch.int32, device=DEV))
        alone = run(row[start:start + length].contiguous(), positions[start:start + length].contiguous(), one, alone_state)
        assert torch.equal(together[start:start + length], alone), f"segment {s}"
        assert torch.equal(state[int(slots[s])], alone_state[0])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n,width,ff,count,top,groups,keep", [
    (1, 64, 48, 6, 2, 3, 2), (9, 128, 256, 5, 2, 1, 1), (7, 48, 24, 5, 3, 5, 5), (40, 96, 70, 8, 3, 4, 2), (300, 128, 96, 16, 4, 4, 2), (33, 36, 10, 1, 1, 1, 1),
    (90, 64, 32, 12, 1, 3, 1), (5, 256, 130, 4, 4, 2, 2), (130, 50, 16, 9, 6, 3, 2),
    (300, 128, 192, 4, 2, 2, 1), (700, 64, 64, 3, 1, 1, 1), (450, 192, 128, 6, 3, 3, 2)])     # bfloat16: tiles of 128 rows
def test_the_router_and_the_experts(dtype, n, width, ff, count, top, groups, keep):
    g = torch.Generator().manual_seed(n + width)
    h = torch.randn(n, width, generator=g).to(dtype)
    w = {"f.router": (torch.randn(count, width, generator=g) * 3.0 * width ** -0.5).to(torch.bfloat16).double()}
    for e in range(count):
        w[f"f.e{e}.gate"] = (torch.randn(ff, width, generator=g) * width ** -0.5).to(dtype).double()
        w[f"f.e{e}.up"] = (torch.randn(ff, width, generator=g) * width ** -0.5).to(dtype).double()
        w[f"f.e{e}.down"] = (torch.randn(width, ff, generator=g) * ff ** -0.5).to(dtype).double()
    c = {"expert": {"ff": ff}, "router": {"experts": count, "top": top, "groups": {"count": groups, "keep": keep}}}
    chosen, weights = plain.route(h.double(), w["f.router"], count, top, groups, keep)
    ids = torch.zeros(n, top, dtype=torch.int32, device=DEV)
    wts = torch.zeros(n, top, dtype=torch.float32, device=DEV)
    x = h.to(DEV)
    ops.moe_route(x, w["f.router"].float().to(DEV), ids, wts, groups=groups, keep=keep, eps=1e-20)
    # (scores that nearly tie may be chosen either way: such rows are left out of the comparison of the choice)
    s = torch.softmax(h.double() @ w["f.router"].T, dim=-1)
    top_scores = s.gather(1, chosen).sort(dim=-1, descending=True).values
    clear = torch.ones(n, dtype=torch.bool)
    rest = s.clone().scatter_(1, chosen, -1.0)
    clear &= (top_scores[:, -1] - rest.max(-1).values).abs() > 1e-4
    got_ids = ids.cpu().long()
    assert clear.float().mean() > 0.5
    for r in range(n):
        if clear[r]:
            assert sorted(got_ids[r].tolist()) == sorted(chosen[r].tolist()), f"row {r}"
            order = {e: i for i, e in enumerate(got_ids[r].tolist())}
            for e, a in zip(chosen[r].tolist(), weights[r].tolist()):
                assert abs(float(wts[r, order[e]]) - a) <= 1e-5 + 1e-4 * a
    tile = ops.moe_tile_rows(n * top, count, dtype, width, ff)
    assert (tile == 128) == (dtype == torch.bfloat16 and (n, ff) in ((300, 192), (700, 64), (450, 128)))
    assert tile in (16, 32, 64, 128)
    plan = torch.zeros(ops.moe_plan_size(n * top, count, tile), dtype=torch.int32, device=DEV)
    ops.moe_plan(ids, plan, count, tile)
    tiles = int(plan[0])
    rows = plan[1 + ops.moe_max_tiles(n * top, count, tile):][:tiles * tile].cpu()
    assert sorted(a for a in rows.tolist() if a >= 0) == list(range(n * top)), "every assignment has one row"
    flat_ids = ids.view(-1).cpu()
    for t in range(tiles):
        e = int(plan[1 + t])
        assert all(int(flat_ids[a]) == e for a in rows[tile * t:tile * t + tile].tolist() if a >= 0)
    stack = lambda names: torch.stack([torch.cat([w[f"f.e{e}.{x}"] for x in names]) for e in range(count)]).to(dtype).to(DEV)
    act = torch.zeros(n * top, ff, dtype=dtype, device=DEV)
    w_up, w_down = stack(("gate", "up")), stack(("down",))
    # the weights' tile-major copies, where the few-row kernels take them
    streamed = dtype == torch.bfloat16 and width % 32 == 0 and ff % 32 == 0
    t_up = ops.tile_weight(w_up.view(-1, width)) if streamed else None
    t_down = ops.tile_weight(w_down.view(-1, ff)) if streamed else None
    ops.moe_experts_up(x, w_up, plan, act, top, "silu", tile, t_up)
    out = torch.full((top, n, width), float("nan"), dtype=torch.float32, device=DEV)
    ops.moe_experts_down(act, w_down, plan, wts, out, tile, t_down)
    rounding = plain.to_bfloat16 if dtype == torch.bfloat16 else plain.same
    want = plain.mixture_of_experts(h.double(), w, "f.", c, rounding)
    got = out.sum(0)
    for r in range(n):
        if clear[r]:
            close(got[r], want[r], dtype, f"row {r}", scale=2.0)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_row_of_the_experts_does_not_depend_on_the_batch(dtype):
    g = torch.Generator().manual_seed(4)
    n, width, ff, count, top = 50, 64, 40, 6, 2
    x = torch.randn(n, width, generator=g).to(dtype).to(DEV)
    router = torch.randn(count, width, generator=g).to(DEV)
    w_up = (torch.randn(count, 2 * ff, width, generator=g) * 0.1).to(dtype).to(DEV)
    w_down = (torch.randn(count, width, ff, generator=g) * 0.1).to(dtype).to(DEV)

    def run(rows):
        m = rows.shape[0]
        ids, wts = torch.zeros(m, top, dtype=torch.int32, device=DEV), torch.zeros(m, top, dtype=torch.float32, device=DEV)
        ops.moe_route(rows, router, ids, wts, groups=3, keep=2)
        tile = ops.moe_tile_rows(m * top, count, torch.float32, width, ff)      # (as for float32: the streaming kernels)
        plan = torch.zeros(ops.moe_plan_size(m * top, count, tile), dtype=torch.int32, device=DEV)
        ops.moe_plan(ids, plan, count, tile)
        act = torch.zeros(m * top, ff, dtype=dtype, device=DEV)
        ops.moe_experts_up(rows, w_up, plan, act, top, "silu", tile)
        out = torch.zeros(top, m, width, dtype=torch.float32, device=DEV)
        ops.moe_experts_down(act, w_down, plan, wts, out, tile)
        return out
    together = run(x)
    for r in (0, 17, 49):
        assert torch.equal(run(x[r:r + 1].contiguous())[:, 0], together[:, r]), f"row {r}"


def _attention_problem(dtype, nh, nkv, d, ps, segs, seed):
    g = torch.Generator().manual_seed(seed)
    n = sum(q for q, _ in segs)
    pages = sum(-(-c // ps) for _, c in segs) + 3
    order = torch.randperm(pages, generator=g).tolist()
    bt = torch.zeros(len(segs), max(-(-c // ps) for _, c in segs), dtype=torch.int32)
    for s, (_, c) in enumerate(segs):
        for p in range(-(-c // ps)):
            bt[s, p] = order.pop()
    cache = torch.randn(pages, 2, nkv, ps * d, generator=g).to(dtype)
    rows = torch.randn(n, nh * d, generator=g).to(dtype)
    q_len = torch.tensor([q for q, _ in segs], dtype=torch.int32)
    ctx = torch.tensor([c for _, c in segs], dtype=torch.int32)
    q_start = (torch.cumsum(q_len, 0) - q_len).to(torch.int32)
    tok_seg = torch.repeat_interleave(torch.arange(len(segs), dtype=torch.int32), q_len.long())
    return rows, cache, bt, tok_seg, q_start, q_len, ctx


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,d,ps,chunk,segs", [
    (4, 2, 32, 16, 24, [(1, 100), (70, 70), (1, 24), (1, 25), (1, 49), (5, 200)]),
    (6, 2, 96, 16, 40, [(1, 41), (1, 40), (130, 300)]),
    (2, 1, 64, 8, 120, [(1, 300), (1, 241), (1, 240), (65, 65), (200, 400)]),
    (3, 3, 20, 8, 7, [(1, 50), (33, 40), (1, 7), (1, 8), (1, 15)]),
    (8, 1, 256, 16, 1000, [(1, 700), (300, 300), (64, 1000)]),
])
def test_a_one_in_the_denominator_inside_chunks_in_every_attention_kernel(dtype, nh, nkv, d, ps, chunk, segs):
    """The sink of score 0 with keys just inside and just outside a chunk's edge, decoded alone and inside prompts.
    Every second head's keys all score far below 0: the one in the denominator takes nearly all the weight and the result
    is nearly zero.  In the other heads scores are so sharp that one key decides, and the sink takes little."""
    rows, cache, bt, tok_seg, q_start, q_len, ctx = _attention_problem(dtype, nh, nkv, d, ps, segs, seed=d + chunk)
    rows *= 2.0
    scale = 2.0 / math.sqrt(d)
    # every key's first element is 3, and the first element of every second head's queries lowers all its scores by 25
    cache[:, 0].view(-1, nkv, ps, d)[..., 0] = 3.0
    rows.view(-1, nh, d)[:, 1::2, 0] = -25.0 / (3.0 * scale)
    out = torch.zeros(rows.shape[0], nh * d, dtype=dtype, device=DEV)
    args = [t.to(DEV) for t in (rows, cache, bt, tok_seg, q_start, q_len, ctx)] + [out]
    plan = ops.plan_paged_attention(q_len.numpy(), ctx.numpy(), num_heads=nh, num_kv_heads=nkv, head_dim=d, page_size=ps,
                                    window=-chunk, dtype=dtype, device=torch.device(DEV))
    ops.paged_attention(*args, num_heads=nh, num_kv_heads=nkv, head_dim=d, page_size=ps, scale=scale, chunk=chunk,
                        max_q_len=int(q_len.max()), max_ctx_len=int(ctx.max()), exact_weights=True, plan=plan,
                        sinks=torch.zeros(nh, dtype=torch.float32, device=DEV))
    torch.cuda.synchronize()
    kview = cache[:, 0].view(-1, nkv, ps, d).double()
    vview = cache[:, 1].view(-1, nkv, d, ps).double()
    weight_of_the_sink = []
    for s, (ql, cl) in enumerate(segs):
        ids = bt[s, :-(-cl // ps)].long()
        keys = kview[ids].permute(0, 2, 1, 3).reshape(-1, nkv, d)[:cl].repeat_interleave(nh // nkv, dim=1)
        values = vview[ids].permute(0, 3, 1, 2).reshape(-1, nkv, d)[:cl].repeat_interleave(nh // nkv, dim=1)
        q = torch.zeros(cl, nh, d, dtype=torch.float64)
        q[cl - ql:] = rows[int(q_start[s]):int(q_start[s]) + ql].double().view(ql, nh, d)
        scores = torch.einsum("ihd,jhd->hij", q, keys) * scale
        weights = plain.softmax_plus_one(scores, plain.chunk_mask(cl, chunk))
        weight_of_the_sink.append(1.0 - weights.sum(-1)[:, cl - ql:])
        want = torch.einsum("hij,jhd->ihd", weights, values)[cl - ql:].reshape(ql, nh * d)
        close(out[int(q_start[s]):int(q_start[s]) + ql], want, dtype, f"segment {s} ({ql} of {cl})")
    share = torch.cat([x.reshape(-1) for x in weight_of_the_sink])
    assert (share > 0.9).float().mean() > 0.3 and (share < 0.01).float().mean() > 0.1, "the sink counts in some rows, not in all"


# ---- the engine -----------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("family", list(FAMILIES))
@pytest.mark.parametrize("name", list(CONFIGS))
def test_replay_matches_plain(folders, name, family, dtype):
    requests = requests_for(name, LENGTHS[name])
    exact = plain_logits(folders[name], requests, torch.float64)
    trace = FAMILIES[family](requests)
    page_size = CONFIGS[name]["page_size"]
    model = load_model(folders[name], dtype, DEV)
    pages = pages_for_max_tokens(max_live_tokens(trace), page_size)
    runner = ModelRunner.create(model, num_pages=pages, page_size=page_size, max_requests=4, poison_freed_pages=True)
    with torch.inference_mode():
        got = replay_and_collect(TraceReplayer(runner), trace)
    runner.cache.check()
    assert not runner.cache.requests
    check_rows(got, folders[name], requests, exact, dtype, sharp=name == "sharp")


@pytest.mark.parametrize("seed", range(10))
def test_configurations_drawn_at_random(tmp_path, seed):
    c = random_config(200 + seed)
    folder = write_folder(c, str(tmp_path / "m"))
    requests = requests_for(c, [37, 18, 150, 64])
    exact = plain_logits(folder, requests, torch.float64)
    for dtype in DTYPES:
        for family in ("portions", "mixed"):
            trace = FAMILIES[family](requests)
            model = load_model(folder, dtype, DEV)
            pages = pages_for_max_tokens(max_live_tokens(trace), c["page_size"])
            runner = ModelRunner.create(model, num_pages=pages, page_size=c["page_size"], max_requests=4, poison_freed_pages=True)
            with torch.inference_mode():
                got = replay_and_collect(TraceReplayer(runner), trace)
            runner.cache.check()
            check_rows(got, folder, requests, exact, dtype)


@pytest.mark.parametrize("seed", range(3))
def test_long_requests_at_middling_sizes(tmp_path, seed):
    """Widths of some hundred and requests of up to 700 tokens, whole (the library's products, the tiled
    kernels, blocks of 64 rows in the attention, hundreds of rows an expert, memories carried over hundreds of
    tokens with decays close to one) and four at a time."""
    c = middling_config(300 + seed)
    folder = write_folder(c, str(tmp_path / "m"))
    requests = requests_for(c, [700, 129, 300, 65])
    exact = plain_logits(folder, requests, torch.float64)
    for dtype in DTYPES:
        for family in ("whole", "mixed"):
            trace = FAMILIES[family](requests) if family == "whole" else trace_mixed(requests, seed=seed, portion_sizes=(2, 64, 100, 128, 29))
            for step in trace:      # every tenth row is enough of a long request
                for e in step["entries"]:
                    e["want"] = [w for w in e["want"] if w % 10 == 0 or len(e["tokens"]) == 1]
            model = load_model(folder, dtype, DEV)
            pages = pages_for_max_tokens(max_live_tokens(trace), 16)
            runner = ModelRunner.create(model, num_pages=pages, page_size=16, max_requests=4, poison_freed_pages=True)
            with torch.inference_mode():
                got = replay_and_collect(TraceReplayer(runner), trace)
            runner.cache.check()
            check_rows(got, folder, requests, exact, dtype, bound=LONG_BOUND)


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_through_chunks_in_a_small_pool(folders, dtype):
    """300 tokens of which 260 are decoded one by one, in a pool that only the chunks make fit; the memories'
    states are carried through every step."""
    requests = requests_for("sharp", [300])
    exact = plain_logits(folders["sharp"], requests, torch.float64)
    model = load_model(folders["sharp"], dtype, DEV)
    runner = ModelRunner.create(model, num_pages=4, page_size=16, max_requests=2, poison_freed_pages=True)
    with torch.inference_mode():
        got = replay_and_collect(TraceReplayer(runner), trace_tail(requests, tail=260))
    runner.cache.check()
    check_rows(got, folders["sharp"], requests, exact, dtype, sharp=True)


def test_a_row_does_not_depend_on_the_batch_or_the_cut(folders):
    name = "sharp"
    requests = requests_for(name, [90, 200])
    model = load_model(folders[name], "float32", DEV)

    def run(trace):
        runner = ModelRunner.create(model, num_pages=40, page_size=16, max_requests=4)
        with torch.inference_mode():
            return replay_and_collect(TraceReplayer(runner), trace)

    one = {"q0": requests["q0"]}
    whole, cut, tail = run(trace_whole(one)), run(trace_portions(one)), run(trace_tail(one, tail=40))
    toks = requests["q0"]
    beside = [{"step": 0, "entries": [{"id": "q0", "tokens": toks[:50], "want": list(range(50))}], "end": []},
              {"step": 1, "entries": [{"id": "q1", "tokens": requests["q1"][:137], "want": []},
                                      {"id": "q0", "tokens": [toks[50]], "want": [0]}], "end": []},
              {"step": 2, "entries": [{"id": "q0", "tokens": toks[51:], "want": list(range(39))},
                                      {"id": "q1", "tokens": requests["q1"][137:], "want": []}], "end": ["q0", "q1"]}]
    mixed = run(beside)
    for key, ref in whole.items():
        for other in (cut, tail, mixed):
            assert (other[key] - ref).abs().max().item() <= 2e-4 * max(1.0, ref.abs().max().item()), key


@pytest.mark.parametrize("graphs", [False, True])
def test_greedy_generation_through_the_entry_point(folders, graphs):
    """`LLM.generate` (scheduler, chunked prefill, sampling kernels, captured graphs or not) against greedy decoding
    with the plain implementation, in float32 so that the tokens are comparable one by one."""
    name = "duo"
    prompts = list(requests_for(name, [37, 5, 64, 18, 1]).values())
    new = 24
    llm = LLM(folders[name], dtype="float32", num_blocks=64, block_size=16, max_prefill_tokens_per_step=32, max_requests=4,
              hip_graphs=graphs)
    outs = llm.generate(prompts, max_new_tokens=new)
    raw, w = read_folder(folders[name])
    for prompt, out in zip(prompts, outs):
        tokens = list(prompt)
        for step in range(new):
            logits = plain.forward(raw, w, tokens)[-1]
            top2 = logits.topk(2).values
            if (top2[0] - top2[1]).item() < 1e-3:       # a tie within rounding: the rest is not comparable
                break
            assert out.token_ids[step] == int(logits.argmax()), f"prompt of {len(prompt)}: token {step} differs"
            tokens.append(out.token_ids[step])
        assert len(out.token_ids) == new
    if graphs:
        assert llm.runner.graph_steps > 0


def test_the_trace_runner_and_the_command_line(folders, tmp_path):
    name = "odd"
    toks = requests_for(name, [45])["q0"]
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": toks[:30], "want": [0, 29]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": toks[30:32], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": toks[32:], "want": [12]}], "end": ["a"]}]
    out = tmp_path / "out"
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folders[name], "--dtype", "float32",
                        "--out", str(out), "--max-tokens", "64"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [line for line in r.stdout.splitlines() if line.startswith("done")] == ["done 0", "done 1", "done 2"]
    exact = plain_logits(folders[name], {"a": toks}, torch.float64)
    first = torch.frombuffer(bytearray((out / "0.f32").read_bytes()), dtype=torch.float32).view(2, -1)
    last = torch.frombuffer(bytearray((out / "2.f32").read_bytes()), dtype=torch.float32).view(1, -1)
    assert not (out / "1.f32").exists()
    compare_rows({("a", 0): first[0], ("a", 29): first[1], ("a", 44): last[0]}, exact, relative=1e-4)
    # the command line: a model folder of a named shape, then greedy generation from it
    made = tmp_path / "made"
    r = subprocess.run([sys.executable, "-m", "wllm_amd.cli", "random-model", "--out", str(made), "--config", "lefisun-tiny",
                        "--seed", "3", "--std", "0.3", "--norm-std", "0.6"], cwd=ROOT, capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    r = subprocess.run([sys.executable, "-m", "wllm_amd.cli", "generate", "--model", str(made), "--dtype", "float32",
                        "--prompt-ids", "5,17,3,200,41", "--max-new-tokens", "6"], cwd=ROOT, capture_output=True, text=True,
                       timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    line = json.loads([x for x in r.stdout.splitlines() if x.startswith("{")][-1])
    raw, w = read_folder(str(made))
    tokens = [5, 17, 3, 200, 41]
    for t in line["token_ids"]:
        logits = plain.forward(raw, w, tokens)[-1]
        if (logits.topk(2).values[0] - logits.topk(2).values[1]).item() < 1e-3:
            break
        assert t == int(logits.argmax())
        tokens.append(t)
    assert len(line["token_ids"]) == 6
