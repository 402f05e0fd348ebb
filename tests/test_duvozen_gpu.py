"""Duvozen on the GPU: each new mechanism's kernel alone against the plain implementation's function of
that mechanism, then the engine (cache, state slots, carried rows, batches, portions, captured graphs, the entry
point) against the plain forward pass, in float32 and bfloat16."""
import copy
import json
import math
import os
import subprocess
import sys

import pytest
import torch

from duvozen_helpers import (CONFIGS, compare_rows, compare_with_rounding, middling_config, plain_logits, random_config, read_folder,
                             requests_for, rounding_noise, to_bfloat16, write_folder)
from helpers import max_live_tokens, replay_and_collect, trace_mixed, trace_portions, trace_tail, trace_whole
from plain import duvozen_plain as plain
from wllm_amd.engine import LLM, ModelRunner
from wllm_amd.engine.replay import TraceReplayer, pages_for_max_tokens
from wllm_amd.kernels import ops
from wllm_amd.parts import load_model

pytestmark = pytest.mark.gpu
DEV = "cuda"
DTYPES = [torch.float32, torch.bfloat16]
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LENGTHS = {"trio": [70, 45, 150, 33, 58], "odd": [40, 66, 25, 151], "sharp": [80, 137, 64, 50], "one_tap": [30, 9, 70]}
FAMILIES = {"whole": trace_whole, "tail": trace_tail, "portions": trace_portions, "mixed": trace_mixed}
# a row's distance from the exact row, as a share of the row's own size or as a multiple of what rounding alone does to
# that row in the plain implementation (`rounding_noise`), whichever is larger: float32 sums in another order; bfloat16
# activations through some ten roundings a layer, and now and then a router or a key that the engine's rounding makes
# win where the plain implementation's does not
BOUND = {torch.float32: dict(relative=1e-4, times=6.0), torch.bfloat16: dict(relative=0.04, outliers=0.1)}
LONG_BOUND = {torch.float32: dict(relative=1e-4, times=6.0), torch.bfloat16: dict(relative=0.04, outliers=0.25)}
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
    root = tmp_path_factory.mktemp("duvozen_gpu")
    return {name: write_folder(name, str(root / name)) for name in CONFIGS}


def _segments(lengths, generator, slots_total):
    q_len = torch.tensor(lengths, dtype=torch.int32)
    q_start = (torch.cumsum(q_len, 0) - q_len).to(torch.int32)
    slots = torch.randperm(slots_total, generator=generator)[:len(lengths)].to(torch.int32)
    return q_len, q_start, slots


def _pieces(total, sizes):
    out, at, i = [], 0, 0
    while at < total:
        n = min(sizes[i % len(sizes)], total - at)
        out.append((at, at + n))
        at, i = at + n, i + 1
    return out


# ---- mechanisms alone ---------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("channels,taps", [(48, 2), (64, 4), (300, 3), (33, 1), (2048, 7)])
def test_the_convolution_of_the_stream_whole_and_in_pieces(dtype, channels, taps):
    """Three requests side by side, whole and cut into pieces down to single tokens, through carried rows that lie
    beside rows of other requests (which must not change) and held other values before they were zeroed."""
    g = torch.Generator().manual_seed(channels + taps)
    lengths = [37, 5, 90]
    xs = [torch.randn(n, channels, generator=g) for n in lengths]
    w = torch.randn(channels, taps, generator=g) * 0.5
    want = [plain.input_convolution(x.double(), w.double()) for x in xs]
    # (rows and offsets in multiples of 16 bytes take the kernel that moves four channels a thread)
    offset, extra, slots_total = (8, 4, 6) if channels % 8 == 0 else (5, 3, 6)
    row = offset + (taps - 1) * channels + extra
    for sizes in ([1000], [16, 5, 2, 1, 1, 7], [1]):
        state = torch.full((slots_total, row), 7.0, device=DEV)
        q_len, q_start, slots = _segments(lengths, g, slots_total)
        state[slots.long()] = 0.0
        state[:, :offset] = 3.0
        done = [0, 0, 0]
        outs = [[], [], []]
        while any(d < n for d, n in zip(done, lengths)):
            live = [i for i in range(3) if done[i] < lengths[i]]
            take = [min(sizes[(done[i] + i) % len(sizes)], lengths[i] - done[i]) for i in live]
            x = torch.cat([xs[i][done[i]:done[i] + t] for i, t in zip(live, take)]).to(DEV)
            ql = torch.tensor(take, dtype=torch.int32)
            qs = (torch.cumsum(ql, 0) - ql).to(torch.int32)
            seg = torch.repeat_interleave(torch.arange(len(live), dtype=torch.int32), ql.long())
            out = torch.zeros(x.shape[0], channels, dtype=dtype, device=DEV)
            # (a step of single tokens moves the carried rows in the launch that reads them)
            ops.stream_conv(x, w.t().contiguous().to(DEV), state, offset, seg.to(DEV), qs.to(DEV), ql.to(DEV), slots[live].to(DEV), out,
                            single_tokens=all(t == 1 for t in take))
            for j, (i, t) in enumerate(zip(live, take)):
                outs[i].append(out[int(qs[j]):int(qs[j]) + t].cpu())
                done[i] += t
        for i in range(3):
            close(torch.cat(outs[i]), want[i], dtype, f"request {i}, pieces {sizes}", scale=3.0)
        others = [s for s in range(slots_total) if s not in slots.tolist()]
        assert (state[others][:, offset:] == 7.0).all() and (state[:, :offset] == 3.0).all() and (state[:, row - extra:][others] == 7.0).all()
        if taps > 1:
            for i in range(3):
                carried = state[int(slots[i]), offset:offset + (taps - 1) * channels].view(taps - 1, channels).cpu()
                tail = torch.cat([torch.zeros(taps - 1, channels), xs[i]])[-(taps - 1):]
                assert torch.equal(carried, tail)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden,taps,stack", [(64, 4, 0), (300, 2, 3), (2048, 3, 0), (48, 1, 2), (600, 9, 0), (4096, 8, 2)])
def test_settling_the_stream_and_the_convolution_in_one_launch(dtype, hidden, taps, stack):
    """For a step of single tokens `norm_add` with `conv` gives the bits of `norm_add` and then `stream_conv`, in the
    stream, in the sublayer's input and in the carried rows."""
    g = torch.Generator().manual_seed(hidden + taps)
    n, slots_total, offset = 7, 9, 4
    x = torch.randn(n, hidden, generator=g)
    delta = torch.randn(stack, n, hidden, generator=g) if stack else torch.randn(n, hidden, generator=g).to(dtype)
    norm_w = (1.0 + 0.3 * torch.randn(hidden, generator=g)).to(DEV)
    w = (torch.randn(taps, hidden, generator=g) * 0.5).to(DEV)
    state0 = torch.randn(slots_total, offset + (taps - 1) * hidden + 2, generator=g)
    slots = torch.randperm(slots_total, generator=g)[:n].to(torch.int32).to(DEV)
    recipe = ops.NormRecipe("layer", norm_w, 1e-5, 0.0)
    seg = torch.arange(n, dtype=torch.int32, device=DEV)
    ones = torch.ones(n, dtype=torch.int32, device=DEV)
    xa, sa = x.clone().to(DEV), state0.clone().to(DEV)
    out_a = torch.zeros(n, hidden, dtype=dtype, device=DEV)
    ops.norm_add(xa, delta=delta.to(DEV), delta_norm=recipe)
    ops.stream_conv(xa, w, sa, offset, seg, seg, ones, slots, out_a, single_tokens=True)
    xb, sb = x.clone().to(DEV), state0.clone().to(DEV)
    out_b = torch.zeros(n, hidden, dtype=dtype, device=DEV)
    ops.norm_add(xb, delta=delta.to(DEV), delta_norm=recipe, out=out_b, conv=(w, sb, offset, slots))
    assert torch.equal(xa, xb) and torch.equal(out_a, out_b) and torch.equal(sa, sb)
    d = (delta.sum(0) if stack else delta).double()
    settled = x.double() + plain.layer_norm(d, norm_w.cpu().double(), 1e-5)
    close(xb, settled, torch.float32, "the stream", scale=4.0)
    for r in range(n):
        carried = state0[int(slots[r]), offset:offset + (taps - 1) * hidden].view(taps - 1, hidden).double()
        seq = torch.cat([carried, settled[r:r + 1]])
        close(out_b[r], settled[r] + (seq * w.cpu().double()).sum(0), dtype, f"row {r}", scale=4.0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,d,dv", [(2, 16, 32), (3, 10, 12), (1, 130, 5), (4, 64, 72), (1, 256, 40), (5, 4, 130)])
def test_a_forget_gate_recurrence_whole_and_token_by_token(dtype, heads, d, dv):
    """The recurrence over a prompt, over the same prompt cut into pieces down to single tokens (through state rows
    that held other values before and lie beside rows that must not change), against the plain mixer."""
    g = torch.Generator().manual_seed(heads * d + dv)
    T, eps = 90, 1e-5
    qw, vw = heads * d, heads * dv
    width = 2 * qw + vw + 3
    eye = torch.eye(width, dtype=torch.float64)
    w = {"m.q": eye[:qw], "m.f": eye[qw:2 * qw], "m.v": eye[2 * qw:2 * qw + vw], "m.o": torch.eye(vw, dtype=torch.float64),
         "m.f.b": torch.randn(qw, generator=g).double(), "m.lower": (torch.rand(qw, generator=g) * 0.95).double(),
         "m.norm": 1.0 + 0.3 * torch.randn(dv, generator=g).double()}
    row = torch.randn(T, width, generator=g)
    row[:, qw:2 * qw] *= 3.0                       # gates from nearly closed to nearly open
    want = plain.forget_gate_recurrence(row.to(dtype).double(), w, "m.", {"heads": heads, "dim": d, "vdim": dv}, eps)
    norm_w = w["m.norm"].float().repeat(heads).to(DEV)
    slots_total, memory = 5, heads * d * dv
    for sizes in ([1000], [16, 5, 2, 1, 33], [1]):
        state = torch.full((slots_total, memory + 4), 9.0, device=DEV)
        state[2] = 0.0
        outs = []
        for lo, hi in _pieces(T, sizes):
            n = hi - lo
            dev_row = row[lo:hi].to(dtype).to(DEV)
            qkf = torch.zeros(3, n, qw, dtype=torch.float32, device=DEV)
            ops.memory_forget_inputs(dev_row, w["m.f.b"].float().to(DEV), w["m.lower"].float().to(DEV), qkf, width=qw, q_activation="silu")
            y = torch.zeros(n, vw, dtype=torch.float32, device=DEV)
            one = lambda v: torch.tensor([v], dtype=torch.int32, device=DEV)
            ops.memory_scan(qkf, dev_row[:, 2 * qw:2 * qw + vw], None, None, state, one(0), one(n), one(2), y, heads=heads,
                            head_dim=d, value_dim=dv, row_decays=True)
            out = torch.zeros(n, vw, dtype=dtype, device=DEV)
            ops.head_norm_gate(y, None, norm_w, out, heads=heads, eps=eps, activation="none")
            outs.append(out.cpu())
        close(torch.cat(outs), want, dtype, f"pieces {sizes}", scale=2.0)
        assert (state[[0, 1, 3, 4]] == 9.0).all()
    # f + (1 - f) is one to rounding, and the decay is the f the gate gives, not one minus what is written
    f = w["m.lower"] + (1 - w["m.lower"]) * torch.sigmoid(row[:8, qw:2 * qw].to(dtype).double() + w["m.f.b"])
    qkf = torch.zeros(3, 8, qw, dtype=torch.float32, device=DEV)
    ops.memory_forget_inputs(row[:8].to(dtype).to(DEV), w["m.f.b"].float().to(DEV), w["m.lower"].float().to(DEV), qkf, width=qw,
                             q_activation="none")
    close(qkf[2], f, torch.float32, "the decay")
    close(qkf[1], 1 - f, torch.float32, "what is written")
    close(qkf[0], row[:8, :qw].to(dtype).double(), torch.float32, "queries as they are")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,d,dims,pairing,scaling,weighted", [
    (4, 2, 32, 16, "half", None, True), (3, 3, 20, 6, "half", None, True), (2, 1, 96, 96, "half", None, True),
    (4, 1, 96, 16, "interleaved", (8.0, 64, 16.0, 1.0), False), (3, 1, 44, 6, "interleaved", (4.0, 16, 4.0, 0.5), False),
    (1, 1, 12, 12, "interleaved", None, True), (5, 1, 64, 0, "half", None, True)])
def test_a_norm_over_each_head_then_a_turn_with_interpolated_frequencies(dtype, nh, nkv, d, dims, pairing, scaling, weighted):
    """`head_prepare` with a weighted RMS norm over every head in front of the rotation, frequencies from the position
    part (interpolated or not), sine and cosine scaled; keys stored where their slots say."""
    from wllm_amd.parts.positions import RotaryPosition
    from wllm_amd.parts.specs import PositionSpec
    g = torch.Generator().manual_seed(d + dims)
    n, ps, eps, base = 45, 8, 1e-5, 500.0
    rows = torch.randn(n, (nh + 2 * nkv) * d + 8, generator=g).to(dtype)
    positions = torch.randint(0, 3000, (n,), generator=g).to(torch.int32)
    wq, wk = 1.0 + 0.3 * torch.randn(d, generator=g), 1.0 + 0.3 * torch.randn(d, generator=g)
    inv_freq, magnitude = None, 1.0
    if dims:
        magnitude = 0.1 * math.log(scaling[0]) + 1.0 if scaling else 1.0
        part = RotaryPosition(PositionSpec(rotary_dim=dims, theta=base, pairing=pairing, ramp=scaling, magnitude=magnitude))
        part.prepare(DEV)
        inv_freq = part.inv_freq
        want_freq = (plain.interpolated_frequencies(dims, base, dict(zip(("factor", "original", "fast", "slow"), scaling)))[0]
                     if scaling else plain.plain_frequencies(dims, base))
        assert torch.allclose(inv_freq.cpu().double(), want_freq, rtol=1e-6)
    pages = 9
    slots = torch.randperm(pages * ps, generator=g)[:n].to(torch.int32)
    cache = torch.zeros(pages, 2, nkv, ps * d, dtype=dtype, device=DEV)
    dev = rows.to(DEV)
    ops.head_prepare(dev, None, positions.to(DEV), inv_freq, slots.to(DEV), cache, num_heads=nh, num_kv_heads=nkv, head_dim=d,
                     page_size=ps, interleaved=pairing == "interleaved", rot_scale=magnitude,
                     head_norm=(wq.to(DEV), wk.to(DEV), eps) if weighted else None)
    x = rows.double()
    q = x[:, :nh * d].view(n, nh, d)
    k = x[:, nh * d:(nh + nkv) * d].view(n, nkv, d)
    if weighted:
        q, k = plain.rms_norm(q, wq.double(), eps), plain.rms_norm(k, wk.double(), eps)
    if dims:
        q, k = (plain.rotate(t, positions, dims, inv_freq.cpu().double(), pairing, magnitude) for t in (q, k))
    # (the angle is a float32 product of a position of some thousands: 1e-4 of a radian)
    close(dev[:, :nh * d], q.reshape(n, -1), dtype, "queries", scale=20.0 if dtype == torch.float32 else 4.0)
    close(dev[:, nh * d:(nh + nkv) * d], k.reshape(n, -1), dtype, "keys", scale=20.0 if dtype == torch.float32 else 4.0)
    assert torch.equal(dev[:, (nh + nkv) * d:].cpu(), rows[:, (nh + nkv) * d:])
    stored = cache[:, 0].view(pages, nkv, ps, d)[(slots // ps).long(), :, (slots % ps).long()]
    assert torch.equal(stored.cpu(), dev[:, nh * d:(nh + nkv) * d].view(n, nkv, d).cpu())
    values = cache[:, 1].view(pages, nkv, d, ps)[(slots // ps).long(), :, :, (slots % ps).long()]
    assert torch.equal(values.cpu(), rows[:, (nh + nkv) * d:(nh + 2 * nkv) * d].view(n, nkv, d))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n,width,ff,count,top,shared", [(5, 64, 32, 4, 2, 48), (40, 48, 24, 5, 5, None), (300, 128, 192, 8, 2, 64),
                                                         (1, 32, 40, 3, 1, 8), (77, 96, 56, 1, 1, None), (450, 64, 128, 16, 3, 128)])
def test_experts_scored_by_sigmoids_weigh_their_input(dtype, n, width, ff, count, top, shared):
    """The router with sigmoid scores that are the weights as they are, the first product with the weight taken out of
    its sums, the second without weights, at sizes of both kernel families; against the plain feed-forward."""
    g = torch.Generator().manual_seed(n + ff)
    h = torch.randn(n, width, generator=g).to(dtype)
    w = {"f.router": (torch.randn(count, width, generator=g) * width ** -0.5).float().double()}
    names = [f"e{e}." for e in range(count)] + (["shared."] if shared else [])
    for e in names:
        size = shared if e == "shared." else ff
        w["f." + e + "gate"] = (torch.randn(size, width, generator=g) * width ** -0.5).to(dtype).double()
        w["f." + e + "up"] = (torch.randn(size, width, generator=g) * width ** -0.5).to(dtype).double()
        w["f." + e + "down"] = (torch.randn(width, size, generator=g) * size ** -0.5).to(dtype).double()
    c = {"router": {"experts": count, "top": top}, "shared": {"ff": shared} if shared else None}
    x = h.to(DEV)
    ids = torch.zeros(n, top, dtype=torch.int32, device=DEV)
    wts = torch.zeros(n, top, dtype=torch.float32, device=DEV)
    ops.moe_route(x, w["f.router"].float().to(DEV), ids, wts, scoring="sigmoid", normalize=False)
    s = torch.sigmoid(h.double() @ w["f.router"].T)
    best = s.topk(top, dim=-1)
    rest = s.clone().scatter_(1, best.indices, -1.0)
    clear = (best.values[:, -1] - rest.max(-1).values).abs() > 1e-4 if top < count else torch.ones(n, dtype=torch.bool)
    assert clear.float().mean() > 0.5
    for r in range(n):
        if clear[r]:
            assert sorted(ids[r].tolist()) == sorted(best.indices[r].tolist()), f"row {r}"
            for e, a in zip(ids[r].tolist(), wts[r].tolist()):
                assert abs(a - float(s[r, e])) <= 1e-5, "the weight is the score itself"
    tile = ops.moe_tile_rows(n * top, count, dtype, width, ff)
    plan = torch.zeros(ops.moe_plan_size(n * top, count, tile), dtype=torch.int32, device=DEV)
    ops.moe_plan(ids, plan, count, tile)
    stack = lambda parts: torch.stack([torch.cat([w[f"f.e{e}.{x}"] for x in parts]) for e in range(count)]).to(dtype).to(DEV)
    w_up, w_down = stack(("gate", "up")), stack(("down",))
    streamed = dtype == torch.bfloat16 and width % 32 == 0 and ff % 32 == 0
    t_up = ops.tile_weight(w_up.view(-1, width)) if streamed else None
    t_down = ops.tile_weight(w_down.view(-1, ff)) if streamed else None
    act = torch.zeros(n * top, ff, dtype=dtype, device=DEV)
    ops.moe_experts_up(x, w_up, plan, act, top, "silu", tile, t_up, in_weights=wts)
    out = torch.full((top, n, width), float("nan"), dtype=torch.float32, device=DEV)
    ops.moe_experts_down(act, w_down, plan, wts, out, tile, t_down, weighted=False)
    rounding = to_bfloat16 if dtype == torch.bfloat16 else plain.same
    cc = dict(c)
    cc["shared"] = None
    want = plain.expert_feed_forward(h.double(), {k: v for k, v in w.items() if "shared" not in k}, "f.", cc, rounding)
    got = out.sum(0)
    for r in range(n):
        if clear[r]:
            close(got[r], want[r], dtype, f"row {r}", scale=2.0)


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
@pytest.mark.parametrize("nh,nkv,d,ps,segs", [
    (4, 2, 32, 16, [(1, 700), (70, 70), (1, 17), (1, 16), (5, 200)]),
    (6, 2, 96, 16, [(1, 641), (130, 300), (1, 1)]),
    (3, 3, 20, 8, [(1, 350), (33, 40), (1, 8), (1, 9)]),
    (8, 1, 256, 16, [(1, 900), (300, 300), (64, 1000)]),
    (5, 1, 96, 16, [(1, 129), (1, 128), (200, 520)]),
])
def test_a_learned_sink_and_a_key_far_away_in_every_attention_kernel(dtype, nh, nkv, d, ps, segs):
    """A number a head in the denominator, large in some heads (their result is nearly zero) and small in others; and in
    every segment one key far back, at a page's first or last slot, that the last query's first head scores far above all
    others: its value is the result.  Decoded tokens and prompts, all kernel families."""
    rows, cache, bt, tok_seg, q_start, q_len, ctx = _attention_problem(dtype, nh, nkv, d, ps, segs, seed=d + ps)
    scale = 1.0 / math.sqrt(d)
    kview = cache[:, 0].view(-1, nkv, ps, d)
    vview = cache[:, 1].view(-1, nkv, d, ps)
    far = []
    for s, (ql, cl) in enumerate(segs):
        j = 0 if cl < 40 else (ps - 1 if s % 2 else ps)             # a page's last slot, or the next page's first
        j = min(j, cl - 1)
        last = int(q_start[s]) + ql - 1
        q0 = rows[last, :d].float()
        kview[int(bt[s, j // ps]), 0, j % ps] = (q0 / q0.norm() * (40.0 / scale) / q0.norm()).to(dtype)     # a score of 40
        far.append((last, j))
    sinks = torch.tensor([(-6.0, 2.0, 12.0)[h % 3] for h in range(nh)])
    out = torch.zeros(rows.shape[0], nh * d, dtype=dtype, device=DEV)
    args = [t.to(DEV) for t in (rows, cache, bt, tok_seg, q_start, q_len, ctx)] + [out]
    plan = ops.plan_paged_attention(q_len.numpy(), ctx.numpy(), num_heads=nh, num_kv_heads=nkv, head_dim=d, page_size=ps,
                                    window=0, dtype=dtype, device=torch.device(DEV))
    ops.paged_attention(*args, num_heads=nh, num_kv_heads=nkv, head_dim=d, page_size=ps, scale=scale,
                        max_q_len=int(q_len.max()), max_ctx_len=int(ctx.max()), exact_weights=True, plan=plan, sinks=sinks.to(DEV))
    torch.cuda.synchronize()
    for s, (ql, cl) in enumerate(segs):
        ids = bt[s, :-(-cl // ps)].long()
        keys = kview.double()[ids].permute(0, 2, 1, 3).reshape(-1, nkv, d)[:cl].repeat_interleave(nh // nkv, dim=1)
        values = vview.double()[ids].permute(0, 3, 1, 2).reshape(-1, nkv, d)[:cl].repeat_interleave(nh // nkv, dim=1)
        q = torch.zeros(cl, nh, d, dtype=torch.float64)
        q[cl - ql:] = rows[int(q_start[s]):int(q_start[s]) + ql].double().view(ql, nh, d)
        weights = plain.causal_softmax(torch.einsum("ihd,jhd->hij", q, keys) * scale, sinks.double())
        want = torch.einsum("hij,jhd->ihd", weights, values)[cl - ql:].reshape(ql, nh * d)
        close(out[int(q_start[s]):int(q_start[s]) + ql], want, dtype, f"segment {s} ({ql} of {cl})")
        last, j = far[s]
        assert weights[0, cl - 1, j] > 0.99, "the far key decides"
        close(out[last, :d], values[j, 0], dtype, f"segment {s}: the far key's value", scale=2.0)
        if nh >= 3:
            assert weights[2, cl - 1].sum() < 0.05 and weights[0 if nh < 4 else 3, cl - 1].sum() > 0.5


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
    """Widths of some hundred and requests of up to 700 tokens, whole (the library's products, the tiled kernels,
    blocks of 64 rows in the attention, hundreds of rows an expert, recurrences carried over hundreds of tokens)
    and four at a time."""
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
def test_long_decoding_with_sharp_attention(folders, dtype):
    """400 tokens of which 300 are decoded one by one: single keys far back decide, sinks count, the recurrence's
    state and the carried rows go through every step."""
    requests = requests_for("sharp", [400])
    exact = plain_logits(folders["sharp"], requests, torch.float64)
    model = load_model(folders["sharp"], dtype, DEV)
    runner = ModelRunner.create(model, num_pages=26, page_size=16, max_requests=2, poison_freed_pages=True)
    with torch.inference_mode():
        got = replay_and_collect(TraceReplayer(runner), trace_tail(requests, tail=300))
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
    name = "trio"
    prompts = list(requests_for(name, [37, 5, 64, 18, 1]).values())
    new = 24
    llm = LLM(folders[name], dtype="float32", num_blocks=64, block_size=16, max_prefill_tokens_per_step=32, max_requests=4,
              hip_graphs=graphs)
    outs = llm.generate(prompts, max_new_tokens=new)
    raw, w = read_folder(folders[name])
    for prompt, out in zip(prompts, outs):
        tokens = list(prompt)
        for step in range(new):
            logits = plain.forward(tokens, w, raw)[-1]
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
    r = subprocess.run([sys.executable, "-m", "wllm_amd.cli", "random-model", "--out", str(made), "--config", "duvozen-tiny",
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
        logits = plain.forward(tokens, w, raw)[-1]
        if (logits.topk(2).values[0] - logits.topk(2).values[1]).item() < 1e-3:
            break
        assert t == int(logits.argmax())
        tokens.append(t)
    assert len(line["token_ids"]) == 6
