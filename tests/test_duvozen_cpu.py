"""Duvozen without a GPU: its configuration, its plan, the plain implementation's own mechanisms against a
second way of computing each, and the engine's bookkeeping around it (a cache or a state row a layer, the rows a
convolution carries for each sublayer, state slots that are zeroed and used again) against the plain
implementation, the kernels replaced by the emulation of their contracts."""
import copy
import math

import pytest
import torch

from duvozen_helpers import (CONFIGS, attention, compare_rows, config, dense, experts, latent, layer, plain_logits, random_config,
                             read_folder, recurrence, requests_for, write_folder)
from helpers import max_live_tokens, replay_and_collect, trace_mixed, trace_portions, trace_tail, trace_whole
from kernel_emulation import EmulatedKernels
from plain import duvozen_plain as plain
from wllm_amd.architectures import DuvozenConfig
from wllm_amd.config import ConfigError
from wllm_amd.engine import ModelRunner
from wllm_amd.engine.replay import TraceReplayer, pages_for_max_tokens
from wllm_amd.kernels import ops
from wllm_amd.parts import build_model, load_model

LENGTHS = {"trio": [70, 45, 90, 33, 58], "odd": [40, 66, 25, 51], "sharp": [80, 37, 64, 50], "one_tap": [30, 9, 21]}
FAMILIES = {"whole": trace_whole, "tail": trace_tail, "portions": trace_portions, "mixed": trace_mixed}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("duvozen")
    return {name: write_folder(name, str(root / name)) for name in CONFIGS}


@pytest.fixture(scope="module")
def exact(folders):
    return {name: plain_logits(folders[name], requests_for(name, LENGTHS[name]), torch.float64) for name in CONFIGS}


# ---- configuration and plan ------------------------------------------------------------------------
def test_the_plan_follows_the_file():
    model = build_model(copy.deepcopy(CONFIGS["trio"]["config"]))
    plan = model.plan
    assert [type(b.mixer).__name__ for b in plan.layers] == ["MatrixMemorySpec", "LatentAttentionSpec", "AttentionSpec",
                                                             "AttentionSpec", "LatentAttentionSpec", "MatrixMemorySpec"]
    assert all(b.arrangement == "post_norm" and b.mixer_norm is None and b.mixer_post_norm.kind == "layer" for b in plan.layers)
    assert all(b.mixer_input_conv.taps == 4 and b.mixer_input_conv.weight.endswith("canon1") for b in plan.layers)
    first, lat, att = plan.layers[0].mixer, plan.layers[1].mixer, plan.layers[2].mixer
    assert first.gating == "forget" and first.q_activation == "silu" and first.gate_weight is None and not first.k_weight
    assert first.lower_bound == "l0.mix.lower" and not first.norm_weight_per_head and first.norm_eps == 1e-5
    assert (lat.num_heads, lat.head_dim, lat.rope_dim, lat.value_dim, lat.kv_rank, lat.scale) == (4, 32, 16, 16, 80, 0.2)
    assert lat.q_weight == "l1.mix.q" and lat.q_rank == 0 and lat.sink_weight is None and lat.gate_weight is None
    assert lat.position.pairing == "interleaved" and lat.position.ramp == (4.0, 64.0, 8.0, 1.0) and lat.weights_in_float32
    assert lat.position.magnitude == pytest.approx(0.1 * math.log(4.0) + 1.0)
    assert plan.layers[4].mixer.position.ramp is None and plan.layers[4].mixer.position.magnitude == 1.0
    assert (att.num_heads, att.num_kv_heads, att.head_dim, att.value_dim, att.scale) == (4, 2, 32, 64, 0.3)
    assert att.position.pairing == "half" and att.position.rotary_dim == 16 and att.sink_weight == "l2.mix.sink"
    assert att.q_head_norm_weight == "l2.mix.q.norm" and att.head_norm_eps == 1e-5 and att.gate_weight == "l2.mix.g"
    moe = plan.layers[0].feed_forward
    assert (moe.num_experts, moe.top, moe.intermediate_size, moe.scoring, moe.normalize, moe.weight_on_input) == (4, 2, 32, "sigmoid", False, True)
    assert moe.shared.intermediate_size == 48 and moe.shared.activation == "silu" and plan.layers[2].feed_forward.shared is None
    assert plan.layers[1].feed_forward.activation == "gelu_tanh"
    assert plan.layers[4].feed_forward is None and plan.layers[4].feed_forward_input_conv is None
    assert plan.embedding.scale == 1.5 and plan.head.weight == "head" and plan.head.logit_scale == 0.7
    names = set(model.expected_tensors())
    assert {"embed", "head", "final.norm", "l0.mix.f.b", "l0.mix.lower", "l0.mlp.shared.up", "l0.mlp.e3.down", "l0.canon2",
            "l1.mix.dkv.norm", "l1.mix.uk", "l2.mix.k.norm", "l2.mix.sink", "l4.canon1"} <= names
    assert "l4.canon2" not in names and "l4.norm2" not in names and "l1.mix.dq" not in names
    shapes = model.expected_tensors()
    assert shapes["l1.mix.q"].shape == (4 * 48, 64) and shapes["l1.mix.dkv"].shape == (96, 64) and shapes["l0.mix.norm"].shape == (32,)
    assert shapes["l2.mix.q.norm"].shape == (32,) and shapes["l0.canon1"].shape == (64, 4)


def test_what_a_request_carries():
    model = build_model(copy.deepcopy(CONFIGS["trio"]["config"]))
    shapes = model.state_shapes()
    assert shapes[0] == (2 * 16 * 32,) and shapes[5] == (4 * 8 * 16,) and 1 not in shapes and 2 not in shapes
    assert shapes[(0, "input_conv")] == (2 * 3 * 64,) and shapes[(4, "input_conv")] == (3 * 64,)
    needs = model.cache_needs()
    assert set(needs) == {1, 2, 3, 4} and needs[1].num_kv_heads == 1 and needs[1].head_dim == 96 and needs[4].head_dim == 32
    assert needs[2].head_dim == 64 and needs[2].num_kv_heads == 2
    one = build_model(copy.deepcopy(CONFIGS["one_tap"]["config"]))
    assert one.state_shapes()[(0, "input_conv")] == (1,)


def test_config_errors_name_the_key():
    good = CONFIGS["trio"]["config"]
    for path, value, word in [(("layers", 1, "mixer", "kv_rank"), None, "kv_rank"), (("layers", 2, "mixer", "kv_heads"), 3, "kv_heads"),
                              (("layers", 1, "mixer", "rot", "dims"), 8, "rot_dim"), (("layers", 0, "type"), "mamba", "type"),
                              (("canon",), None, "canon"), (("layers", 0, "mlp", "router", "top"), 9, "top"),
                              (("layers", 1, "mlp", "kind"), "sparse", "kind"), (("layers", 3, "mixer", "rot", "dims"), 66, "dims")]:
        raw = copy.deepcopy(good)
        at = raw
        for k in path[:-1]:
            at = at[k]
        if value is None:
            del at[path[-1]]
        else:
            at[path[-1]] = value
        with pytest.raises(ConfigError, match=word):
            DuvozenConfig.from_dict(raw)
    assert DuvozenConfig.from_dict(copy.deepcopy(good)).to_dict() == good


# ---- the plain implementation's mechanisms, each against another way of computing it ----------------
def test_the_convolution_is_a_sum_over_the_last_inputs():
    g = torch.Generator().manual_seed(1)
    h, w = torch.randn(9, 5, generator=g).double(), torch.randn(5, 3, generator=g).double()
    out = plain.input_convolution(h, w)
    for t in range(9):
        want = h[t].clone()
        for j in range(3):
            src = t - 2 + j
            if src >= 0:
                want += w[:, j] * h[src]
        assert torch.allclose(out[t], want)


def test_the_forget_gate_recurrence_is_a_weighted_sum_of_what_was_written():
    g = torch.Generator().manual_seed(2)
    T, H, d, dv, width = 12, 2, 3, 4, 6
    w = {"m.q": torch.randn(H * d, width, generator=g).double(), "m.v": torch.randn(H * dv, width, generator=g).double(),
         "m.f": torch.randn(H * d, width, generator=g).double(), "m.f.b": torch.randn(H * d, generator=g).double(),
         "m.lower": torch.rand(H * d, generator=g).double(), "m.norm": torch.ones(dv).double(),
         "m.o": torch.eye(H * dv).double()}
    h = torch.randn(T, width, generator=g).double()
    got = plain.forget_gate_recurrence(h, w, "m.", {"heads": H, "dim": d, "vdim": dv}, 0.0)
    q = plain.silu(h @ w["m.q"].T).view(T, H, d)
    v = (h @ w["m.v"].T).view(T, H, dv)
    low = w["m.lower"]
    f = (low + (1 - low) * torch.sigmoid(h @ w["m.f"].T + w["m.f.b"])).view(T, H, d)
    assert (f >= low.view(H, d)).all() and (f < 1).all()
    for t in range(T):
        o = torch.zeros(H, dv, dtype=torch.float64)
        for s in range(t + 1):
            kept = torch.prod(f[s + 1:t + 1], dim=0)            # what is left at t of what was written at s
            o += torch.einsum("hd,hv->hv", q[t] * kept * (1 - f[s]), v[s])
        o = o / torch.sqrt((o * o).mean(-1, keepdim=True))
        assert torch.allclose(got[t], o.reshape(-1), atol=1e-9)


def test_interpolated_frequencies_keep_fast_pairs_and_stretch_slow_ones():
    scaling = {"factor": 4.0, "original": 512, "fast": 16.0, "slow": 2.0}
    freq, magnitude = plain.interpolated_frequencies(32, 10000.0, scaling)
    base = plain.plain_frequencies(32, 10000.0)
    assert magnitude == pytest.approx(0.1 * math.log(4.0) + 1.0)
    turns = 512 * base / (2 * math.pi)              # turns a pair makes within the original positions
    fast, slow = turns >= 16.0, turns <= 2.0
    assert fast.sum() >= 3 and slow.sum() >= 3 and (~fast & ~slow).sum() >= 2
    assert torch.equal(freq[fast], base[fast]) and torch.allclose(freq[slow], base[slow] / 4.0)
    ratio = base / freq
    assert ((ratio[1:] - ratio[:-1]) >= -1e-12).all() and ((ratio[~fast & ~slow] > 1.0) & (ratio[~fast & ~slow] < 4.0)).any()
    # turning by the interleaved pairing is the half-split pairing of the reordered head
    g = torch.Generator().manual_seed(4)
    x, pos = torch.randn(7, 2, 12, generator=g).double(), torch.arange(7)
    a = plain.rotate(x, pos, 8, base[:4], "interleaved", 1.3)
    order = [0, 2, 4, 6, 1, 3, 5, 7, 8, 9, 10, 11]
    b = plain.rotate(x[..., order], pos, 8, base[:4], "half", 1.3)
    assert torch.allclose(a[..., order], b)


def test_a_sink_takes_its_share_and_brings_nothing():
    g = torch.Generator().manual_seed(5)
    scores = torch.randn(2, 6, 6, generator=g).double()
    sink = torch.tensor([30.0, -30.0]).double()
    p = plain.causal_softmax(scores, sink)
    assert p[0].sum(-1).max() < 1e-9 and torch.allclose(p[1].sum(-1), torch.ones(6).double())
    assert torch.equal(torch.triu(p[1], 1), torch.zeros(6, 6).double())


def test_latent_attention_is_attention_over_expanded_keys_and_values():
    c = {"heads": 2, "dim": 4, "rot_dim": 2, "vdim": 3, "kv_rank": 5, "scale": 0.6, "rot": {"dims": 2, "base": 100.0}}
    g = torch.Generator().manual_seed(6)
    width, T = 7, 8
    w = {"m.q": torch.randn(12, width, generator=g), "m.dkv": torch.randn(7, width, generator=g), "m.dkv.norm": torch.rand(5, generator=g) + 0.5,
         "m.uk": torch.randn(8, 5, generator=g), "m.uv": torch.randn(6, 5, generator=g), "m.o": torch.eye(6)}
    w = {k: v.double() for k, v in w.items()}
    h = torch.randn(T, width, generator=g).double()
    got = plain.latent_attention(h, w, "m.", c, 1e-6)
    # the same through the latent itself: a query head carried into its space, the values expanded afterwards
    down = h @ w["m.dkv"].T
    lat = plain.rms_norm(down[:, :5], w["m.dkv.norm"], 1e-6)
    q = (h @ w["m.q"].T).view(T, 2, 6)
    freq = plain.plain_frequencies(2, 100.0)
    qr = plain.rotate(q[..., 4:], torch.arange(T), 2, freq, "interleaved")
    kr = plain.rotate(down[:, 5:].view(T, 1, 2), torch.arange(T), 2, freq, "interleaved")[:, 0]
    uk, uv = w["m.uk"].view(2, 4, 5), w["m.uv"].view(2, 3, 5)
    q_lat = torch.einsum("thd,hdr->thr", q[..., :4], uk)
    scores = (torch.einsum("thr,sr->hts", q_lat, lat) + torch.einsum("thd,sd->hts", qr, kr)) * 0.6
    mixed = torch.einsum("hts,sr->thr", plain.causal_softmax(scores), lat)
    want = torch.einsum("thr,hvr->thv", mixed, uv).reshape(T, 6)
    assert torch.allclose(got, want, atol=1e-10)


def test_an_expert_weighs_its_input():
    g = torch.Generator().manual_seed(7)
    width, ff, T = 6, 5, 9
    w = {"f.router": torch.randn(3, width, generator=g).double()}
    for e in ("e0.", "e1.", "e2.", "shared."):
        w["f." + e + "gate"], w["f." + e + "up"] = torch.randn(ff, width, generator=g).double(), torch.randn(ff, width, generator=g).double()
        w["f." + e + "down"] = torch.randn(width, ff, generator=g).double()
    h = torch.randn(T, width, generator=g).double()
    c = {"router": {"experts": 3, "top": 2}, "shared": {"ff": ff}}
    got = plain.expert_feed_forward(h, w, "f.", c)
    s = torch.sigmoid(h @ w["f.router"].T)
    for t in range(T):
        order = sorted(range(3), key=lambda e: -float(s[t, e]))[:2]
        want = plain.gated_feed_forward(h[t:t + 1], w, "f.shared.", plain.silu)[0]
        for e in order:
            x = s[t, e] * h[t:t + 1]
            want = want + plain.gated_feed_forward(x, w, f"f.e{e}.", plain.silu)[0]
        assert torch.allclose(got[t], want)
    # the weight is no factor of the output: an expert is not linear in its input
    assert not torch.allclose(got[0], plain.gated_feed_forward(h[:1], w, "f.shared.", plain.silu)[0] + sum(
        s[0, e] * plain.gated_feed_forward(h[:1], w, f"f.e{e}.", plain.silu)[0] for e in sorted(range(3), key=lambda e: -float(s[0, e]))[:2]))


# ---- the engine's bookkeeping, with emulated kernels ---------------------------------------------------
@pytest.mark.parametrize("family", list(FAMILIES))
@pytest.mark.parametrize("name", list(CONFIGS))
def test_replay_matches_plain(folders, exact, name, family):
    requests = requests_for(name, LENGTHS[name])
    trace = FAMILIES[family](requests)
    page_size = CONFIGS[name]["page_size"]
    with ops.use_backend(EmulatedKernels(precise=True)):
        model = load_model(folders[name], "float32", "cpu")
        pages = pages_for_max_tokens(max_live_tokens(trace), page_size)
        runner = ModelRunner.create(model, num_pages=pages, page_size=page_size, max_requests=4, poison_freed_pages=True)
        got = replay_and_collect(TraceReplayer(runner), trace)
    runner.cache.check()
    assert not runner.cache.requests
    compare_rows(got, exact[name], relative=2e-4 if name != "sharp" else 2e-3)


@pytest.mark.parametrize("seed", range(6))
def test_configurations_drawn_at_random(tmp_path, seed):
    c = random_config(100 + seed)
    folder = write_folder(c, str(tmp_path / "m"))
    requests = requests_for(c, [37, 18, 50, 26])
    exact = plain_logits(folder, requests, torch.float64)
    for family in ("portions", "mixed"):
        trace = FAMILIES[family](requests)
        with ops.use_backend(EmulatedKernels(precise=True)):
            model = load_model(folder, "float32", "cpu")
            pages = pages_for_max_tokens(max_live_tokens(trace), c["page_size"])
            runner = ModelRunner.create(model, num_pages=pages, page_size=c["page_size"], max_requests=4, poison_freed_pages=True)
            got = replay_and_collect(TraceReplayer(runner), trace)
        runner.cache.check()
        compare_rows(got, exact, relative=3e-4)


def test_a_slot_that_is_used_again_starts_from_nothing(folders):
    """Two requests one after the other in the one slot there is: the second finds the first's state and carried
    rows zeroed, and its logits are those of a request alone."""
    name = "sharp"
    requests = requests_for(name, [40, 33])
    exact = plain_logits(folders[name], requests, torch.float64)
    with ops.use_backend(EmulatedKernels(precise=True)):
        model = load_model(folders[name], "float32", "cpu")
        runner = ModelRunner.create(model, num_pages=6, page_size=16, max_requests=1, poison_freed_pages=True)
        got = replay_and_collect(TraceReplayer(runner), trace_portions(requests, sizes=(7, 2, 12)))
    compare_rows(got, exact, relative=2e-3)


def test_the_carried_rows_of_both_sublayers_move_with_every_step(folders):
    name = "trio"
    toks = requests_for(name, [12])["q0"]
    with ops.use_backend(EmulatedKernels(precise=True)):
        model = load_model(folders[name], "float32", "cpu")
        runner = ModelRunner.create(model, num_pages=4, page_size=16, max_requests=2)
        rep = TraceReplayer(runner)
        rep.run_step({"step": 0, "entries": [{"id": "a", "tokens": toks[:5], "want": []}], "end": []})
        carried = runner.cache.state[(0, "input_conv")][runner.cache.slot("a")].clone()
        width, taps = 64, 4
        mixer_rows = carried[:(taps - 1) * width].view(taps - 1, width)
        ff_rows = carried[(taps - 1) * width:].view(taps - 1, width)
        raw, w = read_folder(folders[name])
        x = w["embed"][torch.as_tensor(toks[:5])] * raw["embedding"]["scale"]
        assert torch.allclose(mixer_rows.double(), x[2:5], atol=1e-6)         # layer 0's mixer reads the embeddings
        assert not torch.allclose(ff_rows, mixer_rows)                        # its feed-forward what the mixer left
        rep.run_step({"step": 1, "entries": [{"id": "a", "tokens": toks[5:6], "want": []}], "end": []})
        moved = runner.cache.state[(0, "input_conv")][runner.cache.slot("a")][:(taps - 1) * width].view(taps - 1, width)
        assert torch.equal(moved[:2], mixer_rows[1:])                         # a step of one token moves them up by one
