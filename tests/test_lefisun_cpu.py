"""Lefisun without a GPU: its configuration, its plan, the plain implementation's own mechanisms against a
second way of computing each, and the engine's bookkeeping around it (a cache and a state row in one layer,
chunks that give pages back, state slots that are zeroed and used again) against the plain implementation,
the kernels replaced by the emulation of their contracts."""
import copy
import math

import pytest
import torch

from helpers import max_live_tokens, replay_and_collect, trace_mixed, trace_portions, trace_tail, trace_whole
from kernel_emulation import EmulatedKernels
from lefisun_helpers import (CONFIGS, compare_rows, config, experts, left, parallel, plain_logits, random_config, read_folder,
                             requests_for, retention, right, rot, write_folder)
from plain import lefisun_plain as plain
from wllm_amd.architectures import LefisunConfig
from wllm_amd.config import ConfigError
from wllm_amd.engine import ModelRunner
from wllm_amd.engine.replay import TraceReplayer, pages_for_max_tokens
from wllm_amd.kernels import ops
from wllm_amd.parts import build_model, load_model

LENGTHS = {"duo": [70, 45, 90, 33, 58], "odd": [40, 66, 25, 51], "sharp": [80, 37, 64, 50]}
FAMILIES = {"whole": trace_whole, "tail": trace_tail, "portions": trace_portions, "mixed": trace_mixed}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("lefisun")
    return {name: write_folder(name, str(root / name)) for name in CONFIGS}


@pytest.fixture(scope="module")
def exact(folders):
    return {name: plain_logits(folders[name], requests_for(name, LENGTHS[name]), torch.float64) for name in CONFIGS}


# ---- configuration and plan ------------------------------------------------------------------------
def test_the_plan_follows_the_file():
    model = build_model(copy.deepcopy(CONFIGS["duo"]["config"]))
    plan = model.plan
    assert [type(b.mixer).__name__ for b in plan.layers] == ["MatrixMemorySpec", "SideBySideSpec", "SideBySideSpec",
                                                             "MatrixMemorySpec"]
    first, pair = plan.layers[0].mixer, plan.layers[1].mixer
    assert first.gating == "decay" and first.decays == (0.9, 0.99) and first.k_scale == 32 ** -0.5 and first.q_scale == 1.0
    assert first.gate_activation == "silu" and first.norm_weight is None and first.position.rotary_dim == 32
    a, m = pair.left, pair.right
    assert (a.num_heads, a.num_kv_heads, a.head_dim, a.value_dim, a.chunk, a.release_chunk) == (4, 2, 32, 64, 24, 24)
    assert a.sink == 0.0 and a.bias_before_norm and a.output_scale == 1.3 and a.scale == 0.3
    assert a.position.rotary_dim == 16 and a.position.scaling_factor == 4.0 and a.position.pairing == "half"
    assert m.gating == "exponential" and m.gate_cap == 8.0 and m.q_scale == 16 ** -0.5 and m.output_scale == 0.6
    assert m.gate_activation == "sigmoid" and m.norm_weight == "l1.mix.right.norm"
    ff = plan.layers[1].feed_forward
    assert (ff.num_experts, ff.top, ff.num_groups, ff.keep_groups, ff.intermediate_size) == (6, 2, 3, 2, 48)
    assert plan.layers[0].feed_forward.num_groups == 1          # a file without groups: nothing is shut out
    assert plan.layers[2].feed_forward is None and plan.layers[2].feed_forward_norm is None
    assert plan.embedding.scale == 1.5 and plan.head.weight is None
    names = set(model.expected_tensors())
    assert {"embed", "final.norm", "l0.mix.q", "l0.mix.g", "l0.mlp.router", "l0.mlp.e3.down", "l1.mix.left.q.b",
            "l1.mix.left.k.norm", "l1.mix.right.i.b", "l1.mix.right.f", "l1.mix.right.norm", "l1.mlp.e5.gate"} <= names
    assert not any(n.startswith(("l2.mlp", "l2.norm2", "l0.mix.norm")) for n in names) and "head" not in names
    # a parallel layer holds pages (its attention) and a state row (its memory); a retention layer a state row
    assert sorted(model.cache_needs()) == [1, 2] and sorted(model.state_shapes()) == [0, 1, 2, 3]
    assert model.cache_needs()[1].chunk == 24 and model.cache_needs()[2].chunk == 40
    assert model.state_shapes()[0] == (2 * 32 * 16,) and model.state_shapes()[1] == (2 * 16 * 32 + 2 * 16 + 2,)


@pytest.mark.parametrize("change, words", [
    (lambda c: c["layers"][1]["mixer"]["left"].pop("scale"), "scale"),
    (lambda c: c["layers"][1]["mixer"]["left"].update(kv_heads=3), "multiple"),
    (lambda c: c["layers"][1]["mixer"].pop("right_scale"), "right_scale"),
    (lambda c: c["layers"][1]["mixer"]["right"].pop("gate_cap"), "gate_cap"),
    (lambda c: c["layers"][1]["mixer"]["left"]["rot"].update(dims=34), "dims"),
    (lambda c: c["layers"][0].update(type="scan"), "mixers"),
    (lambda c: c["layers"][0]["mixer"].update(decay=[0.5]), "decay"),
    (lambda c: c["layers"][0]["mlp"].update(kind="dense"), "moe"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=5), "top"),
    (lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(count=4), "divide"),
    (lambda c: c.pop("embedding"), "embedding"),
    (lambda c: c.pop("norm"), "norm"),
])
def test_a_file_that_the_design_does_not_cover_is_refused(change, words):
    raw = copy.deepcopy(CONFIGS["duo"]["config"])
    change(raw)
    with pytest.raises(ConfigError, match=words):
        LefisunConfig.from_dict(raw)


def test_the_configuration_writes_the_file_it_read():
    raw = copy.deepcopy(CONFIGS["odd"]["config"])
    cfg = LefisunConfig.from_dict(raw)
    again = LefisunConfig.from_dict(LefisunConfig(cfg.vocab, cfg.width, cfg.embedding_scale, cfg.norm_eps, cfg.layers).to_dict())
    assert again.layers == cfg.layers and again.embedding_scale == cfg.embedding_scale


# ---- the plain mechanisms against a second way of computing each -------------------------------------
def test_retention_is_the_sum_it_unrolls_to():
    """o_t = sum over s <= t of decay^(t-s) (q_t . k_s) v_s / sqrt(d), with both rotated: written out for one head."""
    torch.manual_seed(0)
    T, d, dv, width = 7, 4, 3, 5
    c = {"heads": 1, "dim": d, "vdim": dv, "decay": [0.8], "rot": {"dims": 2, "base": 7.0}}
    w = {"m.q": torch.randn(d, width), "m.k": torch.randn(d, width), "m.v": torch.randn(dv, width),
         "m.g": torch.randn(dv, width), "m.o": torch.eye(dv)}
    w = {k: v.double() for k, v in w.items()}
    h = torch.randn(T, width, dtype=torch.float64)
    got = plain.retention(h, w, "m.", c, 1e-6)
    q, k, v = h @ w["m.q"].T, h @ w["m.k"].T, h @ w["m.v"].T

    def turned(x, t):      # elements 0 and 1 are a pair (dims 2: i = 0 pairs with 1), frequency 7^0 = 1
        out = x.clone()
        out[0] = x[0] * math.cos(t) - x[1] * math.sin(t)
        out[1] = x[1] * math.cos(t) + x[0] * math.sin(t)
        return out
    rows = []
    for t in range(T):
        o = torch.zeros(dv, dtype=torch.float64)
        for s in range(t + 1):
            o += 0.8 ** (t - s) * (turned(q[t], t) @ turned(k[s], s)) / math.sqrt(d) * v[s]
        rows.append(o)
    o = torch.stack(rows)
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + 1e-6)
    g = h @ w["m.g"].T
    assert torch.allclose(got, o * g * torch.sigmoid(g), atol=1e-12)


def test_the_matrix_memory_is_the_weighted_sum_its_maximum_hides():
    """Without the running maximum: C_t = sigma(f) C + exp(i) k v^T, n likewise, o = C^T q / max(|n . q|, 1); the
    maximum only rescales numerator and denominator, up to the floor exp(-m) and the 1e-6."""
    torch.manual_seed(1)
    T, d, dv, width, cap = 9, 3, 2, 4, 2.5
    c = {"heads": 1, "dim": d, "vdim": dv, "gate_cap": cap}
    w = {k: torch.randn(*s).double() for k, s in {"m.q": (d, width), "m.k": (d, width), "m.v": (dv, width), "m.g": (dv, width),
                                                  "m.i": (1, width), "m.f": (1, width), "m.i.b": (1,), "m.f.b": (1,)}.items()}
    w["m.o"], w["m.norm"] = torch.eye(dv, dtype=torch.float64), torch.tensor([0.7, 1.3], dtype=torch.float64)
    h = torch.randn(T, width, dtype=torch.float64)
    got = plain.matrix_memory(h, w, "m.", c, 0.0)
    q, k, v = h @ w["m.q"].T / math.sqrt(d), h @ w["m.k"].T, h @ w["m.v"].T
    log_i = cap * torch.tanh((h @ w["m.i"].T + w["m.i.b"]) / cap)
    forget = torch.sigmoid(cap * torch.tanh((h @ w["m.f"].T + w["m.f.b"]) / cap))
    C, n, rows, m = torch.zeros(d, dv).double(), torch.zeros(d).double(), [], 0.0
    for t in range(T):
        C = forget[t] * C + torch.exp(log_i[t]) * torch.outer(k[t], v[t])
        n = forget[t] * n + torch.exp(log_i[t]) * k[t]
        m = max(math.log(float(forget[t])) + m, float(log_i[t]))
        rows.append((C.T @ q[t]) / (torch.maximum((n @ q[t]).abs(), torch.tensor(1.0).double()) + 1e-6 * math.exp(m)))
    o = torch.stack(rows)
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True)) * w["m.norm"] * torch.sigmoid(h @ w["m.g"].T)
    assert torch.allclose(got, o, atol=1e-9)


def test_the_router_keeps_the_best_groups_only():
    h = torch.eye(8, dtype=torch.float64)[:1] * 1.0
    router = torch.tensor([[3.0, 0.1, 2.9, 0.2, 2.8, 2.7, 0.0, 0.0]], dtype=torch.float64).T @ torch.ones(1, 1, dtype=torch.float64)
    router = torch.cat([router, torch.zeros(8, 7, dtype=torch.float64)], dim=1)
    # groups of two: best scores 3.0, 2.9, 2.8, 0.0; two kept: experts 0..3; the third best expert overall (4) is shut out
    chosen, weights = plain.route(h, router, 8, 3, 4, 2)
    assert sorted(chosen[0].tolist()) == [0, 2, 3]
    assert abs(float(weights.sum()) - 1.0) < 1e-12
    chosen, _ = plain.route(h, router, 8, 3, 4, 4)
    assert sorted(chosen[0].tolist()) == [0, 2, 4]


def test_the_sharp_model_shows_a_key_lost_at_a_chunks_edge_a_sink_left_out_and_a_state_that_starts_elsewhere(folders, monkeypatch):
    raw, w = read_folder(folders["sharp"])
    tokens = requests_for("sharp", [80])["q0"]
    correct = plain.forward(raw, w, tokens)

    def far(other):
        return (other - correct).pow(2).mean(-1).sqrt() / correct.pow(2).mean(-1).sqrt()
    for step in (-1, 1):
        other = copy.deepcopy(raw)
        for entry in other["layers"]:
            if entry["type"] == "parallel":
                entry["mixer"]["left"]["mask"]["size"] += step
        assert (far(plain.forward(other, w, tokens))[24:] > 1e-2).float().mean() > 0.8
    # the sink: a softmax whose denominator holds nothing but the keys
    def no_sink(scores, mask):
        return torch.softmax(scores.masked_fill(~mask, float("-inf")), dim=-1)
    monkeypatch.setattr(plain, "softmax_plus_one", no_sink)
    assert (far(plain.forward(raw, w, tokens)) > 1e-2).float().mean() > 0.8
    monkeypatch.undo()
    # a decay that is a little off moves every row behind the first
    other = copy.deepcopy(raw)
    other["layers"][1]["mixer"]["decay"] = [d * 0.97 for d in other["layers"][1]["mixer"]["decay"]]
    assert (far(plain.forward(other, w, tokens))[4:] > 1e-2).float().mean() > 0.8


# ---- the engine around emulated kernels --------------------------------------------------------------
@pytest.mark.parametrize("family", list(FAMILIES))
@pytest.mark.parametrize("name", list(CONFIGS))
def test_replay_matches_plain(folders, exact, name, family):
    requests = requests_for(name, LENGTHS[name])
    trace = FAMILIES[family](requests)
    page_size = CONFIGS[name]["page_size"]
    with ops.use_backend(EmulatedKernels(splits=3 if family in ("tail", "mixed") else 1)) as emulated:
        model = load_model(folders[name], "float32", "cpu")
        pages = pages_for_max_tokens(max_live_tokens(trace), page_size)
        runner = ModelRunner.create(model, num_pages=pages, page_size=page_size, max_requests=4, poison_freed_pages=True)
        got = replay_and_collect(TraceReplayer(runner), trace)
        runner.cache.check()
        assert not runner.cache.requests
        assert all(g.pool.num_free == g.pool.num_pages for g in runner.cache.groups)
        for op in ("memory_scan", "memory_gates", "head_norm_gate", "moe_route", "moe_experts_down", "band_norm"):
            assert emulated.calls.get(op, 0) > 0, op
    assert len(got) == sum(len(t) for t in requests.values())
    compare_rows(got, exact[name], relative=5e-4 if name == "sharp" else 5e-5)


def test_chunks_give_their_pages_back_while_the_request_runs(folders):
    """A request far longer than the attention's pool: only the chunks make it fit, and freed pages (filled
    with NaN when they are given back) are used again by the same request."""
    c = copy.deepcopy(CONFIGS["sharp"])
    with __import__("tempfile").TemporaryDirectory() as folder:
        write_folder(c, folder)
        requests = requests_for(c, [300])
        reference = plain_logits(folder, requests, torch.float64)
        trace = trace_portions(requests, sizes=(16, 5, 2, 11, 1, 1, 1, 7, 3, 2, 9))
        with ops.use_backend(EmulatedKernels()):
            model = load_model(folder, "float32", "cpu")
            runner = ModelRunner.create(model, num_pages=4, page_size=16, max_requests=2, poison_freed_pages=True)
            got = replay_and_collect(TraceReplayer(runner), trace)
            runner.cache.check()
    compare_rows(got, reference, relative=5e-4)


def test_a_state_slot_that_is_used_again_starts_from_zero(folders):
    """Two slots, five requests one after the other and side by side: a request's memory, normaliser and
    running maximum must not begin where the slot's last holder ended."""
    name = "duo"
    requests = requests_for(name, [30, 21, 17, 26, 12])
    reference = plain_logits(folders[name], requests, torch.float64)
    trace = trace_mixed(requests, seed=3, live=2)
    with ops.use_backend(EmulatedKernels()):
        model = load_model(folders[name], "float32", "cpu")
        runner = ModelRunner.create(model, num_pages=12, page_size=16, max_requests=2, poison_freed_pages=True)
        got = replay_and_collect(TraceReplayer(runner), trace)
        runner.cache.check()
    compare_rows(got, reference, relative=5e-5)


@pytest.mark.parametrize("seed", range(6))
def test_configurations_drawn_at_random(tmp_path, seed):
    c = random_config(100 + seed)
    folder = write_folder(c, str(tmp_path / "m"))
    requests = requests_for(c, [37, 18, 50])
    reference = plain_logits(folder, requests, torch.float64)
    trace = trace_mixed(requests, seed=seed, live=3)
    with ops.use_backend(EmulatedKernels()):
        model = load_model(folder, "float32", "cpu")
        pages = pages_for_max_tokens(max_live_tokens(trace), c["page_size"])
        runner = ModelRunner.create(model, num_pages=pages, page_size=c["page_size"], max_requests=3, poison_freed_pages=True)
        got = replay_and_collect(TraceReplayer(runner), trace)
        runner.cache.check()
    compare_rows(got, reference, relative=5e-4)


@pytest.mark.parametrize("layers", [
    [retention(2, 8, 4, (0.5, 0.9), rot(8, 30.0), experts(16, 2, 2)), retention(1, 4, 6, (1.0,), rot(2, 5.0), None)],   # no pages at all
    [parallel(left(2, 1, 8, 4, chunk=None, rotation=rot(4, 100.0)), right(1, 4, 4, 3.0), None)],     # no mask, no feed-forward
    [parallel(left(1, 1, 4, 8, chunk=1, rotation=rot(4, 9.0, 3.0)), right(2, 4, 2, 1.0), experts(8, 1, 1, 1, 1), 0.0, 1.0)],
])
def test_models_of_one_kind_of_mixer(tmp_path, layers):
    """Also: one expert that every token uses, a chunk of one position (a token sees itself and the sink), and a
    left half that counts for nothing."""
    c = dict(page_size=4, seed=5, config=config(40, 16, copy.deepcopy(layers), scale=0.9))
    folder = write_folder(c, str(tmp_path / "m"))
    requests = requests_for(c, [21, 9, 14])
    reference = plain_logits(folder, requests, torch.float64)
    trace = trace_mixed(requests, seed=1, live=2)
    with ops.use_backend(EmulatedKernels()):
        model = load_model(folder, "float32", "cpu")
        runner = ModelRunner.create(model, num_pages=pages_for_max_tokens(max_live_tokens(trace), 4), page_size=4,
                                    max_requests=2, poison_freed_pages=True)
        got = replay_and_collect(TraceReplayer(runner), trace)
        runner.cache.check()
    compare_rows(got, reference, relative=5e-5)


def test_many_rows_an_expert_take_the_plan_of_large_tiles(tmp_path):
    """bfloat16, sizes in multiples of 64 and a portion of some hundred tokens: the step plans tiles of 128 rows
    (shorter steps of the same request tiles of 16), and the rows are the plain implementation's within bfloat16."""
    c = dict(page_size=16, seed=9, config=config(120, 64, [
        retention(2, 16, 32, (0.9, 0.99), rot(16, 100.0), experts(64, 4, 2, 2, 1)),
        parallel(left(2, 1, 32, 32, chunk=100, rotation=rot(16, 1000.0)), right(2, 16, 16, 5.0), experts(128, 2, 1), 1.0, 1.0)]))
    folder = write_folder(c, str(tmp_path / "m"))
    requests = requests_for(c, [300])
    reference = plain_logits(folder, requests, torch.float64)
    toks = requests["q0"]
    trace = [{"step": 0, "entries": [{"id": "q0", "tokens": toks[:260], "want": list(range(0, 260, 7))}], "end": []},
             {"step": 1, "entries": [{"id": "q0", "tokens": toks[260:], "want": list(range(40))}], "end": ["q0"]}]
    with ops.use_backend(EmulatedKernels()) as emulated:
        model = load_model(folder, "bfloat16", "cpu")
        runner = ModelRunner.create(model, num_pages=20, page_size=16, max_requests=2)
        got = replay_and_collect(TraceReplayer(runner), trace)
        # the first step's two layers took the large tiles, the second step's the small ones
        assert emulated.calls.get("moe_experts_up_tiled", 0) == 2 and emulated.calls.get("moe_experts_down_tiled", 0) == 2
        assert emulated.calls.get("moe_experts_up", 0) == 4
    assert ops.moe_tile_rows(260 * 2, 4, torch.bfloat16, 64, 64) == 128 and ops.moe_tile_rows(40 * 2, 4, torch.bfloat16, 64, 64) == 64
    assert ops.moe_tile_rows(260 * 2, 4, torch.float32, 64, 64) == 64 and ops.moe_tile_rows(260 * 2, 4, torch.bfloat16, 64, 96) == 64
    assert ops.moe_tile_rows(8, 4, torch.bfloat16, 64, 64) == 16 and ops.moe_tile_rows(48, 4, torch.bfloat16, 64, 64) == 32
    compare_rows(got, reference, relative=0.05, outliers=0.1, ceiling=10.0)
