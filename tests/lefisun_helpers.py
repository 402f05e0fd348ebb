"""Shared by the Lefisun tests: small configurations that differ in every size and option, model folders
whose weights make every mechanism count, and the comparison with the plain implementation."""
from __future__ import annotations

import copy
import hashlib
import json
import os

import torch

from plain import lefisun_plain
from tokuvik_helpers import compare_rows, random_ids  # noqa: F401  (the comparison is the same)
from wllm_amd.parts import build_model
from wllm_amd.weights.safetensors_io import write_safetensors


def rot(dims, base=10000.0, factor=None):
    r = {"dims": dims, "base": base}
    if factor is not None:
        r["scaling"] = {"factor": factor}
    return r


def experts(ff, count, top, groups=None, keep=None):
    router = {"experts": count, "top": top}
    if groups is not None:
        router["groups"] = {"count": groups, "keep": keep}
    return {"kind": "moe", "expert": {"ff": ff}, "router": router}


def left(heads, kv_heads, dim, vdim, *, chunk, rotation, scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5,
         "rot": rotation}
    if chunk is not None:
        m["mask"] = {"size": chunk}
    return m


def right(heads, dim, vdim, cap):
    return {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}


def parallel(left_mixer, right_mixer, mlp, left_scale=1.0, right_scale=1.0):
    return {"type": "parallel", "mixer": {"left": left_mixer, "right": right_mixer, "left_scale": left_scale,
                                          "right_scale": right_scale}, "mlp": mlp}


def retention(heads, dim, vdim, decay, rotation, mlp):
    return {"type": "retention", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay), "rot": rotation},
            "mlp": mlp}


def config(vocab, width, layers, *, scale=1.0, eps=1e-6):
    return {"architecture": "Lefisun", "vocab": vocab, "width": width, "embedding": {"scale": scale}, "norm": {"eps": eps},
            "layers": layers}


# Heads the matrix cores take (32 and 64; values narrower and wider than keys), a part of the head rotated with
# scaled positions, chunks that are no multiple of the page, experts in groups of which one is shut out, a layer
# without a feed-forward, a retention layer first.
DUO = dict(page_size=16, seed=21, config=config(160, 64, [
    retention(2, 32, 16, (0.9, 0.99), rot(32, 5000.0), experts(32, 4, 1)),
    parallel(left(4, 2, 32, 64, chunk=24, rotation=rot(16, 10000.0, 4.0), scale=0.3), right(2, 16, 32, 8.0),
             experts(48, 6, 2, 3, 2), 1.3, 0.6),
    parallel(left(2, 1, 64, 32, chunk=40, rotation=rot(64, 300.0), scale=0.2), right(4, 8, 16, 3.0), None, 0.7, 1.1),
    retention(4, 16, 16, (0.5, 0.8, 0.95, 0.999), rot(4, 100.0, 2.0), experts(40, 8, 3, 4, 2)),
], scale=1.5, eps=1e-5))

# Sizes no matrix-core kernel takes (heads of 20 and 12, a width of 48, pages of 8), as many key heads as query heads,
# one head, an expert count that is no power of two with every group kept, a top of all allowed experts, a chunk of 7
# and a chunk longer than any request, two parallel layers in a row.
ODD = dict(page_size=8, seed=22, config=config(97, 48, [
    parallel(left(3, 3, 20, 28, chunk=7, rotation=rot(6, 777.0), scale=0.9), right(3, 10, 12, 4.0), experts(24, 5, 3, 5, 5), 1.0, 2.0),
    parallel(left(1, 1, 12, 8, chunk=500, rotation=rot(12, 10000.0, 8.0), scale=0.5), right(1, 36, 5, 50.0), experts(56, 6, 4, 3, 2),
             2.0, 0.25),
    retention(3, 10, 12, (0.7, 0.97, 1.0), rot(10, 20.0), None),
    retention(1, 36, 20, (0.93,), rot(2, 3.0), experts(30, 3, 1, 3, 1)),
], scale=0.7, eps=1e-6))

# Attention so sharp that single keys decide, gates that reach their cap, routers that choose clearly: a key lost
# or gained at a chunk's edge, a stale slot, a wrong page, a lost state or a sink left out moves the logits by far
# more than rounding.
SHARP = dict(page_size=16, seed=23, sharp=True, config=config(200, 96, [
    parallel(left(4, 1, 32, 32, chunk=16, rotation=rot(8, 10000.0, 2.0), scale=1.2), right(2, 32, 32, 2.0),
             experts(64, 8, 2, 4, 2), 1.0, 1.0),
    retention(3, 32, 32, (0.6, 0.9, 0.98), rot(32, 1000.0), experts(64, 4, 2, 2, 1)),
    parallel(left(2, 2, 64, 32, chunk=21, rotation=rot(64, 50.0), scale=0.8), right(3, 16, 32, 1.0), experts(48, 6, 2, 2, 2),
             1.5, 0.5),
], scale=1.0, eps=1e-6))

CONFIGS = {"duo": DUO, "odd": ODD, "sharp": SHARP}


def middling_config(seed: int) -> dict:
    """Widths of some hundred and heads as a small real model has them: the sizes at which steps of a few hundred
    rows take the library's products, the tiled kernels and the matrix-core attention."""
    import random
    r = random.Random(seed)
    width = r.choice([256, 384, 512])
    kv = r.choice([1, 2])
    dim, vdim = r.choice([(64, 96), (128, 64), (64, 64), (96, 128)])
    heads = kv * r.choice([2, 4])
    mem_heads = r.choice([2, 4])
    layers = [
        parallel(left(heads, kv, dim, vdim, chunk=r.choice([130, 200, 333]), rotation=rot(r.choice([dim, dim // 2]), 10000.0,
                                                                                            r.choice([None, 2.0]))),
                 right(mem_heads, r.choice([32, 48, 64]), r.choice([64, 96]), r.choice([5.0, 15.0])),
                 experts(r.choice([128, 192]), 8, r.choice([2, 3]), 4, r.choice([2, 3])), 1.0, 0.8),
        retention(4, r.choice([32, 64]), r.choice([64, 128]), (0.97, 0.99, 0.995, 0.999), rot(32, 1e5),
                  experts(160, r.choice([4, 6]), 2)),
        parallel(left(4, 4, 64, 64, chunk=r.choice([64, 257]), rotation=rot(32, 500.0)), right(2, 128, 64, 10.0), None, 0.5, 1.0),
        retention(2, 128, 96, (0.9, 0.9995), rot(64, 1e4, 4.0), experts(96, 16, 4, 4, 2)),
    ]
    r.shuffle(layers)
    return dict(page_size=16, seed=seed, config=config(r.choice([1000, 2048]), width, layers, scale=r.choice([1.0, 0.3])))


def random_config(seed: int) -> dict:
    """A configuration drawn from what the design allows: any order of mixers, any sizes."""
    import random
    r = random.Random(seed)
    width = r.choice([32, 48, 64, 80])

    def draw_experts():
        if r.random() < 0.25:
            return None
        groups = r.choice([1, 2, 3, 4])
        per = r.choice([1, 2, 3])
        keep = r.randint(1, groups)
        return experts(r.choice([8, 24, 40, 72]), groups * per, r.randint(1, keep * per), *((groups, keep) if r.random() < 0.8 else
                                                                                           (None, None) if keep == groups == 1
                                                                                           else (groups, keep)))

    def draw_rot(dim):
        dims = r.choice([d for d in (2, 4, 8, 16, 32, dim) if d <= dim and d % 2 == 0])
        return rot(dims, r.choice([10.0, 1000.0, 1e6]), r.choice([None, 2.0, 8.0]))

    layers = []
    for _ in range(r.randint(2, 5)):
        if r.random() < 0.5:
            kv = r.choice([1, 2, 3])
            dim = r.choice([8, 20, 32, 64])
            mem_heads = r.choice([1, 2, 5])
            layers.append(parallel(
                left(kv * r.choice([1, 2, 4]), kv, dim, r.choice([4, 16, 32, 40]), chunk=r.choice([1, 5, 16, 33, 1000]),
                     rotation=draw_rot(dim), scale=r.choice([0.3, 1.0])),
                right(mem_heads, r.choice([4, 16, 33, 70]), r.choice([4, 16, 24, 72]), r.choice([0.5, 5.0, 30.0])),
                draw_experts(), r.choice([0.5, 1.0, 2.0]), r.choice([0.5, 1.0, 2.0])))
        else:
            heads = r.choice([1, 2, 3, 6])
            dim = r.choice([4, 10, 16, 64, 130])
            layers.append(retention(heads, dim, r.choice([4, 16, 24, 72]), [r.choice([0.3, 0.9, 0.99, 1.0]) for _ in range(heads)],
                                    draw_rot(dim), draw_experts()))
    return dict(page_size=r.choice([4, 8, 16]), seed=seed,
                config=config(r.choice([64, 130, 300]), width, layers, scale=r.choice([0.5, 1.0, 3.0]), eps=r.choice([1e-6, 1e-5])))


def _draw(name: str, shape: tuple, seed: int, sharp: bool) -> torch.Tensor:
    g = torch.Generator().manual_seed(seed)
    n = torch.randn(shape, generator=g)
    last = name.rsplit(".", 1)[-1]
    if last in ("norm1", "norm2", "norm"):
        t = 1.0 + 0.3 * n                       # plain weights around one
    elif name.endswith((".i.b", ".f.b")):
        t = (1.0 if name.endswith(".f.b") else 0.0) + n        # forget gates that keep most, input gates of any size
    elif last == "b":
        t = 0.3 * n
    elif last in ("i", "f"):
        t = n * (shape[-1] ** -0.5) * (4.0 if sharp else 1.5)  # log gates of a few units: the cap bends them
    elif last == "router":
        t = n * (shape[-1] ** -0.5) * (6.0 if sharp else 2.0)  # scores that differ
    elif name == "embed":
        t = n
    else:
        t = n * (shape[-1] ** -0.5)             # a projection keeps its input's size
    return t.to(torch.bfloat16)


def write_folder(name, folder: str) -> str:
    """A model folder for one of CONFIGS (or a dict of the same form): config.json and weights that make
    every part count (norm weights around one, biases, gates that reach their cap, routers that choose)."""
    c = CONFIGS[name] if isinstance(name, str) else name
    raw = copy.deepcopy(c["config"])
    expected = build_model(copy.deepcopy(raw)).expected_tensors()
    tensors = {}
    for tensor_name, exp in expected.items():
        stable = int.from_bytes(hashlib.sha256(f"{c['seed']}:{tensor_name}".encode()).digest()[:4], "little")
        tensors[tensor_name] = _draw(tensor_name, tuple(exp.shape), stable, bool(c.get("sharp")))
    os.makedirs(folder, exist_ok=True)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors, metadata={"format": "pt"})
    with open(os.path.join(folder, "config.json"), "w", encoding="utf-8") as f:
        json.dump(raw, f, indent=1, sort_keys=True)
    return folder


def read_folder(folder: str, dtype=torch.float64):
    from wllm_amd.weights.checkpoint import Checkpoint
    with open(os.path.join(folder, "config.json"), encoding="utf-8") as f:
        raw = json.load(f)
    ck = Checkpoint(folder)
    try:
        weights = {n: ck.tensor(n).to(dtype).clone() for n in ck.names()}
    finally:
        ck.close()
    return raw, weights


def requests_for(name, lengths) -> dict:
    c = CONFIGS[name] if isinstance(name, str) else name
    return {f"q{i}": random_ids(1000 * i + c["seed"], n, c["config"]["vocab"]) for i, n in enumerate(lengths)}


def plain_logits(folder: str, requests: dict, dtype=torch.float64) -> dict:
    raw, weights = read_folder(folder, dtype)
    return {rid: lefisun_plain.forward(raw, weights, toks, dtype) for rid, toks in requests.items()}


def rounding_noise(folder: str, requests: dict, dtype, exact: dict) -> dict:
    """How far rounding alone carries every row: the plain implementation in float32, or in float64 with every
    tensor a bfloat16 model holds rounded to bfloat16, against the exact rows.  Some rows amplify rounding (a
    normaliser that nearly cancels, a router between two experts of almost equal score); a row's bound follows it."""
    raw, weights = read_folder(folder, torch.float64)
    noise = {}
    for rid, toks in requests.items():
        if dtype == torch.float32:
            noisy = lefisun_plain.forward(raw, weights, toks, torch.float32).double()
        else:
            noisy = lefisun_plain.forward(raw, weights, toks, torch.float64, lefisun_plain.to_bfloat16)
        d = noisy - exact[rid]
        noise[rid] = (d - d.mean(-1, keepdim=True)).pow(2).mean(-1).sqrt()
    return noise


def compare_with_rounding(collected: dict, exact: dict, noise: dict, *, relative: float, times: float = 4.0,
                          outliers: float = 0.0) -> float:
    """Every collected row against the exact one: the root mean square of the difference (its mean taken off) may be
    `relative` of the exact row's own, or `times` what rounding alone does to that row in the plain implementation,
    whichever is larger.  A share `outliers` of the rows may lie beyond (bfloat16: the engine's rounding falls
    otherwise than the plain implementation's, and another expert or key wins).  Returns the worst error in bounds."""
    errors = {}
    for (rid, pos) in sorted(collected, key=lambda k: (str(k[0]), k[1])):
        got, ref = collected[(rid, pos)].double().cpu(), exact[rid][pos].double()
        assert torch.isfinite(got).all(), f"request {rid!r} position {pos}: logits are not finite"
        d = got - ref
        bound = max(relative * max((ref - ref.mean()).pow(2).mean().sqrt().item(), 1e-3), times * float(noise[rid][pos]))
        errors[(rid, pos)] = (d - d.mean()).pow(2).mean().sqrt().item() / bound
    beyond = {k: e for k, e in errors.items() if e > 1.0}
    assert len(beyond) <= outliers * len(errors), (
        f"{len(beyond)} of {len(errors)} rows beyond the bound; the first: request {next(iter(beyond))[0]!r} position "
        f"{next(iter(beyond))[1]}: {next(iter(beyond.values())):.2f} x the bound")
    return max(errors.values())
