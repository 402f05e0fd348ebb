"""Shared by the Duvozen tests: small configurations that differ in every size and option, model folders
whose weights make every mechanism count, and the comparison with the plain implementation."""
from __future__ import annotations

import copy
import hashlib
import json
import os

import torch

from lefisun_helpers import compare_with_rounding  # noqa: F401  (the comparison is the same)
from plain import duvozen_plain
from tokuvik_helpers import compare_rows, random_ids  # noqa: F401
from wllm_amd.parts import build_model
from wllm_amd.weights.safetensors_io import write_safetensors


def to_bfloat16(x):
    return x.to(torch.bfloat16).to(x.dtype)


def rot(dims, base=10000.0, scaling=None):
    r = {"dims": dims, "base": base}
    if scaling is not None:
        r["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return r


def recurrence(heads, dim, vdim):
    return "hgrn2", {"heads": heads, "dim": dim, "vdim": vdim}


def latent(heads, dim, rot_dim, vdim, kv_rank, *, base=10000.0, scaling=None, scale=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale if scale is not None else (dim + rot_dim) ** -0.5}
    if rot_dim:
        m["rot_dim"], m["rot"] = rot_dim, rot(rot_dim, base, scaling)
    return "latent_attention", m


def attention(heads, kv_heads, dim, vdim, *, rot_dims, base=10000.0, scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5}
    if rot_dims:
        m["rot"] = rot(rot_dims, base)
    return "attention", m


def dense(ff):
    return {"kind": "dense", "ff": ff}


def experts(ff, count, top, shared=None):
    m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": count, "top": top}}
    if shared is not None:
        m["shared"] = {"ff": shared}
    return m


def layer(mixer, mlp):
    return {"type": mixer[0], "mixer": mixer[1], "mlp": mlp}


def config(vocab, width, layers, *, taps, scale=1.0, logit_scale=1.0, eps=1e-6):
    return {"architecture": "Duvozen", "vocab": vocab, "width": width, "embedding": {"scale": scale}, "logit_scale": logit_scale,
            "norm": {"eps": eps}, "canon": {"taps": taps}, "layers": layers}


# Heads the matrix cores take (32, 64 and a latent head of 96), values narrower and wider than keys, a part of the head
# and the whole head turned, interpolated frequencies of which some pairs are fast, some slow and some between, a
# recurrence first, experts with and without the one every token uses, a top of two and three.
TRIO = dict(page_size=16, seed=31, config=config(160, 64, [
    layer(recurrence(2, 16, 32), experts(32, 4, 2, shared=48)),
    layer(latent(4, 32, 16, 16, 80, base=100.0, scaling=(4.0, 64, 8.0, 1.0), scale=0.2), dense(96)),
    layer(attention(4, 2, 32, 64, rot_dims=16, base=10000.0, scale=0.3), experts(48, 6, 3)),
    layer(attention(2, 1, 64, 32, rot_dims=64, base=300.0), dense(80)),
    layer(latent(2, 16, 8, 32, 24, base=50.0), None),
    layer(recurrence(4, 8, 16), dense(72)),
], taps=4, scale=1.5, logit_scale=0.7, eps=1e-5))

# Sizes no matrix-core kernel takes (heads of 20 and 12, a latent of 36 + 6, a width of 48, pages of 8), as many key heads
# as query heads, one head, one expert of which one is chosen, a top of all experts, a convolution of two taps, a
# recurrence whose channels are more than a wavefront, a latent attention without a turned part.
ODD = dict(page_size=8, seed=32, config=config(97, 48, [
    layer(attention(3, 3, 20, 28, rot_dims=6, base=777.0, scale=0.9), experts(24, 5, 5, shared=8)),
    layer(latent(3, 10, 6, 12, 36, base=20.0, scaling=(8.0, 16, 4.0, 0.5), scale=0.5), experts(56, 1, 1)),
    layer(recurrence(1, 130, 5), dense(40)),
    layer(latent(1, 12, 0, 20, 9, scale=0.4), dense(56)),
    layer(recurrence(3, 10, 12), None),
    layer(attention(1, 1, 12, 8, rot_dims=0, scale=0.5), experts(30, 3, 1, shared=30)),
], taps=2, scale=0.7, logit_scale=2.0, eps=1e-6))

# Attention so sharp that single keys decide, sinks that take most of the weight in some heads and little in others,
# forget gates from nearly nothing to nearly one, routers that choose clearly, a convolution as strong as its input:
# a key lost or gained, a stale slot, a wrong page, a lost state or carried row or a sink left out moves the logits
# by far more than rounding.
SHARP = dict(page_size=16, seed=33, sharp=True, config=config(200, 96, [
    layer(attention(4, 1, 32, 32, rot_dims=8, base=10000.0, scale=1.2), experts(64, 8, 2, shared=32)),
    layer(recurrence(3, 32, 32), dense(64)),
    layer(latent(4, 16, 16, 32, 48, base=1000.0, scaling=(8.0, 32, 16.0, 1.0), scale=1.0), experts(48, 6, 2)),
    layer(attention(2, 2, 64, 32, rot_dims=64, base=50.0, scale=0.8), dense(64)),
], taps=3, scale=1.0, logit_scale=1.0, eps=1e-6))

# One tap: the convolution carries nothing from token to token.
ONE_TAP = dict(page_size=4, seed=34, config=config(64, 32, [
    layer(latent(2, 8, 4, 8, 12, base=10.0), dense(24)),
    layer(recurrence(2, 4, 8), experts(16, 2, 1)),
    layer(attention(2, 1, 8, 8, rot_dims=8, base=10.0), None),
], taps=1, scale=1.0, logit_scale=0.5))

CONFIGS = {"trio": TRIO, "odd": ODD, "sharp": SHARP, "one_tap": ONE_TAP}


def middling_config(seed: int) -> dict:
    """Widths of some hundred and heads as a small real model has them: the sizes at which steps of a few hundred
    rows take the library's products, the tiled kernels and the matrix-core attention."""
    import random
    r = random.Random(seed)
    width = r.choice([256, 384, 512])
    kv = r.choice([1, 2])
    dim, vdim = r.choice([(64, 96), (128, 64), (64, 64), (96, 128)])
    layers = [
        layer(attention(kv * r.choice([2, 4]), kv, dim, vdim, rot_dims=r.choice([dim, dim // 2]), base=10000.0),
              experts(r.choice([128, 192]), 8, r.choice([1, 2, 3]), shared=r.choice([None, 128, 64]))),
        layer(latent(r.choice([4, 8]), r.choice([32, 64]), r.choice([16, 32]), r.choice([32, 64]), r.choice([96, 160, 224]),
                     base=1e5, scaling=r.choice([None, (8.0, 256, 32.0, 1.0)])), dense(r.choice([320, 512]))),
        layer(recurrence(r.choice([2, 4]), r.choice([32, 64, 128]), r.choice([64, 96])), experts(96, 16, 4, shared=96)),
        layer(recurrence(4, 48, 64), dense(256)),
        layer(latent(4, 64, 32, 64, 128, base=500.0), None),
    ]
    r.shuffle(layers)
    return dict(page_size=16, seed=seed, config=config(r.choice([1000, 2048]), width, layers, taps=r.choice([2, 3, 4]),
                                                       scale=r.choice([1.0, 0.3]), logit_scale=r.choice([1.0, 0.25])))


def random_config(seed: int) -> dict:
    """A configuration drawn from what the design allows: any order of mixers, any sizes."""
    import random
    r = random.Random(seed)
    width = r.choice([32, 48, 64, 80, 72, 100])

    def draw_mlp():
        u = r.random()
        if u < 0.2:
            return None
        if u < 0.5:
            return dense(r.choice([8, 24, 40, 72]))
        count = r.choice([1, 2, 3, 5, 8, 12])
        return experts(r.choice([8, 24, 40, 72]), count, r.randint(1, min(count, 4)), shared=r.choice([None, 8, 40]))

    layers = []
    for _ in range(r.randint(2, 6)):
        kind = r.choice(["attention", "latent", "recurrence"])
        if kind == "attention":
            kv = r.choice([1, 2, 3])
            dim = r.choice([8, 20, 32, 64])
            dims = r.choice([0] + [d for d in (2, 4, 8, 16, 32, dim) if d <= dim and d % 2 == 0])
            mixer = attention(kv * r.choice([1, 2, 4]), kv, dim, r.choice([4, 16, 32, 40]), rot_dims=dims,
                              base=r.choice([10.0, 1000.0, 1e6]), scale=r.choice([0.3, 1.0]))
        elif kind == "latent":
            scaling = r.choice([None, (r.choice([2.0, 8.0]), r.choice([16, 64, 2048]), r.choice([4.0, 32.0]), r.choice([0.5, 1.0]))])
            mixer = latent(r.choice([1, 2, 5]), r.choice([4, 16, 24]), r.choice([0, 2, 8, 16]), r.choice([4, 16, 40]),
                           r.choice([8, 20, 36, 64]), base=r.choice([10.0, 1000.0, 5e5]), scaling=scaling, scale=r.choice([0.2, 0.7]))
        else:
            mixer = recurrence(r.choice([1, 2, 3, 6]), r.choice([4, 10, 16, 48, 130]), r.choice([4, 16, 24, 72]))
        layers.append(layer(mixer, draw_mlp()))
    return dict(page_size=r.choice([4, 8, 16]), seed=seed,
                config=config(r.choice([64, 130, 300]), width, layers, taps=r.choice([1, 2, 3, 5]), scale=r.choice([0.5, 1.0, 3.0]),
                              logit_scale=r.choice([0.3, 1.0, 2.0]), eps=r.choice([1e-6, 1e-5])))


def _draw(name: str, shape: tuple, seed: int, sharp: bool) -> torch.Tensor:
    g = torch.Generator().manual_seed(seed)
    n = torch.randn(shape, generator=g)
    last = name.rsplit(".", 1)[-1]
    if last in ("norm1", "norm2", "norm"):
        t = 1.0 + 0.3 * n                       # plain weights around one
    elif last == "lower":
        t = torch.rand(shape, generator=g) * (0.98 if sharp else 0.9)      # lower bounds from none to nearly one
    elif name.endswith(".f.b"):
        t = n * (3.0 if sharp else 1.0)
    elif last == "f":
        t = n * (shape[-1] ** -0.5) * (4.0 if sharp else 1.5)
    elif last == "sink":
        t = n * (4.0 if sharp else 1.5)          # in some heads the sink outweighs the keys, in others it hardly counts
    elif last == "router":
        # scores that differ, and logits of a few units at most: beyond some 15 a sigmoid is 1.0 in float32 and two
        # experts tie that differ in exact arithmetic
        t = n * (shape[-1] ** -0.5) * (0.7 if sharp else 1.0)
    elif last in ("canon1", "canon2"):
        t = n * (0.6 if sharp else 0.3)
    elif name == "embed":
        t = n
    else:
        t = n * (shape[-1] ** -0.5)             # a projection keeps its input's size
    return t.to(torch.bfloat16)


def write_folder(name, folder: str) -> str:
    """A model folder for one of CONFIGS (or a dict of the same form): config.json and weights that make
    every part count."""
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
    return {rid: duvozen_plain.forward(toks, weights, raw) for rid, toks in requests.items()}


def rounding_noise(folder: str, requests: dict, dtype, exact: dict) -> dict:
    """How far rounding alone carries every row: the plain implementation in float32, or in float64 with every
    tensor a bfloat16 model holds rounded to bfloat16, against the exact rows."""
    raw, weights = read_folder(folder, torch.float64)
    noise = {}
    for rid, toks in requests.items():
        if dtype == torch.float32:
            noisy = duvozen_plain.forward(toks, {k: v.float() for k, v in weights.items()}, raw).double()
        else:
            noisy = duvozen_plain.forward(toks, weights, raw, to_bfloat16)
        d = noisy - exact[rid]
        noise[rid] = (d - d.mean(-1, keepdim=True)).pow(2).mean(-1).sqrt()
    return noise
