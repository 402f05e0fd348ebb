"""Duvozen, plainly: whole sequences, no cache, no batch, one function a mechanism.

A decoder whose layers put a norm behind each sublayer and none before it,

    x += layer_norm(mixer(x + conv1(x)));   x += layer_norm(ff(x + conv2(x)))        (ff may be absent)

where conv is a short causal convolution over time on each channel of the stream (zeros before the
sequence's start).  The mixer is, layer by layer,

  "hgrn2": a gated linear recurrence a head whose forget gate (bounded below by a learned number a channel)
      also decides what is written: S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T, o_t = S_t^T silu(q_t), with an
      RMS norm over each head's result;
  "latent_attention": causal softmax attention whose keys and values are expanded from one compressed vector
      a token, plus a short rotated part of the key that all heads share (interleaved pairs, frequencies
      interpolated between the original ones and ones divided by a factor, sine and cosine scaled);
  "attention": causal softmax attention with grouped key/value heads, an RMS norm with a weight over each
      query and key head before the rotation (half-split pairs), a learned term a head in the softmax's
      denominator, and an elementwise sigmoid gate on the result.

The feed-forward is gated (gelu in its tanh form), or a mixture of silu-gated experts chosen by the largest
sigmoid scores, whose score multiplies the expert's input, plus an expert every token uses.  The logits are
the head's product behind the model's layer norm, times a factor.

Every function takes and returns tensors of one dtype (float64 in the tests' reference runs); `rounding`
is a function applied wherever a bfloat16 model would hold a tensor in bfloat16, and the identity
otherwise.  Nothing here is shared with the engine.
"""
from __future__ import annotations

import math

import torch


def same(x):
    return x


def layer_norm(x, weight, eps):
    """(x - mean) / sqrt(mean of squared deviations + eps) * weight over the last axis, no bias."""
    mean = x.mean(dim=-1, keepdim=True)
    dev = x - mean
    return dev / torch.sqrt((dev * dev).mean(dim=-1, keepdim=True) + eps) * weight


def rms_norm(x, weight, eps):
    """x / sqrt(mean(x^2) + eps) * weight over the last axis."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * weight


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def input_convolution(h, taps_weight):
    """h [T, C], taps_weight [C, taps]: h_t + sum_j w[:, j] * h_(t - taps + 1 + j), zeros before the start."""
    T, C = h.shape
    taps = taps_weight.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=h.dtype), h], dim=0)
    out = h.clone()
    for j in range(taps):
        out = out + padded[j:j + T] * taps_weight[:, j]
    return out


def plain_frequencies(dims, base):
    i = torch.arange(dims // 2, dtype=torch.float64)
    return float(base) ** (-2.0 * i / dims)


def interpolated_frequencies(dims, base, scaling):
    """Frequencies between the plain ones (fast pairs) and the plain ones divided by `factor` (slow pairs),
    with a linear ramp over the pair index between the pairs that make `fast` and `slow` turns within
    `original` positions; and the factor both sine and cosine are multiplied by."""
    f = plain_frequencies(dims, base)
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def pair_of(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(pair_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(pair_of(float(scaling["slow"]))), dims - 1)
    i = torch.arange(dims // 2, dtype=torch.float64)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate(x, positions, dims, freq, pairing, magnitude=1.0):
    """x [T, heads, d]: the first `dims` elements of every head turn by position * freq[i]; pair i is elements
    (i, i + dims/2) ("half") or (2i, 2i + 1) ("interleaved"); sine and cosine times `magnitude`."""
    angle = positions.to(x.dtype)[:, None] * freq.to(x.dtype)[None, :]
    cos, sin = (torch.cos(angle) * magnitude)[:, None, :], (torch.sin(angle) * magnitude)[:, None, :]
    turned, rest = x[..., :dims], x[..., dims:]
    if pairing == "half":
        u, v = turned[..., :dims // 2], turned[..., dims // 2:]
        out = torch.cat([u * cos - v * sin, v * cos + u * sin], dim=-1)
    else:
        u, v = turned[..., 0::2], turned[..., 1::2]
        out = torch.stack([u * cos - v * sin, v * cos + u * sin], dim=-1).flatten(-2)
    return torch.cat([out, rest], dim=-1)


def causal_softmax(scores, sink=None):
    """scores [H, T, T]; the softmax over the keys j <= i; `sink` [H]: exp(sink) joins the denominator."""
    T = scores.shape[-1]
    mask = torch.tril(torch.ones(T, T, dtype=torch.bool))
    scores = scores.masked_fill(~mask, float("-inf"))
    m = scores.max(dim=-1, keepdim=True).values
    if sink is not None:
        m = torch.maximum(m, sink[:, None, None])
    e = torch.exp(scores - m)
    den = e.sum(dim=-1, keepdim=True)
    if sink is not None:
        den = den + torch.exp(sink[:, None, None] - m)
    return e / den


def forget_gate_recurrence(h, w, p, c, eps, rounding=same):
    """The "hgrn2" mixer.  h [T, width]."""
    T = h.shape[0]
    H, d, dv = c["heads"], c["dim"], c["vdim"]
    q = rounding(silu(rounding(h @ w[p + "q"].T))).view(T, H, d)
    v = rounding(h @ w[p + "v"].T).view(T, H, dv)
    lower = w[p + "lower"]
    f = lower + (1.0 - lower) * torch.sigmoid(rounding(h @ w[p + "f"].T) + w[p + "f.b"])
    f = f.view(T, H, d)
    S = torch.zeros(H, d, dv, dtype=h.dtype)
    out = []
    for t in range(T):
        S = f[t][:, :, None] * S + (1.0 - f[t])[:, :, None] * v[t][:, None, :]
        out.append(torch.einsum("hdv,hd->hv", S, q[t]))
    o = rms_norm(torch.stack(out), w[p + "norm"], eps)                 # [T, H, dv], the weight shared by heads
    return rounding(o.reshape(T, H * dv)) @ w[p + "o"].T


def latent_attention(h, w, p, c, eps, rounding=same):
    """The "latent_attention" mixer."""
    T = h.shape[0]
    H, d, dr, dv, rank = c["heads"], c["dim"], c.get("rot_dim", 0), c["vdim"], c["kv_rank"]
    q = rounding(h @ w[p + "q"].T).view(T, H, d + dr)
    down = rounding(h @ w[p + "dkv"].T)
    latent = rounding(rms_norm(down[:, :rank], w[p + "dkv.norm"], eps))
    k_turned = down[:, rank:].view(T, 1, dr)
    k_plain = rounding(latent @ w[p + "uk"].T).view(T, H, d)
    v = rounding(latent @ w[p + "uv"].T).view(T, H, dv)
    scores = torch.einsum("thd,shd->hts", q[..., :d], k_plain)
    if dr:          # a model may have no turned part
        rot = c["rot"]
        if rot.get("scaling"):
            freq, magnitude = interpolated_frequencies(rot["dims"], rot["base"], rot["scaling"])
        else:
            freq, magnitude = plain_frequencies(rot["dims"], rot["base"]), 1.0
        pos = torch.arange(T)
        q_turned = rounding(rotate(q[..., d:], pos, rot["dims"], freq, "interleaved", magnitude))
        k_turned = rounding(rotate(k_turned, pos, rot["dims"], freq, "interleaved", magnitude))
        scores = scores + torch.einsum("thd,sd->hts", q_turned, k_turned[:, 0])
    scores = scores * c["scale"]
    weights = causal_softmax(scores)
    o = torch.einsum("hts,shd->thd", weights, v)
    return rounding(o.reshape(T, H * dv)) @ w[p + "o"].T


def sink_attention(h, w, p, c, eps, rounding=same):
    """The "attention" mixer."""
    T = h.shape[0]
    H, G, d, dv = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    q = rounding(h @ w[p + "q"].T).view(T, H, d)
    k = rounding(h @ w[p + "k"].T).view(T, G, d)
    v = rounding(h @ w[p + "v"].T).view(T, G, dv)
    gate = rounding(h @ w[p + "g"].T)
    q = rms_norm(q, w[p + "q.norm"], eps)
    k = rms_norm(k, w[p + "k.norm"], eps)
    rot = c.get("rot")
    if rot is not None:
        freq, pos = plain_frequencies(rot["dims"], rot["base"]), torch.arange(T)
        q, k = rotate(q, pos, rot["dims"], freq, "half"), rotate(k, pos, rot["dims"], freq, "half")
    q, k = rounding(q), rounding(k)
    k = k.repeat_interleave(H // G, dim=1)
    v = v.repeat_interleave(H // G, dim=1)
    scores = torch.einsum("thd,shd->hts", q, k) * c["scale"]
    weights = causal_softmax(scores, w[p + "sink"])
    o = torch.einsum("hts,shd->thd", weights, v).reshape(T, H * dv)
    return rounding(o * torch.sigmoid(gate)) @ w[p + "o"].T


def gated_feed_forward(h, w, p, act, rounding=same):
    return rounding(act(rounding(h @ w[p + "gate"].T)) * rounding(h @ w[p + "up"].T)) @ w[p + "down"].T


def expert_feed_forward(h, w, p, c, rounding=same):
    """Experts chosen by the largest sigmoid scores; the score multiplies the chosen expert's input; one more
    expert runs for every token."""
    T = h.shape[0]
    scores = torch.sigmoid(h @ w[p + "router"].T)
    top = torch.topk(scores, c["router"]["top"], dim=-1)
    out = torch.zeros(T, w[p + "e0.down"].shape[0], dtype=h.dtype)
    for t in range(T):
        for s, e in zip(top.values[t], top.indices[t]):
            out[t] += gated_feed_forward(rounding(s * h[t:t + 1]), w, f"{p}e{int(e)}.", silu, rounding)[0]
    if c.get("shared") is not None:
        out = out + gated_feed_forward(h, w, p + "shared.", silu, rounding)
    return out


MIXERS = {"hgrn2": forget_gate_recurrence, "latent_attention": latent_attention, "attention": sink_attention}


def forward(tokens, w, cfg, rounding=same, keep_layers=False):
    """tokens: a list of ids; w: {name: tensor}; cfg: config.json as a dict.  Returns logits [T, vocab] (and the
    stream after every layer)."""
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.as_tensor(tokens)] * cfg["embedding"]["scale"]
    after = []
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = rounding(input_convolution(x, w[p + "canon1"]))
        x = x + layer_norm(MIXERS[layer["type"]](h, w, p + "mix.", layer["mixer"], eps, rounding), w[p + "norm1"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            h = rounding(input_convolution(x, w[p + "canon2"]))
            if mlp["kind"] == "dense":
                y = gated_feed_forward(h, w, p + "mlp.", gelu_tanh, rounding)
            else:
                y = expert_feed_forward(h, w, p + "mlp.", mlp, rounding)
            x = x + layer_norm(y, w[p + "norm2"], eps)
        after.append(x)
    logits = rounding(layer_norm(x, w["final.norm"], eps)) @ w["head"].T * cfg["logit_scale"]
    return (logits, torch.stack(after)) if keep_layers else logits
