"""Lefisun, plainly: whole sequences, no cache, no batch, one function a mechanism.

A decoder of pre-norm layers, x += mixer(rms(x) w1); x += moe(rms(x) w2) (a layer may have no
feed-forward), whose mixer is, layer by layer, either

  "parallel": two mixers side by side on the same input, a_l * left + a_r * right, where left is softmax
      attention inside chunks of the sequence (grouped heads, biases on q, k and v, an RMS norm with a
      weight over the whole query and the whole key projection, rotation of the first elements of
      every head in the half-split pairing with linearly scaled positions, a denominator that holds
      one more 1), and right is the matrix memory of an mLSTM (capped exponential gates with a running
      maximum, a normaliser, a unit norm per head, a sigmoid output gate); or

  "retention": linear attention with a fixed decay a head, rotated queries and keys, a unit norm per
      head and a silu gate.

The feed-forward is a mixture of experts whose router scores are a softmax over all experts, limited
to the experts of the best groups, the chosen scores renormalised.  The head is the embedding table
(without the embedding's factor) behind the model's norm.

Every function takes and returns tensors of one dtype (float64 in the tests' reference runs); `rounding`
is a function applied wherever a bfloat16 model would hold a tensor in bfloat16 (projections and their
activations), and the identity otherwise.  Nothing here is shared with the engine.
"""
from __future__ import annotations

import math

import torch


def same(x):
    return x


def rms_norm(x, weight, eps):
    """x / sqrt(mean(x^2) + eps) * weight over the last axis; weight None: no weight."""
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def rotate_half_split(x, positions, dims, base, factor=1.0):
    """x [T, heads, d]: the first `dims` elements of every head turn, element i paired with i + dims/2,
    by the angle position * base^(-2i/dims) / factor; the rest pass."""
    half = dims // 2
    i = torch.arange(half, dtype=torch.float64)
    freq = (float(base) ** (-2.0 * i / dims) / factor).to(x.dtype)
    angle = positions.to(x.dtype)[:, None] * freq[None, :]          # [T, half]
    cos, sin = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    u, v, rest = x[..., :half], x[..., half:dims], x[..., dims:]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, rest], dim=-1)


def chunk_mask(length, size):
    """[T, T] True where query i may see key j: j <= i and both in the same chunk of `size` positions."""
    i = torch.arange(length)[:, None]
    j = torch.arange(length)[None, :]
    return (j <= i) & ((i // size) == (j // size))


def softmax_plus_one(scores, mask):
    """p_j = exp(s_j) / (1 + sum over the seen keys exp(s_j)): a sink of score 0 that has no value."""
    scores = scores.masked_fill(~mask, float("-inf"))
    m = torch.clamp(scores.max(dim=-1, keepdim=True).values, min=0.0)
    e = torch.exp(scores - m)
    return e / (torch.exp(-m) + e.sum(dim=-1, keepdim=True))


def chunked_attention(h, w, p, c, eps, rounding=same):
    """The left mixer.  h [T, width]; w: tensors by their short names; c: the mixer's sizes."""
    T = h.shape[0]
    H, G, d, dv = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    q = rounding(h @ w[p + "q"].T + w[p + "q.b"])
    k = rounding(h @ w[p + "k"].T + w[p + "k.b"])
    v = rounding(h @ w[p + "v"].T + w[p + "v.b"])
    q = rms_norm(q, w[p + "q.norm"], eps).view(T, H, d)
    k = rms_norm(k, w[p + "k.norm"], eps).view(T, G, d)
    v = v.view(T, G, dv)
    pos = torch.arange(T)
    rot = c["rot"]
    factor = (rot.get("scaling") or {}).get("factor", 1.0)
    q = rounding(rotate_half_split(q, pos, rot["dims"], rot["base"], factor))
    k = rounding(rotate_half_split(k, pos, rot["dims"], rot["base"], factor))
    mask = chunk_mask(T, c["mask"]["size"]) if c.get("mask") else chunk_mask(T, T)
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for head in range(H):
        g = head // (H // G)
        scores = (q[:, head] @ k[:, g].T) * c["scale"]
        out[:, head] = softmax_plus_one(scores, mask) @ v[:, g]
    return rounding(rounding(out.reshape(T, H * dv)) @ w[p + "o"].T)


def capped(z, cap):
    return cap * torch.tanh(z / cap)


def matrix_memory(h, w, p, c, eps, rounding=same):
    """The right mixer: the mLSTM's matrix memory, token by token."""
    T = h.shape[0]
    H, d, dv, cap = c["heads"], c["dim"], c["vdim"], c["gate_cap"]
    q = rounding(h @ w[p + "q"].T).view(T, H, d) * d ** -0.5
    k = rounding(h @ w[p + "k"].T).view(T, H, d)
    v = rounding(h @ w[p + "v"].T).view(T, H, dv)
    log_i = capped(rounding(h @ w[p + "i"].T) + w[p + "i.b"], cap)                                  # [T, H]
    log_f = torch.nn.functional.logsigmoid(capped(rounding(h @ w[p + "f"].T) + w[p + "f.b"], cap))
    S = torch.zeros(H, d, dv, dtype=h.dtype)
    n = torch.zeros(H, d, dtype=h.dtype)
    m = torch.zeros(H, dtype=h.dtype)
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for t in range(T):
        m_new = torch.maximum(log_f[t] + m, log_i[t])
        keep, take = torch.exp(log_f[t] + m - m_new), torch.exp(log_i[t] - m_new)
        S = keep[:, None, None] * S + take[:, None, None] * (k[t][:, :, None] * v[t][:, None, :])
        n = keep[:, None] * n + take[:, None] * k[t]
        m = m_new
        num = torch.einsum("hdv,hd->hv", S, q[t])
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
        out[t] = num / den[:, None]
    o = rms_norm(out, None, eps).reshape(T, H * dv) * w[p + "norm"]
    gate = torch.sigmoid(rounding(h @ w[p + "g"].T))
    return rounding(rounding(o * gate) @ w[p + "o"].T)


def retention(h, w, p, c, eps, rounding=same):
    T = h.shape[0]
    H, d, dv = c["heads"], c["dim"], c["vdim"]
    pos = torch.arange(T)
    rot = c["rot"]
    q = rounding(h @ w[p + "q"].T).view(T, H, d)
    k = rounding(h @ w[p + "k"].T).view(T, H, d)
    v = rounding(h @ w[p + "v"].T).view(T, H, dv)
    factor = (rot.get("scaling") or {}).get("factor", 1.0)
    q = rotate_half_split(q, pos, rot["dims"], rot["base"], factor)
    k = rotate_half_split(k, pos, rot["dims"], rot["base"], factor) * d ** -0.5
    decay = torch.tensor(c["decay"], dtype=h.dtype)
    S = torch.zeros(H, d, dv, dtype=h.dtype)
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for t in range(T):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", S, q[t])
    o = rms_norm(out, None, eps).reshape(T, H * dv)
    g = rounding(h @ w[p + "g"].T)
    return rounding(rounding(o * (g * torch.sigmoid(g))) @ w[p + "o"].T)


def route(h, router, experts, top, groups, keep):
    """The chosen experts [T, top] and their weights: softmax over all experts, only experts of the
    `keep` groups (of `groups` equal groups of neighbours) with the largest best score may be chosen,
    the chosen scores divided by their sum."""
    s = torch.softmax(h @ router.T, dim=-1)                                 # [T, E]
    T = s.shape[0]
    per = experts // groups
    best = s.view(T, groups, per).max(dim=-1).values
    kept = torch.zeros(T, groups, dtype=torch.bool)
    kept.scatter_(1, best.topk(keep, dim=-1).indices, True)
    allowed = kept[:, :, None].expand(T, groups, per).reshape(T, experts)
    chosen = s.masked_fill(~allowed, -1.0).topk(top, dim=-1).indices
    weights = s.gather(1, chosen)
    return chosen, weights / (weights.sum(dim=-1, keepdim=True) + 1e-20)


def mixture_of_experts(h, w, p, c, rounding=same):
    r = c["router"]
    groups = r.get("groups") or {"count": 1, "keep": 1}
    chosen, weights = route(h, w[p + "router"], r["experts"], r["top"], groups["count"], groups["keep"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(chosen[t].tolist(), weights[t]):
            q = f"{p}e{e}."
            gate = rounding(h[t] @ w[q + "gate"].T)
            act = rounding(gate * torch.sigmoid(gate) * rounding(h[t] @ w[q + "up"].T))
            out[t] += a * rounding(act @ w[q + "down"].T)
    return rounding(out)


def mixer(kind, h, w, p, c, eps, rounding=same):
    if kind == "retention":
        return retention(h, w, p, c, eps, rounding)
    left = chunked_attention(h, w, p + "left.", c["left"], eps, rounding)
    right = matrix_memory(h, w, p + "right.", c["right"], eps, rounding)
    return c["left_scale"] * left + c["right_scale"] * right


def forward(config, w, tokens, dtype=torch.float64, rounding=same, layers_out=None):
    """Logits [T, vocab] of one sequence.  w: {tensor name: tensor}; `layers_out`: a list that takes the
    stream after every layer."""
    w = {k: v.to(dtype) for k, v in w.items()}
    eps = config["norm"]["eps"]
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)] * config["embedding"]["scale"]
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}."
        h = rounding(rms_norm(x, w[p + "norm1"], eps))
        x = x + mixer(layer["type"], h, w, p + "mix.", layer["mixer"], eps, rounding)
        if layer.get("mlp") is not None:
            h = rounding(rms_norm(x, w[p + "norm2"], eps))
            x = x + mixture_of_experts(h, w, p + "mlp.", layer["mlp"], rounding)
        if layers_out is not None:
            layers_out.append(x.clone())
    return rounding(rms_norm(x, w["final.norm"], eps)) @ w["embed"].T


def to_bfloat16(x):
    return x.to(torch.bfloat16).to(x.dtype)


def greedy(config, w, prompt, new_tokens):
    tokens = list(prompt)
    for _ in range(new_tokens):
        tokens.append(int(forward(config, w, tokens)[-1].argmax()))
    return tokens[len(prompt):]
