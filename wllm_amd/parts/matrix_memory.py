"""A recurrent mixer whose state is a matrix a head: linear attention in its recurrent form.

    [q | k | v | g | (z_i | z_f)] = W h                one stacked product
    q = q_scale * rot(q),  k = k_scale * rot(k)        float32 from here on (rot: the spec's position, or none)
    S_t = a_t S_(t-1) + b_t k_t v_t^T                  per head, S [head_dim, value_dim], float32
    o_t = S_t^T q_t / den_t
    out = W_o (o / rms_per_head(o) * w * act(g) * output_scale)

With `gating` "decay", a_t is the head's fixed decay and b_t = den_t = 1 (retention).  With "exponential",
the two gate projections give a log input gate and a log forget gate (both bent under a cap), a running
maximum m holds the exponentials in range, a normaliser n_t = a_t n_(t-1) + b_t k_t is carried beside S and
den_t = max(|n_t . q_t|, exp(-m_t)) + den_eps (the matrix memory of an mLSTM).  The normaliser is one more
column of the memory (a value that is always 1), so the recurrence's kernel carries it and leaves n . q beside
the columns' sums; the kernel that norms the heads divides by den first.  With "forget" there is no key
projection: a forget gate a channel, f = l + (1 - l) sigmoid(W_f h + b) with a learned lower bound l, decays the
rows of S and 1 - f stands in the key's place, S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T (the gating of HGRN2);
the gate's projection lies where the keys' would in the stacked product, and the recurrence's kernel takes f as
a decay a row.  Such a mixer may have no output gate, a silu on its queries, and a norm weight of value_dim
numbers that its heads share.

A request carries S (and n, m) from step to step in one float32 state row of the cache manager
([heads * head_dim * value_dim], then [heads * head_dim], then [heads]; zeroed at admission: all three
start at zero).  The kernels walk every segment's tokens in order from that row and leave it for the
next step, so a prompt may be cut anywhere, and a decoded token is a segment of one.  Everything the
kernels read of the step lies in device arrays, so a decode step can be captured in a graph.
"""
from __future__ import annotations

from typing import Optional

import torch

from wllm_amd.kernels import ops
from wllm_amd.parts.common import Product, load_matrix
from wllm_amd.parts.registry import build_position, register_mixer
from wllm_amd.parts.specs import MatrixMemorySpec
from wllm_amd.weights.checkpoint import ExpectedTensor


@register_mixer("matrix_memory")
class MatrixMemoryMixer:
    graph_capturable = True

    def __init__(self, spec: MatrixMemorySpec):
        for name in ("hidden_size", "num_heads", "head_dim", "value_dim"):
            if getattr(spec, name) <= 0:
                raise ValueError(f"{name} must be positive, got {getattr(spec, name)}")
        if spec.head_dim > 256:
            raise ValueError(f"head_dim {spec.head_dim}: the recurrence's kernel keeps at most 256 rows a head")
        if spec.gating not in ("decay", "exponential", "forget"):
            raise ValueError(f"gating {spec.gating!r}: 'decay', 'exponential' or 'forget'")
        if spec.gating == "forget" and (not spec.f_weight or spec.k_weight or spec.position.kind != "none"
                                        or spec.q_scale != 1.0 or spec.k_scale != 1.0):
            raise ValueError("forget gating: a forget projection, no key projection, no rotation and no scales")
        if spec.gating != "forget" and (not spec.k_weight or not spec.gate_weight or spec.q_activation != "none"
                                        or spec.lower_bound):
            raise ValueError(f"gating {spec.gating!r} has key and gate projections and plain queries")
        if spec.q_activation not in ops.QUERY_ACTIVATIONS:
            raise ValueError(f"q_activation {spec.q_activation!r}: one of {sorted(ops.QUERY_ACTIVATIONS)}")
        if spec.gating == "decay" and len(spec.decays) != spec.num_heads:
            raise ValueError(f"decays: one a head ({spec.num_heads}), got {len(spec.decays)}")
        if spec.gating == "exponential" and not (spec.i_weight and spec.f_weight):
            raise ValueError("exponential gating needs the two gate projections")
        if spec.gate_cap is not None and not spec.gate_cap > 0:
            raise ValueError(f"gate_cap must be positive or None, got {spec.gate_cap}")
        if spec.gate_weight and spec.gate_activation not in ("sigmoid", "silu"):
            raise ValueError(f"gate_activation {spec.gate_activation!r}: 'sigmoid' or 'silu'")
        if spec.gate_activation not in ops.GATE_KINDS:
            raise ValueError(f"gate_activation {spec.gate_activation!r}: one of {sorted(ops.GATE_KINDS)}")
        if spec.position.kind == "rope" and (spec.position.pairing != "half" or spec.position.rotary_dim > spec.head_dim):
            raise ValueError("the rotation pairs element j with j + rotary_dim / 2, within the head")
        self.spec = spec
        self.position = build_position(spec.position)
        self.exponential = spec.gating == "exponential"
        self.forget = spec.gating == "forget"
        self.qk_width = spec.num_heads * spec.head_dim
        self.v_width = spec.num_heads * spec.value_dim
        self.v_offset = 2 * self.qk_width
        self.g_offset = self.v_offset + self.v_width
        self.gates_offset = self.g_offset + (self.v_width if spec.gate_weight else 0)
        width = self.gates_offset + (2 * spec.num_heads if self.exponential else 0)
        self.in_width = -(-width // 8) * 8             # rows of the stacked weight, padded with zero rows
        self.memory_size = spec.num_heads * spec.head_dim * spec.value_dim
        self.w_in = self.t_in = self.w_o = self.t_o = None
        self.norm_w = self.i_bias = self.f_bias = self.decays = self.lower = None

    def expected_tensors(self) -> dict:
        s = self.spec
        out = {
            s.q_weight: ExpectedTensor((self.qk_width, s.hidden_size)),
            s.v_weight: ExpectedTensor((self.v_width, s.hidden_size)),
            s.o_weight: ExpectedTensor((s.hidden_size, self.v_width)),
        }
        if s.gate_weight:
            out[s.gate_weight] = ExpectedTensor((self.v_width, s.hidden_size))
        if self.forget:
            out[s.f_weight] = ExpectedTensor((self.qk_width, s.hidden_size))
            for name in (s.f_bias, s.lower_bound):
                if name:
                    out[name] = ExpectedTensor((self.qk_width,), role="vector")
        else:
            out[s.k_weight] = ExpectedTensor((self.qk_width, s.hidden_size))
        if s.norm_weight:
            out[s.norm_weight] = ExpectedTensor((self.v_width if s.norm_weight_per_head else s.value_dim,), role="vector",
                                                init="norm")
        if self.exponential:
            out[s.i_weight] = ExpectedTensor((s.num_heads, s.hidden_size))
            out[s.f_weight] = ExpectedTensor((s.num_heads, s.hidden_size))
            for name in (s.i_bias, s.f_bias):
                if name:
                    out[name] = ExpectedTensor((s.num_heads,), role="vector")
        return out

    def load(self, fetch) -> None:
        s = self.spec
        # (with forget gating the gate's projection lies where the keys' would)
        stacked = [fetch.matrix(name) for name in (s.q_weight, s.f_weight if self.forget else s.k_weight, s.v_weight)]
        if s.gate_weight:
            stacked.append(fetch.matrix(s.gate_weight))
        if self.exponential:
            stacked += [fetch.matrix(s.i_weight), fetch.matrix(s.f_weight)]
        w = torch.cat(stacked, dim=0)
        if w.shape[0] < self.in_width:
            w = torch.cat([w, torch.zeros(self.in_width - w.shape[0], w.shape[1], dtype=w.dtype, device=w.device)], dim=0)
        self.w_in, self.t_in = load_matrix(fetch, w)
        self.w_o, self.t_o = load_matrix(fetch, fetch.matrix(s.o_weight))
        # everything that enters the recurrence is kept in float32
        if s.norm_weight:
            norm_w = fetch.vector(s.norm_weight)
            self.norm_w = fetch.to_device(norm_w if s.norm_weight_per_head else norm_w.repeat(s.num_heads))
        if self.forget:
            self.f_bias = fetch.to_device(fetch.vector(s.f_bias)) if s.f_bias else None
            self.lower = fetch.to_device(fetch.vector(s.lower_bound)) if s.lower_bound else None
        elif self.exponential:
            self.i_bias = fetch.to_device(fetch.vector(s.i_bias)) if s.i_bias else None
            self.f_bias = fetch.to_device(fetch.vector(s.f_bias)) if s.f_bias else None
        else:
            self.decays = torch.tensor([float(d) for d in s.decays], dtype=torch.float32, device=fetch.device)
        self.position.prepare(fetch.device)

    def cache_need(self):
        return None

    def state_shape(self):
        s = self.spec
        return (self.memory_size + ((s.num_heads * s.head_dim + s.num_heads) if self.exponential else 0),)

    def flops(self, tokens: int, keys: float = 0.0) -> float:
        s = self.spec
        return 2.0 * tokens * (s.hidden_size * (self.in_width + self.v_width) + 2 * self.memory_size)

    def forward(self, ctx, entry: int, h: torch.Tensor, product_input: Optional[torch.Tensor] = None):
        s = self.spec
        n = h.shape[0]
        row = ctx.buffer("memory_in", (n, self.in_width), h.dtype)
        ops.linear(h, self.w_in, row, self.t_in)
        state = ctx.state(entry)
        steps = nq = None
        if self.forget:
            qk = ctx.buffer("memory_qkf", (3, n, self.qk_width), torch.float32)
            ops.memory_forget_inputs(row, self.f_bias, self.lower, qk, width=self.qk_width, q_activation=s.q_activation)
        else:
            qk = ctx.buffer("memory_qk", (2, n, self.qk_width), torch.float32)
            ops.memory_inputs(row, ctx.positions, self.position.inv_freq, qk, heads=s.num_heads, head_dim=s.head_dim,
                              q_scale=s.q_scale, k_scale=s.k_scale)
        if self.exponential:
            # the normaliser lies behind the memory in the request's row, the running maxima behind it
            n_offset = self.memory_size
            steps = ctx.buffer("memory_steps", (3, n, s.num_heads), torch.float32)
            nq = ctx.buffer("memory_nq", (n, s.num_heads), torch.float32)
            ops.memory_gates(row[:, self.gates_offset:self.gates_offset + 2 * s.num_heads], self.i_bias, self.f_bias, state,
                             n_offset + self.qk_width, ctx.seg_q_start, ctx.seg_q_len, ctx.state_slots, steps,
                             heads=s.num_heads, cap=s.gate_cap)
        y = ctx.buffer("memory_y", (n, self.v_width), torch.float32)
        ops.memory_scan(qk, row[:, self.v_offset:self.v_offset + self.v_width], steps, self.decays, state,
                        ctx.seg_q_start, ctx.seg_q_len, ctx.state_slots, y, heads=s.num_heads, head_dim=s.head_dim,
                        value_dim=s.value_dim, nq=nq, n_offset=self.memory_size if self.exponential else 0,
                        row_decays=self.forget)
        out = product_input if product_input is not None else ctx.buffer("memory_out", (n, self.v_width), h.dtype)
        gate = row[:, self.g_offset:self.g_offset + self.v_width] if s.gate_weight else None
        ops.head_norm_gate(y, gate, self.norm_w, out, heads=s.num_heads,
                           eps=s.norm_eps, activation=s.gate_activation if s.gate_weight else "none", scale=s.output_scale, nq=nq,
                           floor=steps[2] if self.exponential else None, den_eps=s.den_eps if self.exponential else 0.0)
        return Product("mixer_out", out, self.w_o, self.t_o)
