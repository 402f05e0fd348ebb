"""Latent attention: keys and values are expanded from one compressed vector a token, and only that
vector is cached.

    c_q = rms(W_dq h) * w;  q = W_uq c_q            queries through a latent of their own
    c   = rms(W_dkv h) * w                           the cached vector, kv_rank numbers a token
    k_h = W_uk,h c;  v_h = W_uv,h c                  per head
    score = (q_h . k_h) * scale;  causal;  the softmax's denominator may hold exp(sink_h) once more
    out   = W_o ([heads] * sigmoid(W_g h))

Since q_h . (W_uk,h c) = (W_uk,h^T q_h) . c, the scores are taken against c itself: every query head is
carried into the latent space (a product head by head, `ops.head_linear`), and all heads attend over
one shared key/value head whose keys and values are both c (`ops.paged_attention` with one key/value
head, the cache written by `ops.head_prepare` with `values_are_keys`).  The result per head, a
weighted sum of c, is expanded by W_uv,h afterwards.  So a token costs kv_rank numbers of cache, and a
decode step reads them once for all heads.  kv_rank is padded to a multiple of four with zeros.

Two options.  Queries straight from the input (`q_weight`: q = W_q h, no latent of their own).  And a turned
part (`rope_dim` = r): a query head is [head_dim | r], W_dkv gives kv_rank + r numbers of which the last r, not
normed, are a key part that all heads share; the r elements of every query head and the key part turn by the
position, and the score is (q . k + q_r . k_r) * scale.  The one key/value head then is [k_r | c]: a query head
becomes [q_r | W_uk,h^T q] by one product head by head whose matrix holds an identity for the r elements, the
rotation kernel turns the first r elements of the query heads and of the key head, the cached values are the key
head as it was before the turn, and W_uv,h has zero columns where the turned part lies.  With a turned part the
head is padded to a multiple of 32 where that is at most the kernels' largest head, so that the matrix cores
take it.
"""
from __future__ import annotations

from typing import Optional

import torch

from wllm_amd.cache.manager import CacheNeed
from wllm_amd.kernels import ops
from wllm_amd.parts.common import Product, load_matrix
from wllm_amd.parts.registry import build_position, register_mixer
from wllm_amd.parts.specs import LatentAttentionSpec
from wllm_amd.weights.checkpoint import ExpectedTensor


@register_mixer("latent_attention")
class LatentAttention:
    graph_capturable = True

    def __init__(self, spec: LatentAttentionSpec):
        for name in ("hidden_size", "num_heads", "head_dim", "value_dim", "kv_rank") + (() if spec.q_weight else ("q_rank",)):
            if getattr(spec, name) <= 0:
                raise ValueError(f"{name} must be positive, got {getattr(spec, name)}")
        if spec.q_weight and (spec.q_rank or spec.dq_weight or spec.uq_weight or spec.dq_norm_weight):
            raise ValueError("queries straight from the input have no latent of their own")
        if spec.rope_dim < 0 or (spec.rope_dim > 0) != (spec.position.kind != "none"):
            raise ValueError("a turned part and its position encoding go together")
        if spec.rope_dim and spec.position.rotary_dim != spec.rope_dim:
            raise ValueError(f"the turned part ({spec.rope_dim}) turns whole: rotary_dim {spec.position.rotary_dim}")
        self.turned = spec.rope_dim
        # the one key/value head: the turned part, then the cached vector, padded
        self.rank = -(-(self.turned + spec.kv_rank) // ops.HEAD_DIM_STEP) * ops.HEAD_DIM_STEP
        if self.turned and -(-self.rank // 32) * 32 <= ops.MAX_HEAD_DIM:
            self.rank = -(-self.rank // 32) * 32
        if self.rank > ops.MAX_HEAD_DIM:
            raise ValueError(f"kv_rank {spec.kv_rank} (+ {self.turned}): the attention kernels take heads up to "
                             f"{ops.MAX_HEAD_DIM}, and the cached vector is the one key/value head")
        self.spec = spec
        self.position = build_position(spec.position)
        self.q_in = spec.head_dim + self.turned         # a query head as projected
        self.q_width = spec.num_heads * self.q_in if spec.q_weight else spec.q_rank      # the queries' columns of the stacked product
        self.w_down = self.t_down = None        # [W_dq; W_dkv; W_g] stacked
        self.w_uq = self.t_uq = None
        self.w_qk = None                        # [heads, rank, dim]: W_uk,h^T, a query head into the latent space
        self.w_uv = None                        # [heads, vdim, rank]
        self.w_dq_norm = self.w_dkv_norm = self.sinks = None
        self.w_o = self.t_o = None

    def expected_tensors(self) -> dict:
        s = self.spec
        out = {s.q_weight: ExpectedTensor((self.q_width, s.hidden_size))} if s.q_weight else {
            s.dq_weight: ExpectedTensor((s.q_rank, s.hidden_size)),
            s.dq_norm_weight: ExpectedTensor((s.q_rank,), role="vector", init="norm"),
            s.uq_weight: ExpectedTensor((s.num_heads * self.q_in, s.q_rank)),
        }
        out |= {
            s.dkv_weight: ExpectedTensor((s.kv_rank + self.turned, s.hidden_size)),
            s.dkv_norm_weight: ExpectedTensor((s.kv_rank,), role="vector", init="norm"),
            s.uk_weight: ExpectedTensor((s.num_heads * s.head_dim, s.kv_rank)),
            s.uv_weight: ExpectedTensor((s.num_heads * s.value_dim, s.kv_rank)),
            s.o_weight: ExpectedTensor((s.hidden_size, s.num_heads * s.value_dim)),
        }
        if s.sink_weight:
            out[s.sink_weight] = ExpectedTensor((s.num_heads,), role="vector", init="norm")
        if s.gate_weight:
            out[s.gate_weight] = ExpectedTensor((s.num_heads * s.value_dim, s.hidden_size))
        return out

    def load(self, fetch) -> None:
        s = self.spec
        stacked = [fetch.matrix(s.q_weight if s.q_weight else s.dq_weight), fetch.matrix(s.dkv_weight)]
        if s.gate_weight:
            stacked.append(fetch.matrix(s.gate_weight))
        w = torch.cat(stacked, dim=0)
        if w.shape[0] % 8:       # the kernels read rows that begin at multiples of 16 bytes
            w = torch.cat([w, torch.zeros(8 - w.shape[0] % 8, w.shape[1], dtype=w.dtype, device=w.device)], dim=0)
        self.w_down, self.t_down = load_matrix(fetch, w)
        if not s.q_weight:
            self.w_uq, self.t_uq = load_matrix(fetch, fetch.matrix(s.uq_weight))
        r, heads = self.turned, s.num_heads
        uk = fetch.matrix(s.uk_weight).view(heads, s.head_dim, s.kv_rank)
        uv = fetch.matrix(s.uv_weight).view(heads, s.value_dim, s.kv_rank)
        # a query head [head_dim | r] into the key head's space [r | kv_rank | padding]: W_uk,h^T for the first
        # part, an identity for the turned one; and the way back for the values, which have nothing where the
        # turned part and the padding lie
        w_qk = torch.zeros(heads, self.rank, self.q_in, dtype=uk.dtype, device=uk.device)
        w_qk[:, r:r + s.kv_rank, :s.head_dim] = uk.transpose(1, 2)
        if r:
            w_qk[:, :r, s.head_dim:] = torch.eye(r, dtype=uk.dtype, device=uk.device)
        w_uv = torch.zeros(heads, s.value_dim, self.rank, dtype=uv.dtype, device=uv.device)
        w_uv[:, :, r:r + s.kv_rank] = uv
        self.w_qk = fetch.to_device(w_qk.contiguous())
        self.w_uv = fetch.to_device(w_uv.contiguous())
        if not s.q_weight:
            self.w_dq_norm = fetch.to_device(fetch.vector(s.dq_norm_weight))
        self.position.prepare(fetch.device)
        self.w_dkv_norm = fetch.to_device(fetch.vector(s.dkv_norm_weight))
        if s.sink_weight:
            self.sinks = fetch.to_device(fetch.vector(s.sink_weight))
        self.w_o, self.t_o = load_matrix(fetch, fetch.matrix(s.o_weight))

    def cache_need(self) -> Optional[CacheNeed]:
        return CacheNeed(1, self.rank, None)

    def state_shape(self):
        return None

    def flops(self, tokens: int, keys: float) -> float:
        s = self.spec
        products = s.hidden_size * (self.w_down.shape[0] + s.num_heads * s.value_dim) + s.q_rank * s.num_heads * self.q_in \
            + s.num_heads * self.rank * (self.q_in + s.value_dim)
        return 2.0 * tokens * products + 4.0 * s.num_heads * self.rank * keys

    def _work_items(self, ctx, page_size: int):
        s = self.spec
        shape = dict(num_heads=s.num_heads, num_kv_heads=1, head_dim=self.rank, page_size=page_size, window=0)

        def build(c):
            if c.captured:
                return ops.static_attention_plan(c.num_segments, max_context=c.capture_max_context,
                                                 max_total_keys=c.capture_max_tokens, dtype=c.dtype, device=c.device, **shape)
            return ops.plan_paged_attention(c.host_q_len, c.host_ctx_len, dtype=c.dtype, device=c.device, **shape)

        return ctx.plan(("attention",) + tuple(shape.values()), build, lambda plan, c: plan.update(c.host_q_len, c.host_ctx_len))

    def forward(self, ctx, entry: int, h: torch.Tensor, product_input: Optional[torch.Tensor] = None):
        s = self.spec
        n, heads, rank = h.shape[0], s.num_heads, self.rank
        down = ctx.buffer("latent_down", (n, self.w_down.shape[0]), h.dtype)
        ops.linear(h, self.w_down, down, self.t_down)
        # the row the attention kernels read: the query heads in the key head's space, then the one key head
        # [turned part | cached vector | padding]
        row = ctx.buffer("latent_row", (n, (heads + 1) * rank), h.dtype)
        r, kv0 = self.turned, self.q_width
        latent = (down[:, kv0:kv0 + s.kv_rank], self.w_dkv_norm, s.kv_rank, row[:, heads * rank + r:])
        if s.q_weight:
            q = down[:, :self.q_width]
            ops.band_norm([latent], s.norm_eps)
        else:
            cq = ctx.buffer("latent_cq", (n, s.q_rank), h.dtype)
            ops.band_norm([(down[:, :s.q_rank], self.w_dq_norm, s.q_rank, cq), latent], s.norm_eps)
            q = ctx.buffer("latent_q", (n, heads * self.q_in), h.dtype)
            ops.linear(cq, self.w_uq, q, self.t_uq)
        if r:
            ops.copy_columns(down[:, kv0 + s.kv_rank:kv0 + s.kv_rank + r], row[:, heads * rank:heads * rank + r])
        ops.head_linear(q, self.w_qk, row[:, :heads * rank])
        pages = ctx.pages(entry)
        slots, storage = (pages.slots, pages.storage) if pages.writes else (None, None)
        ops.head_prepare(row, None, ctx.positions, self.position.inv_freq, slots, storage, num_heads=heads, num_kv_heads=1,
                         head_dim=rank, page_size=pages.page_size, values_are_keys=True,
                         interleaved=getattr(self.position, "interleaved", False),
                         rot_scale=getattr(self.position, "magnitude", 1.0))
        mixed = ctx.buffer("latent_mixed", (n, heads * rank), h.dtype)
        ops.paged_attention(
            row, pages.storage, pages.block_tables, ctx.token_segment, ctx.seg_q_start, ctx.seg_q_len, ctx.seg_ctx_len,
            mixed, num_heads=heads, num_kv_heads=1, head_dim=rank, page_size=pages.page_size, scale=s.scale,
            max_q_len=ctx.max_q_len, max_ctx_len=ctx.max_ctx_len, plan=self._work_items(ctx, pages.page_size),
            sinks=self.sinks, exact_weights=s.weights_in_float32)
        out = ctx.buffer("latent_out", (n, heads * s.value_dim), h.dtype)
        ops.head_linear(mixed, self.w_uv, out)
        if s.gate_weight:
            target = product_input if product_input is not None else out
            g0 = kv0 + s.kv_rank + r
            ops.sigmoid_gate(out, down[:, g0:g0 + heads * s.value_dim], target)
            out = target
        elif product_input is not None:
            ops.copy_columns(out, product_input)
            out = product_input
        return Product("mixer_out", out, self.w_o, self.t_o)
