"""The attention mixer: q/k/v projection as one product, rotation and cache write
as one kernel, attention over the request's pages, output projection.

It follows the reference's attention (src/wllm/models/llama.py:82-115 for the
formulas, :143-247 for the cached forms) with one code path for all of them: a
flat batch of segments, each the next tokens of some request, a decoded token
being a segment of one.  Head h of the q/k/v rows is columns h*head_dim ..
(h+1)*head_dim of the projection (llama.py:103-105).  The three projection
matrices are stacked at load so that one product makes the [n, (nh+2nkv)*d]
row the kernels read.

The specification's options widen the row and the steps between projection and attention
(`ops.head_prepare` then stands where `ops.rope_and_cache_write` stands for the plain form): a
rotation of interleaved pairs or of a part of the head, a unit norm of queries and keys, values
that are the keys as projected (the row has no value heads), a cap on the scores, and an output
gate whose projection is stacked behind the heads (row: queries, keys, [values], [gate]) and
multiplied into the attention's result before the output projection, which may have a bias.
Further options: value heads of another size than the key heads (both are padded to the larger in
the row and in the cache, with zeros that add nothing to a score or a result); a mask of chunks
instead of a window; an RMS norm with a weight over the whole query projection and over the whole key
projection (`ops.band_norm`) in place of the norm of each head; a gate of one number a head; and a
layer without key and value projections that reads another layer's cache with its own queries.
And: an RMS norm with a weight over every query head and every key head before the rotation (the weight
has head_dim numbers that the heads share), and a learned number a head in the softmax's denominator.
"""
from __future__ import annotations

from typing import Optional

import torch

from wllm_amd.cache.manager import CacheNeed
from wllm_amd.kernels import ops
from wllm_amd.parts.common import Product, load_matrix, project
from wllm_amd.parts.registry import build_position, register_mixer
from wllm_amd.parts.specs import AttentionSpec
from wllm_amd.weights.checkpoint import ExpectedTensor


@register_mixer("attention")
class PagedAttention:
    graph_capturable = True     # everything it does reads the step's device arrays

    def __init__(self, spec: AttentionSpec):
        if spec.num_heads % spec.num_kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        if spec.window is not None and spec.window <= 0:
            raise ValueError(f"window must be positive or None, got {spec.window}")
        plain = not (spec.softcap or spec.qk_norm_eps is not None or spec.values_are_keys or spec.gate_weight
                     or spec.position.pairing == "interleaved" or spec.value_dim not in (None, spec.head_dim)
                     or spec.chunk or spec.q_norm_weight or spec.k_norm_weight or not spec.owns_cache
                     or spec.sink is not None or spec.output_scale != 1.0 or spec.q_head_norm_weight
                     or spec.k_head_norm_weight or spec.sink_weight or spec.position.magnitude != 1.0)
        if bool(spec.q_head_norm_weight) != bool(spec.k_head_norm_weight) or (
                spec.q_head_norm_weight and (spec.head_norm_eps is None or spec.head_norm_eps < 0)):
            raise ValueError("a norm over each head has a weight for the queries, one for the keys, and head_norm_eps")
        if spec.q_head_norm_weight and (spec.q_norm_weight or spec.k_norm_weight):
            raise ValueError("a norm over each head and a norm over the whole projection: one of the two")
        if spec.q_head_norm_weight and not spec.owns_cache:
            raise ValueError("a norm over each head: the layer has keys of its own")
        if spec.sink_weight and spec.sink is not None:
            raise ValueError("sink and sink_weight: the denominator's term is a constant or a learned number a head")
        if spec.chunk is not None and (spec.chunk <= 0 or spec.window is not None):
            raise ValueError(f"chunk must be positive and excludes a window, got chunk {spec.chunk}, window {spec.window}")
        if (spec.q_norm_weight or spec.k_norm_weight) and spec.band_norm_eps is None:
            raise ValueError("a norm over the whole query or key projection needs band_norm_eps")
        if not spec.owns_cache and (spec.k_weight or spec.v_weight or spec.k_norm_weight or spec.values_are_keys
                                    or spec.qk_norm_eps is not None or spec.position.kind != "none"):
            raise ValueError("a layer without a cache of its own has no key or value projection, and its queries "
                             "are neither rotated nor normed head by head")
        if spec.bias_before_norm and not (spec.q_norm_weight and (spec.k_norm_weight or not spec.owns_cache)):
            raise ValueError("bias_before_norm: the query and key projections have norms over the whole projection")
        if spec.gate_per_head and not spec.gate_weight:
            raise ValueError("gate_per_head without a gate")
        if (plain and spec.head_dim % ops.HEAD_DIM_STEP) or not 0 < spec.head_dim <= ops.MAX_HEAD_DIM:
            raise ValueError(f"head_dim {spec.head_dim}: the attention kernels take multiples of "
                             f"{ops.HEAD_DIM_STEP} up to {ops.MAX_HEAD_DIM}")
        if spec.values_are_keys and (spec.v_weight or spec.v_bias):
            raise ValueError("values_are_keys: there is no value projection to name")
        if spec.softcap is not None and not spec.softcap > 0:
            raise ValueError(f"softcap must be positive or None, got {spec.softcap}")
        if spec.qk_norm_eps is not None and spec.qk_norm_eps < 0:
            raise ValueError(f"qk_norm_eps must not be negative, got {spec.qk_norm_eps}")
        self.spec = spec
        self.position = build_position(spec.position)
        self.w_qkv = None
        self.b_qkv = None
        self.w_o = None
        self.b_o = None
        # the plain form runs the kernels that were written for it; anything else the general ones
        self.plain = plain
        # The kernels take heads of a multiple of four elements.  A head of another size is padded at load with
        # rows of zeros in its projections (and columns of zeros in the output projection): the padding is zero
        # in queries, keys and values, adds nothing to a score or a result, and the unit norm divides by the
        # true size.  Only the general path does this.
        self.vdim = spec.value_dim or spec.head_dim
        largest = max(spec.head_dim, self.vdim)
        self.dim = spec.head_dim if plain else -(-largest // ops.HEAD_DIM_STEP) * ops.HEAD_DIM_STEP
        if not 0 < self.dim <= ops.MAX_HEAD_DIM:
            raise ValueError(f"value_dim {self.vdim}: the attention kernels take heads up to {ops.MAX_HEAD_DIM}")
        self.w_q_norm = self.w_k_norm = None
        self.w_q_head_norm = self.w_k_head_norm = None
        self.b_q = self.b_k = None          # biases that are added in front of the norm over a whole projection
        self.sinks = None

    @property
    def qkv_width(self) -> int:
        """Columns of the projected row: queries, keys, values (unless they are the keys), gate."""
        s = self.spec
        width = self.gate_offset + (self.gate_width if s.gate_weight else 0)
        # a gate of a number a head can leave the row at any width; the kernels read rows that begin at
        # multiples of 16 bytes, so the row is padded (with zero rows of the stacked weight)
        return -(-width // 8) * 8 if s.gate_per_head else width

    @property
    def gate_offset(self) -> int:
        s = self.spec
        kv = ((1 if s.values_are_keys else 2) * s.num_kv_heads) if s.owns_cache else 0
        return (s.num_heads + kv) * self.dim

    @property
    def gate_width(self) -> int:
        """Columns of the gate's projection: a number a head, or one for every element of the heads."""
        return self.spec.num_heads if self.spec.gate_per_head else self.spec.num_heads * self.dim

    def expected_tensors(self) -> dict:
        s = self.spec
        q, kv = s.num_heads * s.head_dim, s.num_kv_heads * s.head_dim
        out = {
            s.q_weight: ExpectedTensor((q, s.hidden_size)),
            s.o_weight: ExpectedTensor((s.hidden_size, s.num_heads * self.vdim)),
        }
        if s.owns_cache:
            out[s.k_weight] = ExpectedTensor((kv, s.hidden_size))
            if not s.values_are_keys:
                out[s.v_weight] = ExpectedTensor((s.num_kv_heads * self.vdim, s.hidden_size))
        if s.gate_weight:
            out[s.gate_weight] = ExpectedTensor((s.num_heads if s.gate_per_head else s.num_heads * self.vdim, s.hidden_size))
        if s.q_norm_weight:
            out[s.q_norm_weight] = ExpectedTensor((q,), role="vector", init="norm")
        if s.k_norm_weight and s.owns_cache:
            out[s.k_norm_weight] = ExpectedTensor((kv,), role="vector", init="norm")
        if s.q_head_norm_weight:
            out[s.q_head_norm_weight] = ExpectedTensor((s.head_dim,), role="vector", init="norm")
            out[s.k_head_norm_weight] = ExpectedTensor((s.head_dim,), role="vector", init="norm")
        if s.sink_weight:
            out[s.sink_weight] = ExpectedTensor((s.num_heads,), role="vector", init="norm")
        for name, width in ((s.q_bias, q), (s.k_bias, kv), (s.v_bias, s.num_kv_heads * self.vdim), (s.o_bias, s.hidden_size)):
            if name is not None:
                out[name] = ExpectedTensor((width,), role="vector")
        if hasattr(self.position, "expected_tensors"):      # a position encoding with tensors of its own
            out.update(self.position.expected_tensors())
        return out

    def load(self, fetch) -> None:
        s = self.spec

        def heads_padded(t: torch.Tensor, axis: int, size: int = s.head_dim) -> torch.Tensor:
            """`t` with every head of `axis` (heads * size long) followed by zeros up to the padded size."""
            pad = self.dim - size
            if not pad:
                return t
            shape = list(t.shape)
            heads = shape[axis] // size
            t = t.unflatten(axis, (heads, size))
            zeros = torch.zeros(shape[:axis] + [heads, pad] + shape[axis + 1:], dtype=t.dtype, device=t.device)
            return torch.cat([t, zeros], dim=axis + 1).flatten(axis, axis + 1)

        stacked = [heads_padded(fetch.matrix(s.q_weight), 0)]
        if s.owns_cache:
            stacked.append(heads_padded(fetch.matrix(s.k_weight), 0))
            if not s.values_are_keys:
                stacked.append(heads_padded(fetch.matrix(s.v_weight), 0, self.vdim))
        if s.gate_weight:
            gate = fetch.matrix(s.gate_weight)
            stacked.append(gate if s.gate_per_head else heads_padded(gate, 0, self.vdim))
        w = torch.cat(stacked, dim=0)
        if w.shape[0] < self.qkv_width:
            w = torch.cat([w, torch.zeros(self.qkv_width - w.shape[0], w.shape[1], dtype=w.dtype, device=w.device)], dim=0)
        self.w_qkv, self.t_qkv = load_matrix(fetch, w)        # the matrix and its tile-major copy
        self.w_o, self.t_o = load_matrix(fetch, heads_padded(fetch.matrix(s.o_weight), 1, self.vdim))
        if s.q_norm_weight:
            self.w_q_norm = fetch.to_device(heads_padded(fetch.vector(s.q_norm_weight), 0))
        if s.k_norm_weight and s.owns_cache:
            self.w_k_norm = fetch.to_device(heads_padded(fetch.vector(s.k_norm_weight), 0))
        if s.o_bias is not None:
            self.b_o = fetch.to_device(fetch.vector(s.o_bias))
        if s.q_bias is not None or s.k_bias is not None or s.v_bias is not None:
            q, kv = s.num_heads * s.head_dim, s.num_kv_heads * s.head_dim
            if not s.owns_cache:
                raise NotImplementedError("biases of the projections of a layer without keys of its own")
            biases = [(s.q_bias, q, s.head_dim), (s.k_bias, kv, s.head_dim)]
            biases += [] if s.values_are_keys else [(s.v_bias, s.num_kv_heads * self.vdim, self.vdim)]
            # (the gate's projection, behind the heads in the row, has none: the bias is shorter than the row)
            found = [fetch.vector(name) if name is not None else None for name, _, _ in biases]
            where = next(v.device for v in found if v is not None)      # a fetcher may make its tensors on the device
            parts = [heads_padded(v if v is not None else torch.zeros(width, device=where), 0, size)
                     for v, (_, width, size) in zip(found, biases)]
            if s.bias_before_norm:
                # the norm kernel adds the queries' and keys' biases as it reads; what is left for the
                # kernel behind it is the values' bias
                self.b_q = fetch.to_device(parts[0]) if s.q_bias is not None else None
                self.b_k = fetch.to_device(parts[1]) if s.k_bias is not None else None
                parts[0], parts[1] = torch.zeros_like(parts[0]), torch.zeros_like(parts[1])
            if not s.bias_before_norm or (len(parts) > 2 and s.v_bias is not None):
                self.b_qkv = fetch.to_device(torch.cat(parts))
        if s.sink is not None:
            self.sinks = torch.full((s.num_heads,), float(s.sink), dtype=torch.float32, device=fetch.device)
        if s.sink_weight:
            self.sinks = fetch.to_device(fetch.vector(s.sink_weight))
        if s.q_head_norm_weight:
            # (a padded head's last elements are zero and stay zero under a weight of zero)
            self.w_q_head_norm = fetch.to_device(heads_padded(fetch.vector(s.q_head_norm_weight), 0))
            self.w_k_head_norm = fetch.to_device(heads_padded(fetch.vector(s.k_head_norm_weight), 0))
        if hasattr(self.position, "load"):
            self.position.load(fetch)
        self.position.prepare(fetch.device)

    def cache_need(self) -> Optional[CacheNeed]:
        s = self.spec
        return CacheNeed(s.num_kv_heads, self.dim, s.window, s.release_chunk if s.chunk else None)

    def state_shape(self):
        return None

    def flops(self, tokens: int, keys: float) -> float:
        """Floating-point operations of `tokens` tokens whose queries see `keys` keys in all (what a
        measurement divides by its time)."""
        s = self.spec
        if s.chunk:
            keys = min(keys, tokens * (s.chunk + 1) / 2.0)      # a query sees half a chunk on average
        return (2.0 * tokens * s.hidden_size * (self.qkv_width + s.num_heads * self.vdim)
                + 2.0 * s.num_heads * (s.head_dim + self.vdim) * keys)

    def _work_items(self, ctx, page_size: int):
        """The step's work items for attention of this shape: made once a step, shared by all
        layers of the shape; of fixed shape and rewritten in place in a captured graph."""
        s = self.spec
        # (the plan depends on these alone: layers that differ in their rows' width or cap share it)
        # (the mask as the one integer the plan takes: a window w > 0, chunks of c positions as -c)
        shape = dict(num_heads=s.num_heads, num_kv_heads=s.num_kv_heads, head_dim=self.dim, page_size=page_size,
                     window=-s.chunk if s.chunk else (s.window or 0))

        def build(c):
            if c.captured:
                return ops.static_attention_plan(c.num_segments, max_context=c.capture_max_context,
                                                 max_total_keys=c.capture_max_tokens, dtype=c.dtype, device=c.device, **shape)
            return ops.plan_paged_attention(c.host_q_len, c.host_ctx_len, dtype=c.dtype, device=c.device, **shape)

        def refresh(plan, c):
            plan.update(c.host_q_len, c.host_ctx_len)

        return ctx.plan(("attention",) + tuple(shape.values()), build, refresh)

    def forward(self, ctx, entry: int, h: torch.Tensor, product_input: Optional[torch.Tensor] = None):
        """`product_input`: a band of columns [n, heads * head_dim] of a wider buffer into which the
        input of the output projection is to be written (a block that makes one product of several
        parts' last products asks for it); the returned `Product` then names that band."""
        s = self.spec
        n = h.shape[0]
        qkv = ctx.buffer("qkv", (n, self.qkv_width), h.dtype)
        pages = ctx.pages(entry)
        slots, storage = (pages.slots, pages.storage) if pages.writes else (None, None)
        # What the position encoding asks for: a table of frequencies that the rotation kernels turn
        # queries and keys by (`inv_freq`, or None), and/or a step of its own on the projected rows
        # before they are cached and read (`apply`).
        inv_freq = self.position.inv_freq
        apply = getattr(self.position, "apply", None)
        rotary_dim = 2 * inv_freq.shape[0] if inv_freq is not None else s.head_dim
        if not self.plain and (self.w_q_norm is not None or not s.owns_cache):
            if apply is not None:
                raise NotImplementedError("a position encoding with a step of its own beside the attention's options")
            # the whole projections are normed before the heads are split: the sums of a split product are
            # made here, and the norm kernel takes the query band and the key band in one launch
            ops.linear(h, self.w_qkv, qkv, self.t_qkv)
            q_width, kv_width = s.num_heads * self.dim, s.num_kv_heads * self.dim
            bands = []
            if self.w_q_norm is not None:
                bands.append((qkv[:, :q_width], self.w_q_norm, s.num_heads * s.head_dim, qkv[:, :q_width], self.b_q))
            if self.w_k_norm is not None:
                bands.append((qkv[:, q_width:q_width + kv_width], self.w_k_norm, s.num_kv_heads * s.head_dim,
                              qkv[:, q_width:q_width + kv_width], self.b_k))
            if bands:
                ops.band_norm(bands, s.band_norm_eps)
            if s.owns_cache:
                ops.head_prepare(
                    qkv, self.b_qkv, ctx.positions, inv_freq, slots, storage, num_heads=s.num_heads,
                    num_kv_heads=s.num_kv_heads, head_dim=self.dim, page_size=pages.page_size,
                    interleaved=getattr(self.position, "interleaved", False), norm_eps=s.qk_norm_eps,
                    values_are_keys=s.values_are_keys, norm_dim=s.head_dim, rot_scale=getattr(self.position, "magnitude", 1.0))
        elif not self.plain:
            if apply is not None:
                raise NotImplementedError("a position encoding with a step of its own beside the attention's options")
            projected = project(ctx, "qkv", h, self.w_qkv, qkv, tiles=self.t_qkv)
            ops.head_prepare(
                qkv, self.b_qkv, ctx.positions, inv_freq, slots, storage, num_heads=s.num_heads,
                num_kv_heads=s.num_kv_heads, head_dim=self.dim, page_size=pages.page_size,
                interleaved=getattr(self.position, "interleaved", False), norm_eps=s.qk_norm_eps,
                values_are_keys=s.values_are_keys, parts=projected if projected.dim() == 3 else None,
                norm_dim=s.head_dim, rot_scale=getattr(self.position, "magnitude", 1.0),
                head_norm=(self.w_q_head_norm, self.w_k_head_norm, s.head_norm_eps) if self.w_q_head_norm is not None else None)
        elif apply is not None:
            ops.linear(h, self.w_qkv, qkv, self.t_qkv)
            if self.b_qkv is not None:
                qkv += self.b_qkv.to(qkv.dtype)
            apply(ctx, qkv, num_heads=s.num_heads, num_kv_heads=s.num_kv_heads, head_dim=s.head_dim)
            ops.rope_and_cache_write(
                qkv, None, ctx.positions, inv_freq, slots, storage,
                num_heads=s.num_heads, num_kv_heads=s.num_kv_heads, head_dim=s.head_dim, page_size=pages.page_size)
        elif ops.qkv_rope_takes(n, h.dtype, h.shape[1], s.head_dim, rotary_dim):
            # a decode step: projection, rotation and cache write in one kernel
            ops.qkv_rope(h, self.w_qkv, qkv, self.b_qkv, ctx.positions, inv_freq, slots, storage,
                         num_heads=s.num_heads, num_kv_heads=s.num_kv_heads, head_dim=s.head_dim,
                         page_size=pages.page_size, tiles=self.t_qkv)
        else:
            # where the product kernel splits its sums, the rotation kernel adds them as it reads
            projected = project(ctx, "qkv", h, self.w_qkv, qkv, tiles=self.t_qkv)
            parts = projected if projected.dim() == 3 else None
            ops.rope_and_cache_write(
                qkv, self.b_qkv, ctx.positions, inv_freq, slots, storage,
                num_heads=s.num_heads, num_kv_heads=s.num_kv_heads, head_dim=s.head_dim, page_size=pages.page_size,
                parts=parts)
        attn = ctx.buffer("attn", (n, s.num_heads * self.dim), h.dtype)
        ops.paged_attention(
            qkv, pages.storage, pages.block_tables, ctx.token_segment, ctx.seg_q_start, ctx.seg_q_len,
            ctx.seg_ctx_len, attn, num_heads=s.num_heads, num_kv_heads=s.num_kv_heads, head_dim=self.dim,
            page_size=pages.page_size, scale=s.scale, window=s.window or 0,
            max_q_len=ctx.max_q_len, max_ctx_len=ctx.max_ctx_len,
            plan=self._work_items(ctx, pages.page_size), softcap=s.softcap or 0.0, exact_weights=s.weights_in_float32,
            chunk=s.chunk or 0, sinks=self.sinks)
        if s.gate_weight:
            # the gate's columns lie behind the heads in the projected row
            gate = qkv[:, self.gate_offset:self.gate_offset + self.gate_width]
            target = product_input if product_input is not None else attn
            ops.sigmoid_gate(attn, gate, target, per=self.dim if s.gate_per_head else 1)
            attn = target
            if s.output_scale != 1.0:
                ops.copy_columns(attn, attn, s.output_scale)
        elif product_input is not None or s.output_scale != 1.0:
            target = product_input if product_input is not None else attn
            ops.copy_columns(attn, target, s.output_scale)
            attn = target
        # the stream adds the output projection: at once, or through the next norm, partial sums and all
        return Product("mixer_out", attn, self.w_o, self.t_o, bias=self.b_o)
