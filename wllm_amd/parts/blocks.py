"""Arrangements of a mixer and a feed-forward around the residual stream.

"pre_norm": x += mixer(norm(x)); x += feed_forward(norm(x)), the reference's
decoder layer (src/wllm/models/gemma.py:83-93).  The residual stream is float32.
A part's contribution is not added at once: it is left pending on the stream and
the next norm kernel adds it while it normalises, so the sum is formed in
float32 and the stream is read and written once per norm.  In a decode step of few
rows the norm kernel can fall away altogether (`ResidualStream`).

"parallel": h = norm(x); x += mixer(h) + feed_forward(h).  One norm, both parts read its
output.  Both parts end in a product (attention's output projection, the feed-forward's down
projection), and the sum of two products is one product over the two inputs side by side:
[a | f] [Wo | Wd]^T.  The block lays the two weights side by side at load, lets the parts write
their products' inputs into the two bands of one buffer, and makes that one product: the sum is
formed in the product's float32 accumulators, and the stream sees one contribution.

"sandwich": x += post(mixer(pre(x))); x += post(feed_forward(pre(x))): a norm behind each sublayer as
well as before it, then, if the layer has one, a per-layer token input that reads the stream itself.
A sublayer's product stays pending together with the norm it has to pass (`pending_norm`), and the
next norm kernel normalises it, adds it and normalises the sum for the next sublayer in one pass.

"post_norm": x += post(mixer(x)); x += post(feed_forward(x)): no norm in front of a sublayer, which reads
the stream itself, optionally through a short convolution over time (`InputConv`: the stream's value plus
a weighted sum of its last few values, channel by channel).  The convolution's last inputs are state that
the block, not its mixer, carries for a request: the block names it in `state_shapes()` and finds it
under (run, name).
"""
from __future__ import annotations

from typing import Optional

import torch

from wllm_amd.kernels import ops
from wllm_amd.parts.common import Product
from wllm_amd.parts.registry import build_feed_forward, build_mixer, build_norm, register_block
from wllm_amd.parts.specs import BlockSpec, InputConvSpec
from wllm_amd.weights.checkpoint import ExpectedTensor


class ResidualStream:
    """x (float32 [n, H]) plus a contribution not yet added to it.

    Two ways lead from one part to the next.  The general one: the part's contribution (a tensor,
    or a stack of partial sums) stays pending and the next norm kernel adds it while it
    normalises.  The short one, for the few rows of a decode step: a contribution that is still a
    product (`common.Product`) is added to x by the product kernel itself, which also leaves the
    rows' sums of squares (`sumsq`); a next part that can apply the norm while it reads x
    (`takes_norm_on_load`) then needs no norm kernel at all."""

    def __init__(self, x: torch.Tensor, pending: Optional[torch.Tensor] = None):
        self.x = x
        self.pending = pending
        self.pending_bias: Optional[torch.Tensor] = None      # float32 [H]: a row that comes with `pending`
        self.pending_norm = None       # an `ops.NormRecipe`: `pending` passes this norm before it is added
        self.sumsq: Optional[torch.Tensor] = None      # float32 [n, bands]: sums of squares of x as it is now

    def normed(self, norm, out: torch.Tensor, rows=None) -> torch.Tensor:
        """norm(x + pending).  Without `rows` the sum becomes the new x."""
        if self.pending_norm is not None:
            if getattr(norm, "takes_delta_norm", False) and self.pending_bias is None:
                norm.forward(self.x, out, delta=self.pending, rows=rows, delta_norm=self.pending_norm)
                if rows is None:
                    self.pending = self.pending_norm = None
                    self.sumsq = None
                return out
            if rows is not None:
                raise NotImplementedError("gathered rows of a stream whose pending part has a norm, under a norm "
                                          "that cannot apply it")
            self.settle()
        if self.pending_bias is not None:
            norm.forward(self.x, out, delta=self.pending, rows=rows, delta_bias=self.pending_bias)
        else:
            norm.forward(self.x, out, delta=self.pending, rows=rows)
        if rows is None and (self.pending is not None or self.pending_bias is not None):
            self.pending = self.pending_bias = None
            self.sumsq = None
        return out

    def settle(self, addend: Optional[torch.Tensor] = None) -> None:
        """x takes what is pending, and `addend` (float32, x's shape) with it, without a norm."""
        if self.pending is None and self.pending_bias is None and addend is None:
            return
        if self.pending_norm is not None:
            ops.norm_add(self.x, delta=self.pending, delta_norm=self.pending_norm)
            self.pending = self.pending_norm = None
            self.sumsq = None
            if self.pending_bias is None and addend is None:
                return
        ops.stream_add(self.x, addend, self.pending, self.pending_bias)
        self.pending = self.pending_bias = None
        self.sumsq = None

    def input_for(self, ctx, norm, part):
        """What `part` gets as its input: the normalised stream as a tensor, or, where the part and
        the norm allow it, the recipe to normalise it while reading (`ops.NormOnLoad`)."""
        n, hidden = self.x.shape
        if (self.pending is None and self.pending_bias is None and self.sumsq is not None and hasattr(norm, "on_load")
                and getattr(part, "takes_norm_on_load", lambda *a: False)(n, ctx.dtype)):
            return norm.on_load(self.x, self.sumsq, ctx.dtype)
        return self.normed(norm, ctx.buffer("normed", (n, hidden), ctx.dtype))

    def as_activations(self, ctx) -> torch.Tensor:
        """The stream itself (what is pending added) in the activation type, for a part that reads it
        without a norm."""
        n, hidden = self.x.shape
        if ctx.dtype == torch.float32:
            self.settle()
            return self.x
        out = ctx.buffer("stream_cast", (n, hidden), ctx.dtype)
        if self.pending_bias is not None:
            self.settle()
        ops.norm_add(self.x, delta=self.pending, delta_norm=self.pending_norm, out=out)
        self.pending = self.pending_norm = None
        self.sumsq = None
        return out

    def add(self, ctx, y, norm=None) -> None:
        """`norm` (a norm part): the contribution passes it before it is added (a norm behind a sublayer)."""
        if self.pending is not None or self.pending_bias is not None:
            raise RuntimeError("a contribution is already pending; normalise before adding another")
        if norm is not None:
            if isinstance(y, Product):
                if y.bias is not None:
                    raise NotImplementedError("a product with a bias under a norm behind its sublayer")
                y = y.make(ctx)
            self.pending, self.pending_norm = y, norm.recipe()
            return
        if isinstance(y, Product):
            n, hidden = self.x.shape
            self.pending_bias = y.bias
            if y.bias is None and y.x.is_contiguous() and ops.linear_residual_takes(n, y.x.dtype, hidden, y.x.shape[1]):
                sumsq = ctx.buffer("sumsq", ops.linear_residual_sumsq_shape(n, hidden), torch.float32)
                ops.linear_residual(y.x, y.weight, self.x, sumsq, y.tiles)
                self.sumsq = sumsq
                return
            y = y.make(ctx)
        self.pending = y


@register_block("pre_norm")
class PreNormBlock:
    def __init__(self, spec: BlockSpec):
        self.spec = spec
        self.mixer = build_mixer(spec.mixer)
        self.mixer_norm = build_norm(spec.mixer_norm)
        # a layer may be its mixer alone
        self.feed_forward = self.feed_forward_norm = None
        if spec.feed_forward is not None:
            if spec.feed_forward_norm is None:
                raise ValueError("a pre-norm block's feed-forward has a norm before it")
            self.feed_forward = build_feed_forward(spec.feed_forward)
            self.feed_forward_norm = build_norm(spec.feed_forward_norm)

    def parts(self) -> list:
        own = [self.mixer_norm, self.mixer]
        return own + ([self.feed_forward_norm, self.feed_forward] if self.feed_forward is not None else [])

    def forward(self, ctx, entry: int, stream: ResidualStream) -> None:
        h = stream.input_for(ctx, self.mixer_norm, self.mixer)
        stream.add(ctx, self.mixer.forward(ctx, entry, h))
        if self.feed_forward is None:
            return
        h = stream.input_for(ctx, self.feed_forward_norm, self.feed_forward)
        stream.add(ctx, self.feed_forward.forward(ctx, h))


@register_block("parallel")
class ParallelBlock:
    """x += mixer(h) + feed_forward(h) with h = norm(x), as one product over both parts' inputs."""

    def __init__(self, spec: BlockSpec):
        if spec.feed_forward_norm is not None:
            raise ValueError("a parallel block has one norm; feed_forward_norm must be None")
        self.spec = spec
        self.mixer = build_mixer(spec.mixer)
        self.feed_forward = build_feed_forward(spec.feed_forward) if spec.feed_forward is not None else None
        self.mixer_norm = build_norm(spec.mixer_norm)
        self.w_joint = self.t_joint = None      # [Wo | Wd] and its tile-major copy, once loaded
        self.k_mixer = self.k_ff = 0

    def parts(self) -> list:
        own = [self.mixer_norm, self.mixer] + ([self.feed_forward] if self.feed_forward is not None else [])
        return own + [self]         # the block itself loads last: it joins what its parts loaded

    def expected_tensors(self) -> dict:
        return {}

    def load(self, fetch) -> None:
        """Lays the two last weights side by side, [Wo | Wd], for the one product of `forward`, and
        lets go of the parts' own copies.  Parts whose last product is not a plain attribute pair
        (`w_o`/`w_down`) keep theirs, and the block adds the two products one after the other."""
        m, f = self.mixer, self.feed_forward
        if f is None or getattr(m, "w_o", None) is None or getattr(f, "w_down", None) is None:
            return
        self.k_mixer, self.k_ff = m.w_o.shape[1], f.w_down.shape[1]
        self.w_joint = torch.cat([m.w_o, f.w_down], dim=1).contiguous()
        self.t_joint = ops.tile_weight(self.w_joint) if getattr(fetch, "tiled_copies", False) else None
        m.w_o = m.t_o = f.w_down = f.t_down = None

    def forward(self, ctx, entry: int, stream: ResidualStream) -> None:
        n, hidden = stream.x.shape
        h = stream.normed(self.mixer_norm, ctx.buffer("normed", (n, hidden), ctx.dtype))
        if self.feed_forward is None:
            stream.add(ctx, self.mixer.forward(ctx, entry, h))
            return
        if self.w_joint is None:
            # two products, one after the other: the second waits as the stream's pending contribution
            stream.add(ctx, self.mixer.forward(ctx, entry, h))
            stream.settle()
            stream.add(ctx, self.feed_forward.forward(ctx, h))
            return
        both = ctx.buffer("joint_in", (n, self.k_mixer + self.k_ff), ctx.dtype)
        a = self.mixer.forward(ctx, entry, h, product_input=both[:, :self.k_mixer])
        f = self.feed_forward.forward(ctx, h, product_input=both[:, self.k_mixer:])
        bias = a.bias if f.bias is None else (f.bias if a.bias is None else a.bias + f.bias)
        stream.add(ctx, Product("block_out", both, self.w_joint, self.t_joint, bias=bias))


@register_block("sandwich")
class SandwichBlock:
    """x += post(mixer(pre(x))); x += post(feed_forward(pre(x))); then the layer's token input."""

    def __init__(self, spec: BlockSpec):
        if spec.mixer_post_norm is None or (spec.feed_forward is not None and (
                spec.feed_forward_norm is None or spec.feed_forward_post_norm is None)):
            raise ValueError("a sandwich block has a norm before and behind each of its sublayers")
        self.spec = spec
        self.mixer = build_mixer(spec.mixer)
        self.mixer_norm = build_norm(spec.mixer_norm)
        self.mixer_post_norm = build_norm(spec.mixer_post_norm)
        self.feed_forward = self.feed_forward_norm = self.feed_forward_post_norm = None
        if spec.feed_forward is not None:
            self.feed_forward = build_feed_forward(spec.feed_forward)
            self.feed_forward_norm = build_norm(spec.feed_forward_norm)
            self.feed_forward_post_norm = build_norm(spec.feed_forward_post_norm)
        self.side = None
        if spec.side is not None:
            from wllm_amd.parts.token_side import TokenSide
            self.side = TokenSide(spec.side)

    def parts(self) -> list:
        own = [self.mixer_norm, self.mixer, self.mixer_post_norm]
        if self.feed_forward is not None:
            own += [self.feed_forward_norm, self.feed_forward, self.feed_forward_post_norm]
        return own + ([self.side] if self.side is not None else [])

    def forward(self, ctx, entry: int, stream: ResidualStream) -> None:
        h = stream.input_for(ctx, self.mixer_norm, self.mixer)
        stream.add(ctx, self.mixer.forward(ctx, entry, h), norm=self.mixer_post_norm)
        if self.feed_forward is not None:
            h = stream.input_for(ctx, self.feed_forward_norm, self.feed_forward)
            stream.add(ctx, self.feed_forward.forward(ctx, h), norm=self.feed_forward_post_norm)
        if self.side is not None:
            stream.add(ctx, self.side.forward(ctx, stream.as_activations(ctx)), norm=self.side.norm)


class InputConv:
    """h_t + sum_j w[:, j] * h_(t - taps + 1 + j) on the residual stream, in float32, from the request's carried
    rows (its last taps - 1 values of the stream; zeros for a fresh request, which are the zeros before a
    sequence's start) and into them."""

    def __init__(self, spec: InputConvSpec):
        if spec.taps < 1 or spec.taps > 64 or spec.size <= 0:
            raise ValueError(f"an input convolution has 1 to 64 taps over a positive number of channels, got {spec}")
        self.spec = spec
        self.weight = None

    @property
    def carried(self) -> int:
        """Floats a request carries for this convolution."""
        return (self.spec.taps - 1) * self.spec.size

    def expected_tensors(self) -> dict:
        return {self.spec.weight: ExpectedTensor((self.spec.size, self.spec.taps), role="vector")}

    def load(self, fetch) -> None:
        # the taps stay float32, a row a tap: the kernel's threads read neighbouring channels of one tap
        self.weight = fetch.to_device(fetch.vector(self.spec.weight).t().contiguous())

    def forward(self, ctx, state: torch.Tensor, offset: int, stream: ResidualStream) -> torch.Tensor:
        n, hidden = stream.x.shape
        out = ctx.buffer("conv_in", (n, hidden), ctx.dtype)
        single = ctx.max_q_len == 1 and ctx.num_segments == n       # a step of single tokens, a captured graph among them
        if single and stream.pending is not None and stream.pending_bias is None:
            # no token reads another's row: the launch that settles the stream also convolves and moves the carried rows
            ops.norm_add(stream.x, delta=stream.pending, delta_norm=stream.pending_norm, out=out,
                         conv=(self.weight, state, offset, ctx.state_slots))
            stream.pending = stream.pending_norm = None
            stream.sumsq = None
            return out
        stream.settle()         # the convolution reads other tokens' rows of the stream: they take what is pending first
        ops.stream_conv(stream.x, self.weight, state, offset, ctx.token_segment, ctx.seg_q_start, ctx.seg_q_len,
                        ctx.state_slots, out, single_tokens=single)
        return out


@register_block("post_norm")
class PostNormBlock:
    """x += post(mixer(read(x))); x += post(feed_forward(read(x))), read being the stream itself or its short
    convolution over time."""
    STATE = "input_conv"

    def __init__(self, spec: BlockSpec):
        if spec.mixer_norm is not None or spec.feed_forward_norm is not None:
            raise ValueError("a post-norm block has no norm in front of a sublayer")
        if spec.mixer_post_norm is None or (spec.feed_forward is not None and spec.feed_forward_post_norm is None):
            raise ValueError("a post-norm block has a norm behind each of its sublayers")
        if spec.feed_forward is None and spec.feed_forward_input_conv is not None:
            raise ValueError("a convolution in front of a feed-forward that is not there")
        self.spec = spec
        self.mixer = build_mixer(spec.mixer)
        self.mixer_post_norm = build_norm(spec.mixer_post_norm)
        self.mixer_conv = InputConv(spec.mixer_input_conv) if spec.mixer_input_conv is not None else None
        self.feed_forward = self.feed_forward_post_norm = self.feed_forward_conv = None
        if spec.feed_forward is not None:
            self.feed_forward = build_feed_forward(spec.feed_forward)
            self.feed_forward_post_norm = build_norm(spec.feed_forward_post_norm)
            if spec.feed_forward_input_conv is not None:
                self.feed_forward_conv = InputConv(spec.feed_forward_input_conv)

    def parts(self) -> list:
        own = [self.mixer_conv, self.mixer, self.mixer_post_norm, self.feed_forward_conv, self.feed_forward,
               self.feed_forward_post_norm]
        return [p for p in own if p is not None]

    def state_shapes(self) -> dict:
        """The block's own state: the two convolutions' carried rows, the mixer's first."""
        convs = [c for c in (self.mixer_conv, self.feed_forward_conv) if c is not None]
        # (a convolution of one tap carries nothing, and still names a row)
        return {self.STATE: (max(1, sum(c.carried for c in convs)),)} if convs else {}

    def _read(self, ctx, entry: int, stream: ResidualStream, conv, offset: int) -> torch.Tensor:
        if conv is None:
            return stream.as_activations(ctx)
        return conv.forward(ctx, ctx.state((entry, self.STATE)), offset, stream)

    def forward(self, ctx, entry: int, stream: ResidualStream) -> None:
        h = self._read(ctx, entry, stream, self.mixer_conv, 0)
        stream.add(ctx, self.mixer.forward(ctx, entry, h), norm=self.mixer_post_norm)
        if self.feed_forward is not None:
            offset = self.mixer_conv.carried if self.mixer_conv is not None else 0
            h = self._read(ctx, entry, stream, self.feed_forward_conv, offset)
            stream.add(ctx, self.feed_forward.forward(ctx, h), norm=self.feed_forward_post_norm)
