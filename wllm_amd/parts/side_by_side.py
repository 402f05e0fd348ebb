"""Two mixers side by side: both read the same normalised input, and the result is the sum of theirs.

Each of the two ends in a product (its output projection) and weighs its own result with its
`output_scale`, so the sum of the two is one product over the two inputs side by side,
[a | b] [Wa | Wb]^T: the two weights are laid side by side at load, the two mixers write their products'
inputs into the two bands of one buffer, and the stream gets one `Product` whose sum is formed in the
product's float32 accumulators.  At most one of the two pages a cache and at most one carries a state:
the layer's run has one cache and one state row, which the part that asked for it finds under the run's
own number.
"""
from __future__ import annotations

from typing import Optional

import torch

from wllm_amd.kernels import ops
from wllm_amd.parts.common import Product
from wllm_amd.parts.registry import build_mixer, register_mixer
from wllm_amd.parts.specs import SideBySideSpec


@register_mixer("side_by_side")
class SideBySideMixer:
    def __init__(self, spec: SideBySideSpec):
        self.spec = spec
        self.left = build_mixer(spec.left)
        self.right = build_mixer(spec.right)
        for what in ("cache_need", "state_shape"):
            if getattr(self.left, what)() is not None and getattr(self.right, what)() is not None:
                raise ValueError(f"both mixers of a pair ask for a {what.split('_')[0]}; a layer's run has one")
        self.w_o = self.t_o = None
        self.k_left = self.k_right = 0

    @property
    def graph_capturable(self) -> bool:
        return getattr(self.left, "graph_capturable", False) and getattr(self.right, "graph_capturable", False)

    def sub_parts(self) -> tuple:
        return (self.left, self.right)

    def expected_tensors(self) -> dict:
        return {**self.left.expected_tensors(), **self.right.expected_tensors()}

    def load(self, fetch) -> None:
        self.left.load(fetch)
        self.right.load(fetch)
        a, b = self.left, self.right
        if getattr(a, "w_o", None) is None or getattr(b, "w_o", None) is None:
            raise ValueError("the mixers of a pair end in a product and keep its weight as `w_o`")
        self.k_left, self.k_right = a.w_o.shape[1], b.w_o.shape[1]
        self.w_o = torch.cat([a.w_o, b.w_o], dim=1).contiguous()
        self.t_o = ops.tile_weight(self.w_o) if getattr(fetch, "tiled_copies", False) else None
        a.w_o = a.t_o = b.w_o = b.t_o = None

    def cache_need(self):
        return self.left.cache_need() or self.right.cache_need()

    def state_shape(self):
        return self.left.state_shape() or self.right.state_shape()

    def flops(self, tokens: int, keys: float = 0.0) -> float:
        return self.left.flops(tokens, keys) + self.right.flops(tokens, keys)

    def forward(self, ctx, entry: int, h: torch.Tensor, product_input: Optional[torch.Tensor] = None):
        n = h.shape[0]
        both = product_input if product_input is not None else ctx.buffer(
            "pair_in", (n, self.k_left + self.k_right), h.dtype)
        a = self.left.forward(ctx, entry, h, product_input=both[:, :self.k_left])
        b = self.right.forward(ctx, entry, h, product_input=both[:, self.k_left:])
        bias = a.bias if b.bias is None else (b.bias if a.bias is None else a.bias + b.bias)
        return Product("mixer_out", both, self.w_o, self.t_o, bias=bias)
