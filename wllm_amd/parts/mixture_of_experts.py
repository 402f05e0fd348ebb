"""A mixture of gated feed-forward experts of which every token uses a few.

    z = W_router x (float32);  s = softmax(z) over all experts
    only experts of the `keep_groups` best of `num_groups` groups of neighbours may be chosen
    the `top` allowed experts with the largest s; weights s / (sum of the chosen + weight_eps)
    y = sum over the chosen e of weight_e * down_e(act(gate_e(x)) * up_e(x))

The experts' matrices are stacked at load ([experts, 2 * ff, width]: an expert's gate rows, then its up
rows; [experts, width, ff]).  A step routes its tokens, sorts the (token, expert) pairs by expert on the
device (`ops.moe_plan`: tiles of rows of one expert) and runs the two products expert by expert on
the matrix cores, each tile with its expert's weights: tiles of 16 to 64 rows past which an expert's
weights stream where the experts get few rows each (decoded tokens), tiles of 128 rows through shared
memory where they get many (a prompt's portion).  The second product weighs a pair's result and
leaves it in the slice of its slot of a float32 stack [top, tokens, width], which whoever adds the
feed-forward to the stream (the next norm kernel) adds in order: the weighted sum is formed in float32
and takes no pass of its own.  Nothing of the routing is read on the host.

Options: the scores may be sigmoids of the logits, every expert by itself (`scoring`), and the chosen scores
may be the weights as they are (`normalize` False); the weight may multiply the expert's input instead of its
output (`weight_on_input`: the factor is taken out of the first product's two sums and multiplied in before the
activation, and the second product's results are not weighed); and one more gated feed-forward may run for
every token (`shared`), whose result is one more slice of the stack.
"""
from __future__ import annotations

import torch

from wllm_amd.kernels import ops
from wllm_amd.parts.feed_forward import GatedMLP
from wllm_amd.parts.registry import register_feed_forward
from wllm_amd.parts.specs import MixtureOfExpertsSpec
from wllm_amd.weights.checkpoint import ExpectedTensor


@register_feed_forward("mixture_of_experts")
class MixtureOfExperts:
    routed_tensors = ("w_up", "w_down")      # a step reads the chosen experts' share of these: `bytes_read`

    def __init__(self, spec: MixtureOfExpertsSpec):
        if spec.activation not in ops.ACTIVATIONS:
            raise ValueError(f"activation {spec.activation!r} is not implemented; known: {ops.ACTIVATIONS}")
        if not 0 < spec.num_experts <= ops.MOE_MAX_EXPERTS:
            raise ValueError(f"num_experts {spec.num_experts}: from 1 to {ops.MOE_MAX_EXPERTS}")
        if spec.num_groups <= 0 or spec.num_experts % spec.num_groups or not 0 < spec.keep_groups <= spec.num_groups:
            raise ValueError(f"num_groups ({spec.num_groups}) must divide num_experts ({spec.num_experts}), and "
                             f"keep_groups ({spec.keep_groups}) lie between 1 and num_groups")
        if not 0 < spec.top <= spec.keep_groups * (spec.num_experts // spec.num_groups):
            raise ValueError(f"top ({spec.top}): at most the experts of the kept groups")
        if spec.scoring not in ops.MOE_SCORINGS:
            raise ValueError(f"scoring {spec.scoring!r}: one of {sorted(ops.MOE_SCORINGS)}")
        self.spec = spec
        self.shared = GatedMLP(spec.shared) if spec.shared is not None else None
        self.w_router = self.w_up = self.w_down = None
        self.t_up = self.t_down = None          # the stacks' tile-major copies, which the few-row kernels stream

    def _names(self, e: int) -> tuple:
        s = self.spec
        p = f"{s.expert_prefix}{e}."
        return p + s.gate_name, p + s.up_name, p + s.down_name

    def expected_tensors(self) -> dict:
        s = self.spec
        # the router works in float32: its weight is kept so (exact from a bfloat16 file)
        out = {s.router_weight: ExpectedTensor((s.num_experts, s.hidden_size), role="vector")}
        for e in range(s.num_experts):
            gate, up, down = self._names(e)
            out[gate] = ExpectedTensor((s.intermediate_size, s.hidden_size))
            out[up] = ExpectedTensor((s.intermediate_size, s.hidden_size))
            out[down] = ExpectedTensor((s.hidden_size, s.intermediate_size))
        if self.shared is not None:
            out.update(self.shared.expected_tensors())
        return out

    def sub_parts(self) -> tuple:
        return (self.shared,) if self.shared is not None else ()

    def load(self, fetch) -> None:
        s = self.spec
        if self.shared is not None:
            self.shared.load(fetch)
        ups, downs = [], []
        for e in range(s.num_experts):
            gate, up, down = self._names(e)
            ups.append(torch.cat([fetch.matrix(gate), fetch.matrix(up)], dim=0))
            downs.append(fetch.matrix(down))
        self.w_up = fetch.to_device(torch.stack(ups).contiguous())
        self.w_down = fetch.to_device(torch.stack(downs).contiguous())
        self.w_router = fetch.to_device(fetch.vector(s.router_weight))
        if (getattr(fetch, "tiled_copies", False) and self.w_up.dtype == torch.bfloat16 and s.intermediate_size % 32 == 0
                and s.hidden_size % 32 == 0):
            # a band of 16 rows never holds rows of two experts (nor gate rows beside up rows)
            self.t_up = ops.tile_weight(self.w_up.view(-1, s.hidden_size))
            self.t_down = ops.tile_weight(self.w_down.view(-1, s.intermediate_size))

    def flops(self, tokens: int) -> float:
        s = self.spec
        shared = self.shared.flops(tokens) if self.shared is not None else 0.0
        return 2.0 * tokens * s.hidden_size * (3 * s.top * s.intermediate_size + s.num_experts) + shared

    def bytes_read(self, tokens: int) -> float:
        """Bytes of expert weights a step of `tokens` tokens reads if the router spreads the tokens evenly: every
        expert that at least one token chooses, once (experts * (1 - (1 - top / experts) ** tokens) of them)."""
        s = self.spec
        used = s.num_experts * (1.0 - (1.0 - s.top / s.num_experts) ** tokens)
        return 3.0 * used * s.intermediate_size * s.hidden_size * self.w_up.element_size()

    def forward(self, ctx, h, product_input=None):
        if product_input is not None:
            raise NotImplementedError("a mixture of experts ends in a product a token and expert, not in one product")
        s = self.spec
        n = h.shape[0]
        ids = ctx.buffer("moe_ids", (n, s.top), torch.int32)
        weights = ctx.buffer("moe_weights", (n, s.top), torch.float32)
        ops.moe_route(h, self.w_router, ids, weights, groups=s.num_groups, keep=s.keep_groups, eps=s.weight_eps,
                      scoring=s.scoring, normalize=s.normalize)
        rows = ops.moe_tile_rows(n * s.top, s.num_experts, h.dtype, s.hidden_size, s.intermediate_size)
        plan = ctx.buffer("moe_plan", (ops.moe_plan_size(n * s.top, s.num_experts, rows),), torch.int32)
        ops.moe_plan(ids, plan, s.num_experts, rows)
        act = ctx.buffer("moe_act", (n * s.top, s.intermediate_size), h.dtype)
        ops.moe_experts_up(h, self.w_up, plan, act, s.top, s.activation, rows, self.t_up,
                           in_weights=weights if s.weight_on_input else None)
        out = ctx.buffer("moe_out", (s.top + (1 if self.shared is not None else 0), n, s.hidden_size), torch.float32)
        ops.moe_experts_down(act, self.w_down, plan, weights, out[:s.top], rows, self.t_down, weighted=not s.weight_on_input)
        if self.shared is not None:
            # the expert every token uses: its product's float32 sums are the stack's last slice
            last = self.shared.forward(ctx, h)
            if h.dtype == torch.float32 or n <= 64:
                ops.linear(last.x, last.weight, out[s.top], last.tiles)
            else:
                # many rows: the product as every other of this size is made (in the activation type), then into its slice
                out[s.top].zero_()
                ops.stream_add(out[s.top], delta=last.make(ctx))
        return out
