"""Duvozen as a plan of parts.

A decoder whose layers have no norm in front of a sublayer and a layer norm (a weight, no bias) behind it:
x += norm1(mixer(read(x))), then (if the layer has a feed-forward) x += norm2(ff(read(x))), where read(x) is the
stream plus a short causal convolution of it over time (`canon1` for the mixer, `canon2` for the feed-forward,
[width, taps]).  The file picks each layer's mixer: a gated linear recurrence whose forget gate also decides what
is written (HGRN2); latent attention over one cached compressed vector a token and a short turned key part that
the heads share; or softmax attention with grouped key heads, an RMS norm over each query and key head before the
rotation, a learned term a head in the softmax's denominator and an elementwise gate on its result.  The
feed-forward is gated (gelu in its tanh form) or a mixture of silu-gated experts chosen by their sigmoid scores,
the score multiplying the expert's input, with an expert that every token uses.  The head is a matrix of its
own behind the model's layer norm, and the logits are multiplied by a factor.  Tensor names: `embed`, `head`,
`final.norm`, and per layer i `l<i>.norm1`, `.norm2`, `.canon1`, `.canon2`, `l<i>.mix.*`,
`l<i>.mlp.{gate,up,down}` or `l<i>.mlp.{router, e<j>.{gate,up,down}, shared.{gate,up,down}}`.

What the design fixes (and the file does not carry): the factor of sine and cosine where the frequencies are
interpolated, 0.1 ln(factor) + 1.
"""
from __future__ import annotations

import math

from wllm_amd.architectures.duvozen_config import DuvozenConfig
from wllm_amd.config.registry import register_architecture
from wllm_amd.parts.specs import (
    AttentionSpec,
    BlockSpec,
    EmbeddingSpec,
    GatedMLPSpec,
    HeadSpec,
    InputConvSpec,
    LatentAttentionSpec,
    MatrixMemorySpec,
    MixtureOfExpertsSpec,
    ModelPlan,
    NormSpec,
    PositionSpec,
    ScheduleEntry,
)

# the design names no longest sequence: a request is as long as the cache lets it be
NO_POSITION_LIMIT = 1 << 30


def _position(rotation, pairing: str) -> PositionSpec:
    if rotation is None:
        return PositionSpec(kind="none")
    magnitude = 1.0
    if rotation.scaling is not None:
        magnitude = 0.1 * math.log(rotation.scaling[0]) + 1.0
    return PositionSpec(kind="rope", rotary_dim=rotation.dims, theta=rotation.base, pairing=pairing, ramp=rotation.scaling,
                        magnitude=magnitude)


def duvozen_plan(cfg: DuvozenConfig) -> ModelPlan:
    def norm(name: str) -> NormSpec:
        return NormSpec(size=cfg.width, eps=cfg.norm_eps, weight=name, kind="layer")

    def gated(prefix: str, ff: int, activation: str) -> GatedMLPSpec:
        return GatedMLPSpec(hidden_size=cfg.width, intermediate_size=ff, activation=activation, gate_weight=prefix + "gate",
                            up_weight=prefix + "up", down_weight=prefix + "down")

    layers, ignored = [], []
    for i, layer in enumerate(cfg.layers):
        m, q = layer.mixer, f"l{i}."
        p = q + "mix."
        if layer.type == "hgrn2":
            mixer = MatrixMemorySpec(
                hidden_size=cfg.width, num_heads=m.heads, head_dim=m.dim, value_dim=m.vdim, gating="forget",
                q_activation="silu", q_weight=p + "q", k_weight="", v_weight=p + "v", gate_weight=None, o_weight=p + "o",
                f_weight=p + "f", f_bias=p + "f.b", lower_bound=p + "lower", norm_weight=p + "norm",
                norm_weight_per_head=False, norm_eps=cfg.norm_eps, gate_activation="none")
        elif layer.type == "latent_attention":
            mixer = LatentAttentionSpec(
                hidden_size=cfg.width, num_heads=m.heads, head_dim=m.dim, value_dim=m.vdim, kv_rank=m.kv_rank,
                scale=m.scale, norm_eps=cfg.norm_eps, q_weight=p + "q", dkv_weight=p + "dkv",
                dkv_norm_weight=p + "dkv.norm", uk_weight=p + "uk", uv_weight=p + "uv", o_weight=p + "o",
                rope_dim=m.rot_dim, position=_position(m.rotation, "interleaved"), weights_in_float32=True)
        else:
            mixer = AttentionSpec(
                hidden_size=cfg.width, num_heads=m.heads, num_kv_heads=m.kv_heads, head_dim=m.dim, value_dim=m.vdim,
                scale=m.scale, position=_position(m.rotation, "half"), q_weight=p + "q", k_weight=p + "k",
                v_weight=p + "v", o_weight=p + "o", gate_weight=p + "g", q_head_norm_weight=p + "q.norm",
                k_head_norm_weight=p + "k.norm", head_norm_eps=cfg.norm_eps, sink_weight=p + "sink",
                weights_in_float32=True)
        ff = None
        if layer.mlp is not None and layer.mlp.kind == "dense":
            ff = gated(q + "mlp.", layer.mlp.ff, "gelu_tanh")
        elif layer.mlp is not None:
            e = layer.mlp
            ff = MixtureOfExpertsSpec(
                hidden_size=cfg.width, intermediate_size=e.ff, num_experts=e.experts, top=e.top, activation="silu",
                router_weight=q + "mlp.router", expert_prefix=q + "mlp.e", scoring="sigmoid", normalize=False,
                weight_on_input=True,
                shared=gated(q + "mlp.shared.", e.shared_ff, "silu") if e.shared_ff is not None else None)
        else:
            ignored += [q + "norm2", q + "canon2"]
        layers.append(BlockSpec(
            arrangement="post_norm", mixer=mixer, feed_forward=ff, mixer_norm=None, feed_forward_norm=None,
            mixer_post_norm=norm(q + "norm1"), feed_forward_post_norm=norm(q + "norm2") if ff is not None else None,
            mixer_input_conv=InputConvSpec(cfg.width, cfg.taps, q + "canon1"),
            feed_forward_input_conv=InputConvSpec(cfg.width, cfg.taps, q + "canon2") if ff is not None else None))
    return ModelPlan(
        embedding=EmbeddingSpec(vocab_size=cfg.vocab, hidden_size=cfg.width, weight="embed", scale=cfg.embedding_scale),
        layers=tuple(layers), schedule=tuple(ScheduleEntry(layer=i) for i in range(len(layers))),
        final_norm=norm("final.norm"),
        head=HeadSpec(vocab_size=cfg.vocab, hidden_size=cfg.width, weight="head", logit_scale=cfg.logit_scale),
        max_positions=NO_POSITION_LIMIT, ignored_tensor_suffixes=tuple(ignored))


register_architecture("Duvozen", DuvozenConfig.from_dict, duvozen_plan)
