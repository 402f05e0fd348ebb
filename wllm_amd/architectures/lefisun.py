"""Lefisun as a plan of parts.

A decoder of pre-norm layers, x += mixer(rms(x)); x += experts(rms(x)) (a layer may have no
feed-forward), whose mixer the file picks layer by layer.  "parallel": two mixers side by side on the
same input, their results weighed and added: on the left softmax attention inside chunks of the sequence
(grouped heads, biases on q, k and v, an RMS norm with a weight over the whole query and the whole key
projection behind the biases, rotation of the first elements of every head in the half-split pairing
with linearly scaled positions, one more 1 in the softmax's denominator, value heads of a size of
their own); on the right a matrix memory with exponential gates (the mLSTM's: capped log gates, a running
maximum, a normaliser, a unit norm a head, a weight, a sigmoid gate).  "retention": a matrix memory
with a fixed decay a head, rotated queries and keys, a unit norm a head and a silu gate.  The
feed-forward is a mixture of silu-gated experts with a softmax router limited to the best groups.  The
head is the embedding table (without the embedding's factor) after the model's norm.  Tensor names:
`embed`, `final.norm`, and per layer i `l<i>.norm1`, `l<i>.norm2`, `l<i>.mix.*` (`.left.*` and `.right.*`
in a parallel mixer), `l<i>.mlp.router`, `l<i>.mlp.e<j>.{gate,up,down}`.
"""
from __future__ import annotations

from wllm_amd.architectures.lefisun_config import LefisunConfig
from wllm_amd.config.registry import register_architecture
from wllm_amd.parts.specs import (
    AttentionSpec,
    BlockSpec,
    EmbeddingSpec,
    HeadSpec,
    MatrixMemorySpec,
    MixtureOfExpertsSpec,
    ModelPlan,
    NormSpec,
    PositionSpec,
    ScheduleEntry,
    SideBySideSpec,
)

# the design names no longest sequence: a request is as long as the cache lets it be
NO_POSITION_LIMIT = 1 << 30
DEN_EPS = 1e-6              # what the matrix memory's denominator is raised by
ROUTER_EPS = 1e-20          # what the sum of the chosen experts' scores is raised by


def _position(rotation) -> PositionSpec:
    if rotation is None:
        return PositionSpec(kind="none")
    return PositionSpec(kind="rope", rotary_dim=rotation.dims, theta=rotation.base, pairing="half",
                        scaling_factor=rotation.scaling_factor)


def lefisun_plan(cfg: LefisunConfig) -> ModelPlan:
    def norm(name: str) -> NormSpec:
        return NormSpec(size=cfg.width, eps=cfg.norm_eps, weight=name, kind="rms")

    layers = []
    for i, layer in enumerate(cfg.layers):
        m, p = layer.mixer, f"l{i}.mix."
        if layer.type == "parallel":
            a, r = m.left, m.right
            left = AttentionSpec(
                hidden_size=cfg.width, num_heads=a.heads, num_kv_heads=a.kv_heads, head_dim=a.dim, value_dim=a.vdim,
                scale=a.scale, chunk=a.chunk, release_chunk=a.chunk, position=_position(a.rotation),
                q_weight=p + "left.q", k_weight=p + "left.k", v_weight=p + "left.v", o_weight=p + "left.o",
                q_bias=p + "left.q.b", k_bias=p + "left.k.b", v_bias=p + "left.v.b",
                q_norm_weight=p + "left.q.norm", k_norm_weight=p + "left.k.norm", band_norm_eps=cfg.norm_eps,
                bias_before_norm=True, sink=0.0, weights_in_float32=True, output_scale=m.left_scale)
            right = MatrixMemorySpec(
                hidden_size=cfg.width, num_heads=r.heads, head_dim=r.dim, value_dim=r.vdim, gating="exponential",
                gate_cap=r.gate_cap, den_eps=DEN_EPS, q_scale=r.dim ** -0.5, norm_eps=cfg.norm_eps,
                norm_weight=p + "right.norm", gate_activation="sigmoid", output_scale=m.right_scale,
                q_weight=p + "right.q", k_weight=p + "right.k", v_weight=p + "right.v", gate_weight=p + "right.g",
                o_weight=p + "right.o", i_weight=p + "right.i", i_bias=p + "right.i.b", f_weight=p + "right.f",
                f_bias=p + "right.f.b")
            mixer = SideBySideSpec(left=left, right=right)
        else:
            mixer = MatrixMemorySpec(
                hidden_size=cfg.width, num_heads=m.heads, head_dim=m.dim, value_dim=m.vdim, gating="decay",
                decays=m.decay, k_scale=m.dim ** -0.5, position=_position(m.rotation), norm_eps=cfg.norm_eps,
                gate_activation="silu", q_weight=p + "q", k_weight=p + "k", v_weight=p + "v", gate_weight=p + "g",
                o_weight=p + "o")
        q = f"l{i}."
        e = layer.mlp
        feed_forward = None
        if e is not None:
            feed_forward = MixtureOfExpertsSpec(
                hidden_size=cfg.width, intermediate_size=e.ff, num_experts=e.experts, top=e.top, num_groups=e.groups,
                keep_groups=e.keep, weight_eps=ROUTER_EPS, activation="silu", router_weight=q + "mlp.router",
                expert_prefix=q + "mlp.e")
        layers.append(BlockSpec(arrangement="pre_norm", mixer=mixer, feed_forward=feed_forward, mixer_norm=norm(q + "norm1"),
                                feed_forward_norm=norm(q + "norm2") if e is not None else None))
    return ModelPlan(
        embedding=EmbeddingSpec(vocab_size=cfg.vocab, hidden_size=cfg.width, weight="embed", scale=cfg.embedding_scale),
        layers=tuple(layers), schedule=tuple(ScheduleEntry(layer=i) for i in range(len(layers))),
        final_norm=norm("final.norm"), head=HeadSpec(vocab_size=cfg.vocab, hidden_size=cfg.width),
        max_positions=NO_POSITION_LIMIT,
        # a layer without a feed-forward does not need its second norm; a file may still carry it
        ignored_tensor_suffixes=tuple(f"l{i}.norm2" for i, layer in enumerate(cfg.layers) if layer.mlp is None))


register_architecture("Lefisun", LefisunConfig.from_dict, lefisun_plan)
