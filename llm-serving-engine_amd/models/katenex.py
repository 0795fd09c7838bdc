"""The Katenex decoder as a list of parts: several copies of the residual stream with learned reads and writes,
layers whose mixer is softmax attention beside a gated linear recurrence or the gated delta rule with a decay per
key channel, and a mixture of gated experts chosen within the best groups."""

from __future__ import annotations

from ..config.katenex import KatenexConfig, KatenexDeltaMixer, KatenexParallelMixer
from ..parts import (
    GatedDeltaSpec,
    GatedRecurrenceSpec,
    HyperBlockSpec,
    LayerDefinition,
    LayerRun,
    LinearScaling,
    ModelSpec,
    NamedPart,
    NormedAttentionSpec,
    ParallelMixersSpec,
    RMSNormSpec,
    RoutedExpertsSpec,
    StreamCopiesSpec,
    StreamNormSpec,
)
from ..registry import register_architecture


def _mixer_spec(config: KatenexConfig, mixer):
    if isinstance(mixer, KatenexParallelMixer):
        left, right = mixer.left, mixer.right
        attention = NormedAttentionSpec(
            hidden_size=config.width, num_heads=left.heads, num_kv_heads=left.kv_heads, dim=left.dim, vdim=left.vdim,
            scale=left.scale, eps=config.norm_eps, norm=None, pairing="half",
            rot_dims=left.rot.dims if left.rot is not None else 0, theta=left.rot.base if left.rot is not None else 10000.0,
            scaling=LinearScaling(left.rot.factor) if left.rot is not None and left.rot.factor is not None else None,
        )
        recurrence = GatedRecurrenceSpec(hidden_size=config.width, width=right.width, blocks=right.blocks, taps=right.conv, rate=8.0)
        return ParallelMixersSpec((("left.", attention, mixer.left_scale), ("right.", recurrence, mixer.right_scale)))
    assert isinstance(mixer, KatenexDeltaMixer)
    return GatedDeltaSpec(
        hidden_size=config.width, num_heads=mixer.heads, num_kv_heads=mixer.kv_heads, dim=mixer.dim, vdim=mixer.vdim,
        taps=mixer.conv, eps=config.norm_eps, decay="channel", decay_rank=mixer.decay_rank, gate_rank=mixer.gate_rank,
        gate_activation="sigmoid",
    )


def _feed_forward_spec(config: KatenexConfig, mlp):
    if mlp is None:
        return None
    return RoutedExpertsSpec(
        hidden_size=config.width, num_experts=mlp.experts, top=mlp.top, expert_size=mlp.expert_ff, route_scale=mlp.scale,
        activation="silu", scoring="softmax", shared_size=mlp.shared_ff, shared_activation="silu", gated=True, correction=False,
        groups=mlp.groups, keep_groups=mlp.keep, renormalise=True, shared_gate=False,
    )


def katenex_spec(config: KatenexConfig) -> ModelSpec:
    norm = RMSNormSpec(config.width, config.norm_eps, weight_name="")
    copies, learned = (config.streams, True) if config.streams is not None else (1, False)
    layers, ignored = [], []
    for index, layer in enumerate(config.layers):
        feed_forward = _feed_forward_spec(config, layer.mlp)
        block = HyperBlockSpec(copies, norm, _mixer_spec(config, layer.mixer), norm if feed_forward is not None else None, feed_forward,
                               learned_links=learned)
        layers.append(LayerDefinition(f"l{index}.", block))
        if feed_forward is None:  # a folder may still hold what belongs to the feed-forward that is not there
            ignored += [f"l{index}.norm2", f"l{index}.hc2.in", f"l{index}.hc2.out", f"l{index}.hc2.mix"]
    return ModelSpec(
        vocab_size=config.vocab,
        hidden_size=config.width,
        layers=tuple(layers),
        run_order=tuple(LayerRun(index) for index in range(len(layers))),
        final_norm=StreamNormSpec(config.width, config.norm_eps, copies, weight_name=""),
        tie_embeddings=False,
        embedding_name="embed",
        final_norm_name="final.norm",
        head_name="head",
        input_parts=(NamedPart("embedding.", StreamCopiesSpec(copies, config.embedding_scale)),),
        ignored_tensors=tuple(ignored),
    )


register_architecture("Katenex", KatenexConfig, katenex_spec)
