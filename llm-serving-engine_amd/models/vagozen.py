"""The Vagozen decoder as a list of parts: layers of window attention with kept first tokens, of retention or of
latent attention, each with a dense or a routed feed-forward (or none), a norm before and behind every sublayer
with a learned vector on what is added, a run of layers that is walked several times, and scaled logits from the
embedding's own table."""

from __future__ import annotations

from ..config.vagozen import (
    VagozenAttentionMixer,
    VagozenConfig,
    VagozenDenseMLP,
    VagozenExpertsMLP,
    VagozenLatentMixer,
    VagozenRetentionMixer,
)
from ..parts import (
    AddedPassSpec,
    DecayAttentionSpec,
    GatedMLPSpec,
    LatentAttentionSpec,
    LayerDefinition,
    LayerRun,
    ModelSpec,
    NamedPart,
    NormedAttentionSpec,
    RMSNormSpec,
    RoutedExpertsSpec,
    SandwichBlockSpec,
    YarnScaling,
)
from ..registry import register_architecture


def _yarn(rot) -> YarnScaling | None:
    return YarnScaling(*rot.scaling) if rot is not None and rot.scaling is not None else None


def _mixer_spec(config: VagozenConfig, mixer):
    if isinstance(mixer, VagozenAttentionMixer):
        rot = mixer.rot
        return NormedAttentionSpec(
            hidden_size=config.width, num_heads=mixer.heads, num_kv_heads=mixer.kv_heads, dim=mixer.dim, vdim=mixer.vdim,
            scale=mixer.scale, eps=config.norm_eps, window=mixer.window, bias=True, norm=None,
            rot_dims=rot.dims if rot is not None else 0, theta=rot.base if rot is not None else 10000.0, scaling=_yarn(rot),
            pairing="adjacent", keep_first=mixer.keep_first,
        )
    if isinstance(mixer, VagozenRetentionMixer):
        rot = mixer.rot
        return DecayAttentionSpec(
            hidden_size=config.width, num_heads=mixer.heads, dim=mixer.dim, vdim=mixer.vdim, decays=mixer.decay, eps=config.norm_eps,
            activation="none", gate="silu", norm="head", norm_weight=False, rot_dims=rot.dims if rot is not None else 0,
            theta=rot.base if rot is not None else 10000.0, pairing="half", key_scale=float(mixer.dim) ** -0.5,
        )
    assert isinstance(mixer, VagozenLatentMixer)
    return LatentAttentionSpec(
        hidden_size=config.width, num_heads=mixer.heads, dim=mixer.dim, rot_dim=mixer.rot_dim, vdim=mixer.vdim, q_rank=mixer.q_rank,
        kv_rank=mixer.kv_rank, scale=mixer.scale, eps=config.norm_eps, rot_dims=mixer.rot.dims, theta=mixer.rot.base, scaling=_yarn(mixer.rot),
    )


def _feed_forward_spec(config: VagozenConfig, mlp):
    if mlp is None:
        return None
    if isinstance(mlp, VagozenDenseMLP):
        return GatedMLPSpec(config.width, mlp.ff, "limited_swish", names=("gate", "up", "down"), limit=mlp.limit)
    assert isinstance(mlp, VagozenExpertsMLP)
    # a softmax over the chosen logits alone: the softmax over all of them, renormalised over the chosen
    return RoutedExpertsSpec(
        hidden_size=config.width, num_experts=mlp.experts, top=mlp.top, expert_size=mlp.expert_ff, route_scale=1.0,
        activation="limited_swish", scoring="softmax", gated=True, correction=False, renormalise=True, router_bias=True, limit=mlp.limit,
    )


def vagozen_spec(config: VagozenConfig) -> ModelSpec:
    norm = RMSNormSpec(config.width, config.norm_eps, weight_name="")
    layers, ignored = [], []
    for index, layer in enumerate(config.layers):
        feed_forward = _feed_forward_spec(config, layer.mlp)
        block = SandwichBlockSpec(
            norm, _mixer_spec(config, layer.mixer), norm, norm if feed_forward is not None else None, feed_forward,
            norm if feed_forward is not None else None,
            mixer_norm_name="norm1", mixer_out_norm_name="norm1b", feed_forward_norm_name="norm2", feed_forward_out_norm_name="norm2b",
        )
        layers.append(LayerDefinition(f"l{index}.", block))
        if feed_forward is None:  # a folder may still hold the norms and the vector of the feed-forward that is not there
            ignored += [f"l{index}.norm2", f"l{index}.norm2b", f"l{index}.ls2"]
    count = len(config.layers)
    loop = config.loop
    if loop is None:
        order = [LayerRun(index) for index in range(count)]
    else:
        order = [LayerRun(index) for index in range(loop.start)]
        for number in range(loop.times):
            order += [LayerRun(index, enters=number if index == loop.start else None) for index in range(loop.start, loop.stop)]
        order += [LayerRun(index) for index in range(loop.stop, count)]
    return ModelSpec(
        vocab_size=config.vocab,
        hidden_size=config.width,
        layers=tuple(layers),
        run_order=tuple(order),
        # logits = table . (norm(x) weight) * logit_scale: the constant rides on the last norm's weight
        final_norm=RMSNormSpec(config.width, config.norm_eps, weight_name="", weight_scale=config.logit_scale),
        tie_embeddings=True,
        embedding_name="embed",
        final_norm_name="final.norm",
        pass_entry=NamedPart("loop.", AddedPassSpec(config.width, loop.times)) if loop is not None else None,
        ignored_tensors=tuple(ignored),
    )


register_architecture("Vagozen", VagozenConfig, vagozen_spec)
