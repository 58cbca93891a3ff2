"""The Dafutar decoder as a list of parts: layers of latent attention or of the gated delta rule, each with a
dense or a routed feed-forward (or none), layer norms, and a run of layers that is walked several times."""

from __future__ import annotations

from ..config.dafutar import DafutarConfig, DafutarDeltaMixer, DafutarDenseMLP, DafutarExpertsMLP, DafutarLatentMixer
from ..parts import (
    GatedDeltaSpec,
    GatedMLPSpec,
    JoinedPassSpec,
    LatentAttentionSpec,
    LayerDefinition,
    LayerNormSpec,
    LayerRun,
    ModelSpec,
    NamedPart,
    PreNormBlockSpec,
    RoutedExpertsSpec,
    YarnScaling,
)
from ..registry import register_architecture


def _mixer_spec(config: DafutarConfig, mixer):
    if isinstance(mixer, DafutarLatentMixer):
        return LatentAttentionSpec(
            hidden_size=config.width, num_heads=mixer.heads, dim=mixer.dim, rot_dim=mixer.rot_dim, vdim=mixer.vdim,
            q_rank=mixer.q_rank, kv_rank=mixer.kv_rank, scale=mixer.scale, eps=config.norm_eps,
            rot_dims=mixer.rot.dims, theta=mixer.rot.base,
            scaling=YarnScaling(*mixer.rot.scaling) if mixer.rot.scaling is not None else None,
        )
    assert isinstance(mixer, DafutarDeltaMixer)
    return GatedDeltaSpec(
        hidden_size=config.width, num_heads=mixer.heads, num_kv_heads=mixer.kv_heads, dim=mixer.dim, vdim=mixer.vdim,
        taps=mixer.conv, eps=config.norm_eps,
    )


def _feed_forward_spec(config: DafutarConfig, mlp):
    if mlp is None:
        return None
    if isinstance(mlp, DafutarDenseMLP):
        return GatedMLPSpec(config.width, mlp.ff, "gelu_tanh", names=("gate", "up", "down"))
    assert isinstance(mlp, DafutarExpertsMLP)
    return RoutedExpertsSpec(
        hidden_size=config.width, num_experts=mlp.experts, top=mlp.top, expert_size=mlp.expert_ff, route_scale=mlp.scale,
        activation="gelu", scoring="sigmoid", shared_size=mlp.shared_ff, shared_activation="gelu",
    )


def dafutar_spec(config: DafutarConfig) -> ModelSpec:
    norm = LayerNormSpec(config.width, config.norm_eps, weight_name="", bias_name=".b")
    layers, ignored = [], []
    for index, layer in enumerate(config.layers):
        feed_forward = _feed_forward_spec(config, layer.mlp)
        block = PreNormBlockSpec(
            norm, _mixer_spec(config, layer.mixer), norm if feed_forward is not None else None, feed_forward,
            mixer_norm_name="norm1", mixer_name="mix.", feed_forward_norm_name="norm2", feed_forward_name="mlp.",
        )
        layers.append(LayerDefinition(f"l{index}.", block))
        if feed_forward is None:  # a folder may still hold the norm of the feed-forward that is not there
            ignored += [f"l{index}.norm2", f"l{index}.norm2.b"]
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
        final_norm=norm,
        tie_embeddings=False,
        embedding_name="embed",
        final_norm_name="final.norm",
        head_name="head",
        pass_entry=NamedPart("loop.", JoinedPassSpec(config.width, loop.times)) if loop is not None else None,
        ignored_tensors=tuple(ignored),
    )


register_architecture("Dafutar", DafutarConfig, dafutar_spec)
