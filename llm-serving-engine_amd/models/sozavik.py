"""The Sozavik decoder as a list of parts: layers whose norms act on the sublayers' results, with a mixer of
normed window attention (two kinds) or of decaying linear attention, a dense feed-forward, and capped logits."""

from __future__ import annotations

from ..config.sozavik import SozavikAttentionMixer, SozavikConfig, SozavikLightningMixer
from ..parts import (
    DecayAttentionSpec,
    GatedMLPSpec,
    LayerDefinition,
    LayerRun,
    ModelSpec,
    NamedPart,
    NormedAttentionSpec,
    OutputNormBlockSpec,
    RMSNormSpec,
    SoftCapSpec,
    WavelengthScaling,
)
from ..registry import register_architecture


def _mixer_spec(config: SozavikConfig, kind: str, mixer, values: str | None):
    if isinstance(mixer, SozavikLightningMixer):
        return DecayAttentionSpec(
            hidden_size=config.width, num_heads=mixer.heads, dim=mixer.dim, vdim=mixer.vdim, decays=mixer.decay, eps=config.norm_eps,
            activation="silu", gate="sigmoid",
        )
    assert isinstance(mixer, SozavikAttentionMixer)
    common = dict(
        hidden_size=config.width, num_heads=mixer.heads, num_kv_heads=mixer.kv_heads, dim=mixer.dim, vdim=mixer.vdim,
        scale=mixer.scale, eps=config.norm_eps, window=mixer.window, values=values, values_name="first",
    )
    if kind == "attention":
        rot = mixer.rot
        return NormedAttentionSpec(
            **common, bias=True, norm="head", rot_dims=rot.dims, theta=rot.base,
            scaling=WavelengthScaling(*rot.scaling) if rot.scaling is not None else None,
            soft_cap=mixer.softcap, sink=True, gate=True,
        )
    return NormedAttentionSpec(**common, bias=False, norm="row")


def sozavik_spec(config: SozavikConfig) -> ModelSpec:
    norm = RMSNormSpec(config.width, config.norm_eps, weight_name="")
    layers, ignored = [], []
    given = False  # whether an earlier layer gives its values to the layers that mix
    for index, layer in enumerate(config.layers):
        values = None
        if isinstance(layer.mixer, SozavikAttentionMixer):
            if layer.mixer.v_mix:
                values, given = ("take" if given else "give"), True
            else:
                ignored.append(f"l{index}.mix.vmix")
        feed_forward = GatedMLPSpec(config.width, layer.mlp.ff, "relu", names=("gate", "up", "down")) if layer.mlp is not None else None
        block = OutputNormBlockSpec(
            norm, _mixer_spec(config, layer.type, layer.mixer, values), norm if feed_forward is not None else None, feed_forward,
            mixer_norm_name="norm1", mixer_name="mix.", feed_forward_norm_name="norm2", feed_forward_name="mlp.",
        )
        layers.append(LayerDefinition(f"l{index}.", block))
        if feed_forward is None:
            ignored.append(f"l{index}.norm2")
    return ModelSpec(
        vocab_size=config.vocab,
        hidden_size=config.width,
        layers=tuple(layers),
        run_order=tuple(LayerRun(index) for index in range(len(layers))),
        final_norm=norm,
        tie_embeddings=False,
        embedding_name="embed",
        final_norm_name="final.norm",
        head_name="head",
        output_parts=(NamedPart("", SoftCapSpec(config.logit_softcap)),) if config.logit_softcap is not None else (),
        ignored_tensors=tuple(ignored),
    )


register_architecture("Sozavik", SozavikConfig, sozavik_spec)
