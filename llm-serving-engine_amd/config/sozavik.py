"""The typed configuration of the Sozavik decoder, read from its own config.json.

config.json gives every size and every constant that differs between models of the design: `vocab`, `width`,
`norm.eps`, `logit_softcap` and `layers` (per layer its `type`, the `mixer`'s sizes and constants and its `mlp`, or
null for none).  Nothing here has a default but what may be absent.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, ClassVar

from .model import ArchitectureConfig, ConfigError, KeyReader

LAYER_TYPES = ("attention", "attention_2", "lightning")


@dataclass(frozen=True)
class SozavikRotary:
    base: float
    dims: int
    scaling: tuple[float, float, float, float] | None  # factor, low, high, original


@dataclass(frozen=True)
class SozavikAttentionMixer:
    """`type` "attention": biased projections, a norm per head, part-rotated heads, capped scores, a sink and a gate a
    head.  `type` "attention_2": no biases, norms over the whole projections, no positions, plain scores."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int | None
    v_mix: bool
    softcap: float | None = None
    rot: SozavikRotary | None = None


@dataclass(frozen=True)
class SozavikLightningMixer:
    heads: int
    dim: int
    vdim: int
    decay: tuple[float, ...]


@dataclass(frozen=True)
class SozavikDenseMLP:
    ff: int


@dataclass(frozen=True)
class SozavikLayer:
    type: str
    mixer: SozavikAttentionMixer | SozavikLightningMixer
    mlp: SozavikDenseMLP | None


def _mapping(value: Any, where: str) -> dict[str, Any]:
    if not isinstance(value, dict):
        raise ConfigError(f"{where} must be a mapping, got {value!r}")
    return value


def _read_mixer(kind: str, values: dict[str, Any], where: str):
    reader = KeyReader(values, where)
    if kind == "lightning":
        heads = reader.integer("heads")
        decay = values.get("decay")
        if isinstance(decay, (int, float)) and not isinstance(decay, bool):  # one number for all heads
            decay = [decay] * heads
        if not isinstance(decay, list) or len(decay) != heads or any(isinstance(d, bool) or not isinstance(d, (int, float)) for d in decay):
            raise ConfigError(f"{where}: 'decay' must list one number a head")
        return SozavikLightningMixer(heads=heads, dim=reader.integer("dim"), vdim=reader.integer("vdim"), decay=tuple(float(d) for d in decay))
    heads = reader.integer("heads")
    window = None  # (no mask: every earlier token is seen)
    if values.get("mask") is not None:
        window = KeyReader(_mapping(values["mask"], f"{where}.mask"), f"{where}.mask").integer("size")
    rot, softcap = None, None
    if kind == "attention":
        found = KeyReader(_mapping(values.get("rot"), f"{where}.rot"), f"{where}.rot")
        scaling = None
        if found.optional("scaling"):
            scale_reader = KeyReader(_mapping(values["rot"]["scaling"], f"{where}.rot.scaling"), f"{where}.rot.scaling")
            scaling = tuple(scale_reader.number(name) for name in ("factor", "low", "high", "original"))
        rot = SozavikRotary(found.number("base"), found.integer("dims", minimum=2), scaling)
        softcap = reader.number("softcap") if reader.optional("softcap") is not None else None
    return SozavikAttentionMixer(
        heads=heads, kv_heads=reader.integer("kv_heads", default=heads), dim=reader.integer("dim"), vdim=reader.integer("vdim"),
        scale=reader.number("scale"), window=window, v_mix=reader.boolean("v_mix", default=False), softcap=softcap, rot=rot,
    )


def _read_mlp(values: Any, where: str):
    if values is None:
        return None
    reader = KeyReader(_mapping(values, where), where)
    reader.choice("kind", choices=("dense",))
    return SozavikDenseMLP(reader.integer("ff"))


@dataclass(frozen=True)
class SozavikConfig(ArchitectureConfig):
    architecture: ClassVar[str] = "Sozavik"

    vocab: int
    width: int
    norm_eps: float
    layers: tuple[SozavikLayer, ...]
    logit_softcap: float | None = None

    def __post_init__(self) -> None:
        if not self.layers:
            raise ConfigError("Sozavik config: no layers")
        shared = None
        for index, layer in enumerate(self.layers):
            mixer, where = layer.mixer, f"Sozavik config: layer {index}"
            if isinstance(mixer, SozavikLightningMixer):
                if any(not 0.0 < d <= 1.0 for d in mixer.decay):
                    raise ConfigError(f"{where}: a decay lies in (0, 1]")
                continue
            if mixer.heads % mixer.kv_heads:
                raise ConfigError(f"{where}: heads must be a multiple of kv_heads")
            if mixer.rot is not None and (mixer.rot.dims % 2 or mixer.rot.dims > mixer.dim):
                raise ConfigError(f"{where}: rot.dims must be even and at most dim")
            if mixer.softcap is not None and not mixer.softcap > 0:
                raise ConfigError(f"{where}: softcap must be positive")
            if mixer.v_mix:
                if shared is not None and shared != mixer.kv_heads * mixer.vdim:
                    raise ConfigError(f"{where}: layers that mix values have values of one size")
                shared = mixer.kv_heads * mixer.vdim
        if self.logit_softcap is not None and not self.logit_softcap > 0:
            raise ConfigError("Sozavik config: logit_softcap must be positive")

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    @classmethod
    def from_dict(cls, values: dict[str, Any]) -> "SozavikConfig":
        reader = KeyReader(values, "Sozavik config")
        norm = KeyReader(_mapping(values.get("norm"), "Sozavik config: norm"), "Sozavik config: norm")
        entries = values.get("layers")
        if not isinstance(entries, list):
            raise ConfigError("Sozavik config: 'layers' must be a list")
        layers = []
        for index, entry in enumerate(entries):
            where = f"Sozavik config: layers[{index}]"
            entry = _mapping(entry, where)
            kind = KeyReader(entry, where).choice("type", choices=LAYER_TYPES)
            mixer = _read_mixer(kind, _mapping(entry.get("mixer"), f"{where}.mixer"), f"{where}.mixer")
            layers.append(SozavikLayer(kind, mixer, _read_mlp(entry.get("mlp"), f"{where}.mlp")))
        cap = reader.number("logit_softcap") if reader.optional("logit_softcap") is not None else None
        return cls(
            vocab=reader.integer("vocab"), width=reader.integer("width"), norm_eps=norm.number("eps"), layers=tuple(layers),
            logit_softcap=cap if cap else None,
        )

    def to_config_json(self) -> dict[str, Any]:
        layers = []
        for layer in self.layers:
            mixer = layer.mixer
            if isinstance(mixer, SozavikLightningMixer):
                described: dict[str, Any] = {"heads": mixer.heads, "dim": mixer.dim, "vdim": mixer.vdim, "decay": list(mixer.decay)}
            else:
                described = {"heads": mixer.heads, "kv_heads": mixer.kv_heads, "dim": mixer.dim, "vdim": mixer.vdim,
                             "scale": mixer.scale, "v_mix": mixer.v_mix}
                if mixer.window is not None:
                    described["mask"] = {"size": mixer.window}
                if mixer.rot is not None:
                    rot: dict[str, Any] = {"base": mixer.rot.base, "dims": mixer.rot.dims}
                    if mixer.rot.scaling is not None:
                        rot["scaling"] = dict(zip(("factor", "low", "high", "original"), mixer.rot.scaling))
                    described["rot"] = rot
                if mixer.softcap is not None:
                    described["softcap"] = mixer.softcap
            feed = {"kind": "dense", "ff": layer.mlp.ff} if layer.mlp is not None else None
            layers.append({"type": layer.type, "mixer": described, "mlp": feed})
        values: dict[str, Any] = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                                  "norm": {"eps": self.norm_eps}, "layers": layers}
        if self.logit_softcap is not None:
            values["logit_softcap"] = self.logit_softcap
        return values
