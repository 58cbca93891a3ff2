"""The typed configuration of the Dafutar decoder, read from its own config.json.

config.json gives every size and every constant that differs between models of the design: `vocab`, `width`,
`norm.eps`, `layers` (per layer its `type`, the `mixer`'s sizes and its `mlp`, or null for none) and `loop`
(layers `start` .. `stop - 1` run `times` times in a row).  Nothing here has a default but what may be absent.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, ClassVar

from .model import ArchitectureConfig, ConfigError, KeyReader


@dataclass(frozen=True)
class DafutarRotary:
    base: float
    dims: int
    scaling: tuple[float, float, float, float] | None  # factor, original, fast, slow


@dataclass(frozen=True)
class DafutarLatentMixer:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    rot: DafutarRotary


@dataclass(frozen=True)
class DafutarDeltaMixer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int


@dataclass(frozen=True)
class DafutarDenseMLP:
    ff: int


@dataclass(frozen=True)
class DafutarExpertsMLP:
    experts: int
    top: int
    scale: float
    expert_ff: int
    shared_ff: int | None


@dataclass(frozen=True)
class DafutarLayer:
    type: str  # "latent_attention" | "delta"
    mixer: DafutarLatentMixer | DafutarDeltaMixer
    mlp: DafutarDenseMLP | DafutarExpertsMLP | None


@dataclass(frozen=True)
class DafutarLoop:
    start: int
    stop: int
    times: int


def _mapping(value: Any, where: str) -> dict[str, Any]:
    if not isinstance(value, dict):
        raise ConfigError(f"{where} must be a mapping, got {value!r}")
    return value


def _read_mixer(kind: str, values: dict[str, Any], where: str):
    reader = KeyReader(values, where)
    if kind == "latent_attention":
        rot = KeyReader(_mapping(reader._get(("rot",), None) or {}, f"{where}.rot"), f"{where}.rot")
        found = rot.optional("scaling")
        scaling = None
        if found:
            scale_reader = KeyReader(_mapping(found, f"{where}.rot.scaling"), f"{where}.rot.scaling")
            scaling = tuple(scale_reader.number(name) for name in ("factor", "original", "fast", "slow"))
        rot_dim = reader.integer("rot_dim")
        rotary = DafutarRotary(rot.number("base"), rot.integer("dims", default=rot_dim, minimum=2), scaling)
        return DafutarLatentMixer(
            heads=reader.integer("heads"), dim=reader.integer("dim"), rot_dim=rot_dim, vdim=reader.integer("vdim"),
            q_rank=reader.integer("q_rank"), kv_rank=reader.integer("kv_rank"), scale=reader.number("scale"), rot=rotary,
        )
    if kind == "delta":
        heads = reader.integer("heads")
        return DafutarDeltaMixer(
            heads=heads, kv_heads=reader.integer("kv_heads", default=heads), dim=reader.integer("dim"),
            vdim=reader.integer("vdim"), conv=reader.integer("conv"),
        )
    raise ConfigError(f"{where}: unknown layer type {kind!r} (known: latent_attention, delta)")


def _read_mlp(values: Any, where: str):
    if values is None:
        return None
    reader = KeyReader(_mapping(values, where), where)
    kind = reader.choice("kind", choices=("dense", "moe"))
    if kind == "dense":
        return DafutarDenseMLP(reader.integer("ff"))
    router = KeyReader(_mapping(values.get("router"), f"{where}.router"), f"{where}.router")
    expert = KeyReader(_mapping(values.get("expert"), f"{where}.expert"), f"{where}.expert")
    shared = values.get("shared")
    shared_ff = KeyReader(_mapping(shared, f"{where}.shared"), f"{where}.shared").integer("ff") if shared else None
    return DafutarExpertsMLP(
        experts=router.integer("experts"), top=router.integer("top"), scale=router.number("scale"),
        expert_ff=expert.integer("ff"), shared_ff=shared_ff,
    )


@dataclass(frozen=True)
class DafutarConfig(ArchitectureConfig):
    architecture: ClassVar[str] = "Dafutar"

    vocab: int
    width: int
    norm_eps: float
    layers: tuple[DafutarLayer, ...]
    loop: DafutarLoop | None = None

    def __post_init__(self) -> None:
        if not self.layers:
            raise ConfigError("Dafutar config: no layers")
        for index, layer in enumerate(self.layers):
            if isinstance(layer.mixer, DafutarDeltaMixer) and layer.mixer.heads % layer.mixer.kv_heads:
                raise ConfigError(f"Dafutar config: layer {index}: heads must be a multiple of kv_heads")
            if isinstance(layer.mixer, DafutarLatentMixer) and (layer.mixer.rot.dims % 2 or layer.mixer.rot.dims > layer.mixer.rot_dim):
                raise ConfigError(f"Dafutar config: layer {index}: rot.dims must be even and at most rot_dim")
            if isinstance(layer.mlp, DafutarExpertsMLP) and layer.mlp.top > layer.mlp.experts:
                raise ConfigError(f"Dafutar config: layer {index}: more experts a token than there are")
        if self.loop is not None and not 0 <= self.loop.start < self.loop.stop <= len(self.layers):
            raise ConfigError("Dafutar config: loop must name layers start < stop within the model")

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    @classmethod
    def from_dict(cls, values: dict[str, Any]) -> "DafutarConfig":
        reader = KeyReader(values, "Dafutar config")
        norm = KeyReader(_mapping(values.get("norm"), "Dafutar config: norm"), "Dafutar config: norm")
        layers = []
        entries = values.get("layers")
        if not isinstance(entries, list):
            raise ConfigError("Dafutar config: 'layers' must be a list")
        for index, entry in enumerate(entries):
            where = f"Dafutar config: layers[{index}]"
            entry = _mapping(entry, where)
            kind = KeyReader(entry, where).choice("type", choices=("latent_attention", "delta"))
            mixer = _read_mixer(kind, _mapping(entry.get("mixer"), f"{where}.mixer"), f"{where}.mixer")
            layers.append(DafutarLayer(kind, mixer, _read_mlp(entry.get("mlp"), f"{where}.mlp")))
        loop = None
        if values.get("loop"):
            loop_reader = KeyReader(_mapping(values["loop"], "Dafutar config: loop"), "Dafutar config: loop")
            loop = DafutarLoop(loop_reader.integer("start", minimum=0), loop_reader.integer("stop"), loop_reader.integer("times"))
        return cls(vocab=reader.integer("vocab"), width=reader.integer("width"), norm_eps=norm.number("eps"), layers=tuple(layers), loop=loop)

    def to_config_json(self) -> dict[str, Any]:
        layers = []
        for layer in self.layers:
            mixer = layer.mixer
            if isinstance(mixer, DafutarLatentMixer):
                rot: dict[str, Any] = {"base": mixer.rot.base, "dims": mixer.rot.dims}
                if mixer.rot.scaling is not None:
                    rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), mixer.rot.scaling))
                described = {"heads": mixer.heads, "dim": mixer.dim, "rot_dim": mixer.rot_dim, "vdim": mixer.vdim,
                             "q_rank": mixer.q_rank, "kv_rank": mixer.kv_rank, "scale": mixer.scale, "rot": rot}
            else:
                described = {"heads": mixer.heads, "kv_heads": mixer.kv_heads, "dim": mixer.dim, "vdim": mixer.vdim, "conv": mixer.conv}
            mlp = layer.mlp
            if isinstance(mlp, DafutarDenseMLP):
                feed: Any = {"kind": "dense", "ff": mlp.ff}
            elif isinstance(mlp, DafutarExpertsMLP):
                feed = {"kind": "moe", "expert": {"ff": mlp.expert_ff}, "router": {"experts": mlp.experts, "top": mlp.top, "scale": mlp.scale}}
                if mlp.shared_ff is not None:
                    feed["shared"] = {"ff": mlp.shared_ff}
            else:
                feed = None
            layers.append({"type": layer.type, "mixer": described, "mlp": feed})
        values: dict[str, Any] = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                                  "norm": {"eps": self.norm_eps}, "layers": layers}
        if self.loop is not None:
            values["loop"] = {"start": self.loop.start, "stop": self.loop.stop, "times": self.loop.times}
        return values
