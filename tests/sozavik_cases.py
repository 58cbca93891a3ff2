"""Small Sozavik models for the tests: configurations as config.json mappings, random tensors that make every
mechanism count, and model folders.

The sizes differ from layer to layer and avoid coincidences (dim != vdim, heads / kv_heads of 1, 2 and 3, rot.dims
below dim, windows that are no multiple of a page, scales that are no power of dim, decays that differ from layer to
layer, a feed-forward as wide as nothing else, a layer without one, layers that mix values and one that does not)."""

from __future__ import annotations

from pathlib import Path

import torch

from tests.dafutar_cases import run_steps, tokens_of, write_folder as _write_folder  # noqa: F401  (generic helpers)

STRETCH = {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64}


def attention(heads=6, kv_heads=2, dim=24, vdim=40, window=13, scale=0.31, softcap=9.0, dims=10, scaling=STRETCH, base=500.0, v_mix=True):
    rot = {"base": base, "dims": dims}
    if scaling is not None:
        rot["scaling"] = dict(scaling)
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": window},
                                           "rot": rot, "scale": scale, "softcap": softcap, "v_mix": v_mix}}


def attention_2(heads=5, kv_heads=5, dim=40, vdim=16, window=21, scale=0.23, v_mix=True):
    return {"type": "attention_2", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": window},
                                             "scale": scale, "v_mix": v_mix}}


def lightning(heads=3, dim=16, vdim=24, decay=(0.7, 0.95, 0.995)):
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}}


def dense(ff=56):
    return {"kind": "dense", "ff": ff}


def config_of(layers, vocab=67, width=40, eps=1e-4, logit_softcap=7.5):
    """`layers`: [(mixer entry, mlp or None)]."""
    values = {"architecture": "Sozavik", "vocab": vocab, "width": width, "norm": {"eps": eps},
              "layers": [dict(mixer, mlp=mlp) for mixer, mlp in layers]}
    if logit_softcap is not None:
        values["logit_softcap"] = logit_softcap
    return values


# A model with every kind of layer, in an order of its own, and sizes that differ wherever they can.
MIXED = config_of(
    [
        (attention_2(heads=4, kv_heads=2, dim=24, vdim=40, window=9, scale=0.4), dense(24)),
        (lightning(heads=3, dim=16, vdim=24), dense(56)),
        (attention(heads=6, kv_heads=2, dim=24, vdim=40, window=13), None),
        (attention(heads=2, kv_heads=1, dim=40, vdim=8, window=30, dims=40, scaling=None, v_mix=False, softcap=3.0), dense(48)),
        (lightning(heads=2, dim=32, vdim=16, decay=(1.0, 0.5)), dense(16)),
        (attention_2(heads=5, kv_heads=5, dim=40, vdim=16, window=21), dense(72)),
    ]
)


def random_tensors(values: dict, seed: int, *, sharp: bool = False) -> dict[str, torch.Tensor]:
    """bfloat16 tensors (the precision model folders hold) by the model's own list of names and shapes.  Matrices are
    drawn so that activations stay of order one; norms, biases, sinks and blends are far enough from one and zero
    to matter.  `sharp`: queries and keys are large, so that a softmax looks at one key."""
    from llmserve_amd.registry import resolve_architecture

    architecture = resolve_architecture(values)
    spec = architecture.build_spec(architecture.config_class.from_dict(values))
    generator = torch.Generator().manual_seed(seed)
    tensors = {}
    for name, wanted in spec.tensors().items():
        shape = wanted.shape
        last = name.rsplit(".", 1)[-1]
        if name == "embed":
            value = torch.randn(shape, generator=generator)
        elif last == "vmix":
            value = 0.2 + 0.6 * torch.rand(shape, generator=generator)
        elif last == "sink":
            value = 1.5 * torch.randn(shape, generator=generator) + 1.0
        elif last == "b":
            value = 0.3 * torch.randn(shape, generator=generator)
        elif wanted.role == "norm":
            value = (2.5 if sharp and name.endswith((".q.norm", ".k.norm")) else 1.0) + 0.3 * torch.randn(shape, generator=generator)
        elif last == "g":
            value = 2.0 * torch.randn(shape, generator=generator) / shape[-1] ** 0.5
        else:
            value = 1.4 * torch.randn(shape, generator=generator) / shape[-1] ** 0.5
        tensors[name] = value.to(torch.bfloat16)
    return tensors


def write_folder(folder: Path, values: dict, seed: int = 1, *, sharp: bool = False, tensors: dict | None = None) -> Path:
    return _write_folder(folder, values, seed, tensors=tensors if tensors is not None else random_tensors(values, seed, sharp=sharp))
