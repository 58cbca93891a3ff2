"""Small Dafutar models for the tests: configurations as config.json mappings, random tensors that make every
mechanism count, model folders, and helpers that run a schedule of steps through a runner.

The sizes differ from layer to layer and avoid coincidences (dim != vdim, heads / kv_heads of 1, 2 and 3, rot.dims
below rot_dim, convolutions of 2 to 5 taps, one to three experts a token, a layer without a feed-forward, a loop
that starts at the first layer or leaves layers behind it)."""

from __future__ import annotations

import json
from pathlib import Path

import torch

from llmserve_amd.engine import StepEntry
from llmserve_amd.weights import read_config


def latent(heads=3, dim=16, rot_dim=8, vdim=24, q_rank=20, kv_rank=24, scale=0.3, dims=None, scaling="yarn", base=10000.0):
    rot = {"base": base, "dims": rot_dim if dims is None else dims}
    if scaling == "yarn":
        rot["scaling"] = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}
    elif scaling is not None:
        rot["scaling"] = scaling
    return {"type": "latent_attention", "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank,
                                                   "kv_rank": kv_rank, "scale": scale, "rot": rot}}


def delta(heads=4, kv_heads=2, dim=16, vdim=24, conv=3):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}}


def dense(ff=40):
    return {"kind": "dense", "ff": ff}


def moe(experts=5, top=2, scale=1.25, ff=12, shared=20):
    found = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "scale": scale}}
    if shared is not None:
        found["shared"] = {"ff": shared}
    return found


def config_of(layers, loop=None, vocab=61, width=32, eps=1e-5):
    """`layers`: [(mixer entry, mlp or None)]."""
    values = {"architecture": "Dafutar", "vocab": vocab, "width": width, "norm": {"eps": eps},
              "layers": [dict(mixer, mlp=mlp) for mixer, mlp in layers]}
    if loop is not None:
        values["loop"] = dict(zip(("start", "stop", "times"), loop))
    return values


# A model with every kind of layer, a loop over the middle, and sizes that differ wherever they can.
MIXED = config_of(
    [
        (delta(heads=4, kv_heads=2, dim=16, vdim=24, conv=3), dense(40)),
        (latent(heads=3, dim=16, rot_dim=8, vdim=24, q_rank=20, kv_rank=24, dims=6), moe(5, 2, 1.25, 12, 20)),
        (delta(heads=3, kv_heads=3, dim=24, vdim=8, conv=2), moe(4, 3, 0.75, 8, None)),
        (latent(heads=2, dim=8, rot_dim=8, vdim=16, q_rank=12, kv_rank=40, scaling=None), None),
        (delta(heads=6, kv_heads=2, dim=8, vdim=16, conv=5), moe(3, 1, 2.0, 16, 8)),
    ],
    loop=(1, 4, 3),
)


def random_tensors(values: dict, seed: int, *, sharp: bool = False) -> dict[str, torch.Tensor]:
    """bfloat16 tensors (the precision model folders hold) by the model's own list of names and shapes.  Matrices
    are drawn so that activations stay of order one; norms, biases, decays and corrections are far enough from
    one and zero to matter.  `sharp`: decays near one (the state remembers far back)."""
    from llmserve_amd.registry import resolve_architecture

    architecture = resolve_architecture(values)
    spec = architecture.build_spec(architecture.config_class.from_dict(values))
    generator = torch.Generator().manual_seed(seed)
    tensors = {}
    for name, wanted in spec.tensors().items():
        shape = wanted.shape
        last = name.rsplit(".", 1)[-1]
        if name in ("embed",):
            value = torch.randn(shape, generator=generator)
        elif last == "A_log":
            value = torch.randn(shape, generator=generator) * 0.5 + (-5.0 if sharp else -1.0)
        elif last == "dt_bias":
            value = torch.randn(shape, generator=generator)
        elif last == "correction":
            value = 0.4 * torch.randn(shape, generator=generator)
        elif last == "conv":
            value = torch.randn(shape, generator=generator) / shape[1] ** 0.5
        elif name == "loop.step":
            value = 0.3 * torch.randn(shape, generator=generator)
        elif last == "b" and len(shape) == 1:  # a norm's bias
            value = 0.2 * torch.randn(shape, generator=generator)
        elif wanted.role == "norm":
            value = 1.0 + 0.3 * torch.randn(shape, generator=generator)
        elif last in ("router", "sg", "a"):
            value = 2.0 * torch.randn(shape, generator=generator) / shape[-1] ** 0.5
        else:
            value = 1.4 * torch.randn(shape, generator=generator) / shape[-1] ** 0.5
        tensors[name] = value.to(torch.bfloat16)
    return tensors


def write_folder(folder: Path, values: dict, seed: int = 1, *, sharp: bool = False, tensors: dict | None = None) -> Path:
    from safetensors.torch import save_file

    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(values, indent=1))
    tensors = tensors if tensors is not None else random_tensors(values, seed, sharp=sharp)
    save_file({name: value.contiguous() for name, value in tensors.items()}, str(folder / "model.safetensors"))
    read_config(folder)  # the folder is one the engine accepts
    return folder


def tokens_of(count: int, vocab: int, seed: int) -> list[int]:
    return torch.randint(0, vocab, (count,), generator=torch.Generator().manual_seed(seed)).tolist()


def run_steps(runner, steps, prompts, at: dict | None = None) -> dict[tuple[str, int], torch.Tensor]:
    """`steps`: [[(request, count)]]: each step gives every named request its next `count` tokens and wants the
    logits of all of them.  A request ends with its last token.  Returns {(request, position): logits}.  `at` (how
    far each request has come) may be the caller's, to go on over several calls."""
    at = {} if at is None else at
    for name in prompts:
        at.setdefault(name, 0)
    found = {}
    for step in steps:
        entries, rows, ended = [], [], []
        for name, count in step:
            first = at[name]
            entries.append(StepEntry(name, prompts[name][first : first + count], range(count)))
            rows += [(name, first + i) for i in range(count)]
            at[name] = first + count
            if at[name] == len(prompts[name]):
                ended.append(name)
        logits = runner.step(entries, create_missing=True).float().cpu()
        for row, key in enumerate(rows):
            found[key] = logits[row].clone()
        for name in ended:
            runner.end_request(name)
        runner.cache.check_invariants()
    return found
