"""A plain, slow implementation of the Sozavik decoder, one function per mechanism, in float64 on the CPU.

It shares no code with the engine: it reads a model folder's config.json as a plain dict and its tensors by
name, and runs a whole sequence at once (no cache, no pages, no state slots).  The tests compare the engine
with it; `forward` also returns the residual stream after every layer.

Notation: W x means `x @ W.T` for a weight stored [out, in]; positions count from 0; n tokens.
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch

F = torch.float64


def read_folder(folder):
    from safetensors import safe_open

    folder = Path(folder)
    config = json.loads((folder / "config.json").read_text())
    tensors = {}
    with safe_open(str(folder / "model.safetensors"), framework="pt", device="cpu") as source:
        for name in source.keys():
            value = source.get_tensor(name)
            tensors[name] = value.to(F) if value.dtype.is_floating_point else value
    return config, tensors


# ---------------------------------------------------------------------------- small functions


def silu(z):
    return z * torch.sigmoid(z)


def rms_normalise(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def soft_cap(z, cap):
    return cap * torch.tanh(z / cap)


# ---------------------------------------------------------------------------- rotary


def stretched_frequencies(dims, base, scaling):
    """f_i = base^(-2i / dims); a frequency whose wavelength is short beside the original context stays, a long
    one is divided by `factor`, and between the two the two are blended by where the wavelength lies."""
    frequencies = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    if not scaling:
        return torch.tensor(frequencies, dtype=F)
    factor, low, high, original = (float(scaling[name]) for name in ("factor", "low", "high", "original"))
    out = []
    for f in frequencies:
        wavelength = 2.0 * math.pi / f
        if wavelength < original / high:
            out.append(f)
        elif wavelength > original / low:
            out.append(f / factor)
        else:
            s = (original / wavelength - low) / (high - low)
            out.append((1.0 - s) * f / factor + s * f)
    return torch.tensor(out, dtype=F)


def rotate_pairs(x, positions, frequencies):
    """x [n, heads, dim]: the first 2 len(frequencies) dimensions of every head turn in pairs (2i, 2i + 1)."""
    dims = 2 * len(frequencies)
    angles = positions.to(F)[:, None] * frequencies[None, :]  # [n, dims / 2]
    cos, sin = angles.cos()[:, None, :], angles.sin()[:, None, :]
    out = x.clone()
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


# ---------------------------------------------------------------------------- attention over a window


def window_attention(q, k, v, scale, window, cap=None, sinks=None):
    """q [n, H, d], k [n, G, d], v [n, G, dv] -> [n, H, dv].  Token i sees j with 0 <= i - j < window.  With
    `sinks` [H], each head's denominator has exp(sink) more, with no value to it."""
    n, heads, _ = q.shape
    share = heads // k.shape[1]
    out = torch.zeros((n, heads, v.shape[-1]), dtype=F)
    for h in range(heads):
        g = h // share
        for i in range(n):
            first = max(0, i - window + 1)
            scores = (k[first : i + 1, g] @ q[i, h]) * scale
            if cap is not None:
                scores = soft_cap(scores, cap)
            peak = scores.max() if sinks is None else torch.maximum(scores.max(), sinks[h])
            weights = torch.exp(scores - peak)
            total = weights.sum() + (torch.exp(sinks[h] - peak) if sinks is not None else 0.0)
            out[i, h] = (weights / total) @ v[first : i + 1, g]
    return out


def window_of(m, n):
    """The mask's size; a mixer without a mask sees every earlier token."""
    return m["mask"]["size"] if m.get("mask") else n


def mix_values(v, shared, tensors, prefix):
    """The first layer that mixes gives its values (a token's, all heads side by side) to the later ones: they take
    (1 - a) v + a v_first."""
    if "first" not in shared:
        shared["first"] = v.reshape(v.shape[0], -1)
        return v
    a = tensors[prefix + "vmix"]
    return (1.0 - a) * v + a * shared["first"].reshape(v.shape)


def attention_mixer(h, positions, m, tensors, prefix, eps, shared):
    """The mixer with per-head norms, part-rotated heads, capped scores, a sink a head and a gate a head."""
    n = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ tensors[prefix + "q"].T + tensors[prefix + "q.b"]).view(n, H, d)
    k = (h @ tensors[prefix + "k"].T + tensors[prefix + "k.b"]).view(n, G, d)
    v = (h @ tensors[prefix + "v"].T + tensors[prefix + "v.b"]).view(n, G, dv)
    q = rms_normalise(q, eps) * tensors[prefix + "q.norm"]
    k = rms_normalise(k, eps) * tensors[prefix + "k.norm"]
    rot = m["rot"]
    frequencies = stretched_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
    q, k = rotate_pairs(q, positions, frequencies), rotate_pairs(k, positions, frequencies)
    if m.get("v_mix"):
        v = mix_values(v, shared, tensors, prefix)
    mixed = window_attention(q, k, v, m["scale"], window_of(m, n), cap=m.get("softcap"), sinks=tensors[prefix + "sink"])
    gate = torch.sigmoid(h @ tensors[prefix + "g"].T)  # [n, H]
    mixed = mixed * gate[:, :, None]
    return mixed.reshape(n, H * dv) @ tensors[prefix + "o"].T


def attention_2_mixer(h, m, tensors, prefix, eps, shared):
    """The mixer whose queries and keys are normed as whole rows and carry no positions."""
    n = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms_normalise(h @ tensors[prefix + "q"].T, eps) * tensors[prefix + "q.norm"]
    k = rms_normalise(h @ tensors[prefix + "k"].T, eps) * tensors[prefix + "k.norm"]
    v = (h @ tensors[prefix + "v"].T).view(n, G, dv)
    if m.get("v_mix"):
        v = mix_values(v, shared, tensors, prefix)
    mixed = window_attention(q.view(n, H, d), k.view(n, G, d), v, m["scale"], window_of(m, n))
    return mixed.reshape(n, H * dv) @ tensors[prefix + "o"].T


# ---------------------------------------------------------------------------- the decaying state


def lightning_mixer(h, m, tensors, prefix, eps):
    """Per head a matrix S [d, dv] from zero: S <- decay S + k v^T, read out as S^T q, token by token."""
    n = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ tensors[prefix + "q"].T).view(n, H, d)
    k = silu(h @ tensors[prefix + "k"].T).view(n, H, d)
    v = silu(h @ tensors[prefix + "v"].T).view(n, H, dv)
    decay = torch.tensor(m["decay"], dtype=F)
    out = torch.zeros((n, H, dv), dtype=F)
    for head in range(H):
        S = torch.zeros((d, dv), dtype=F)
        for t in range(n):
            S = decay[head] * S + torch.outer(k[t, head], v[t, head])
            out[t, head] = S.T @ q[t, head]
    read = rms_normalise(out.reshape(n, H * dv), eps) * tensors[prefix + "norm"]
    read = read * torch.sigmoid(h @ tensors[prefix + "g"].T)
    return read @ tensors[prefix + "o"].T


# ---------------------------------------------------------------------------- feed-forward, the whole model


def dense_feed_forward(h, tensors, prefix):
    return (torch.relu(h @ tensors[prefix + "gate"].T) * (h @ tensors[prefix + "up"].T)) @ tensors[prefix + "down"].T


def forward(config, tensors, tokens):
    """(logits [n, vocab], the stream after every layer [layers, n, width]) of one sequence from position 0."""
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(len(tokens))
    eps = config["norm"]["eps"]
    x = tensors["embed"][tokens]
    shared: dict = {}
    streams = []
    for index, layer in enumerate(config["layers"]):
        prefix = f"l{index}."
        kind, m = layer["type"], layer["mixer"]
        if kind == "attention":
            mixed = attention_mixer(x, positions, m, tensors, prefix + "mix.", eps, shared)
        elif kind == "attention_2":
            mixed = attention_2_mixer(x, m, tensors, prefix + "mix.", eps, shared)
        elif kind == "lightning":
            mixed = lightning_mixer(x, m, tensors, prefix + "mix.", eps)
        else:
            raise ValueError(f"unknown layer type {kind!r}")
        x = x + rms_normalise(mixed, eps) * tensors[prefix + "norm1"]
        if layer.get("mlp") is not None:
            fed = dense_feed_forward(x, tensors, prefix + "mlp.")
            x = x + rms_normalise(fed, eps) * tensors[prefix + "norm2"]
        streams.append(x)
    logits = (rms_normalise(x, eps) * tensors["final.norm"]) @ tensors["head"].T
    if config.get("logit_softcap"):
        logits = soft_cap(logits, config["logit_softcap"])
    return logits, torch.stack(streams)
