"""A plain, slow implementation of the Dafutar decoder, one function per mechanism, in float64 on the CPU.

It shares no code with the engine: it reads a model folder's config.json as a plain dict and its tensors by
name, and runs a whole sequence at once (no cache, no pages, no state slots).  The tests compare the engine
with it; `forward` also returns the residual stream after every layer run.

Notation: W x means `x @ W.T` for a weight stored [out, in]; positions count from 0.
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


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z**3)))


def gelu_erf(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def silu(z):
    return z * torch.sigmoid(z)


def rms_normalise(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def layer_norm(x, weight, bias, eps):
    mean = x.mean(-1, keepdim=True)
    variance = ((x - mean) ** 2).mean(-1, keepdim=True)
    return (x - mean) / torch.sqrt(variance + eps) * weight + bias


# ---------------------------------------------------------------------------- rotary with YaRN


def rotary_frequencies(dims, base, scaling=None):
    """(frequencies [dims / 2], magnitude).  With scaling: the dimension index at which a wavelength of
    `original / t` turns is d(t) = dims ln(original / (2 pi t)) / (2 ln base); pairs below d(fast) keep
    their frequency, pairs above d(slow) have it divided by `factor`, a linear ramp between."""
    index = torch.arange(dims // 2, dtype=F)
    plain = base ** (-2.0 * index / dims)
    if not scaling:
        return plain, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def turn(t):
        return dims * math.log(original / (2.0 * math.pi * t)) / (2.0 * math.log(base))

    low = max(math.floor(turn(float(scaling["fast"]))), 0)
    high = min(math.ceil(turn(float(scaling["slow"]))), dims - 1)
    ramp = ((index - low) / max(high - low, 0.001)).clamp(0.0, 1.0)
    return plain / factor * ramp + plain * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_interleaved(x, positions, frequencies, magnitude, dims):
    """x [T, ..., width]: pairs (2i, 2i+1) of the first `dims` columns turn by positions * frequencies[i];
    the other columns pass."""
    shape = [len(positions)] + [1] * (x.dim() - 2) + [dims // 2]
    angles = positions.to(F).view(-1, *[1] * (x.dim() - 1)) * frequencies.view(*[1] * (x.dim() - 1), -1)
    cos, sin = (angles.cos() * magnitude).view(shape), (angles.sin() * magnitude).view(shape)
    out = x.clone()
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


# ---------------------------------------------------------------------------- mixers


def latent_attention(h, w, m, eps, positions):
    """h [T, width]; w: the mixer's tensors by their short names; m: the mixer's config."""
    heads, dim, rot_dim, vdim, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    T = h.shape[0]
    latent_q = rms_normalise(h @ w["dq"].T, eps) * w["dq.norm"]
    q = (latent_q @ w["uq"].T).view(T, heads, dim + rot_dim)
    down = h @ w["dkv"].T
    latent = rms_normalise(down[:, :rank], eps) * w["dkv.norm"]
    shared_key = down[:, rank:]  # [T, rot_dim], one for all heads
    rot = m["rot"]
    frequencies, magnitude = rotary_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
    q_rot = rotate_interleaved(q[..., dim:], positions, frequencies, magnitude, rot["dims"])
    k_rot = rotate_interleaved(shared_key, positions, frequencies, magnitude, rot["dims"])
    keys = (latent @ w["uk"].T).view(T, heads, dim)
    values = (latent @ w["uv"].T).view(T, heads, vdim)
    scores = torch.einsum("thd,shd->hts", q[..., :dim], keys) + torch.einsum("thr,sr->hts", q_rot, k_rot)
    scores = scores * m["scale"]
    visible = positions.view(-1, 1) >= positions.view(1, -1)
    scores = scores.masked_fill(~visible, float("-inf"))
    weights = torch.softmax(scores, dim=-1)
    mixed = torch.einsum("hts,shv->thv", weights, values).reshape(T, heads * vdim)
    return mixed @ w["o"].T


def short_convolution(x, taps_weight):
    """x [T, channels], taps_weight [channels, taps], the last column the current token's; zeros before the start."""
    T, taps = x.shape[0], taps_weight.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, x.shape[1], dtype=x.dtype), x])
    out = torch.zeros_like(x)
    for j in range(taps):
        out += padded[j : j + T] * taps_weight[:, j]
    return out


def gated_delta(h, w, m, eps):
    heads, kv_heads, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = silu(short_convolution(h @ w["q"].T, w["q.conv"])).view(T, kv_heads, dim)
    k = silu(short_convolution(h @ w["k"].T, w["k.conv"])).view(T, kv_heads, dim)
    v = silu(short_convolution(h @ w["v"].T, w["v.conv"])).view(T, heads, vdim)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dim**-0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w["b"].T)  # [T, heads]
    decay = torch.exp(-torch.exp(w["A_log"]) * torch.nn.functional.softplus(h @ w["a"].T + w["dt_bias"]))
    group = heads // kv_heads
    state = torch.zeros(heads, dim, vdim, dtype=F)
    out = torch.zeros(T, heads, vdim, dtype=F)
    for t in range(T):
        for head in range(heads):
            kt, qt = k[t, head // group], q[t, head // group]
            S = state[head] * decay[t, head]
            u = beta[t, head] * (v[t, head] - S.T @ kt)
            S = S + torch.outer(kt, u)
            out[t, head] = S.T @ qt
            state[head] = S
    out = rms_normalise(out, eps) * w["norm"]
    gate = silu(h @ w["g"].T).view(T, heads, vdim)
    return (out * gate).reshape(T, heads * vdim) @ w["o"].T


# ---------------------------------------------------------------------------- feed-forwards


def dense_feed_forward(h, w):
    return (gelu_tanh(h @ w["gate"].T) * (h @ w["up"].T)) @ w["down"].T


def small_expert(h, up, down):
    return gelu_erf(h @ up.T) @ down.T


def routed_feed_forward(h, w, m):
    router = m["router"]
    scores = torch.sigmoid(h @ w["router"].T)  # [T, experts]
    chosen = torch.topk(scores + w["correction"], router["top"], dim=-1).indices
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e in chosen[t].tolist():
            out[t] += router["scale"] * scores[t, e] * small_expert(h[t], w[f"e{e}.up"], w[f"e{e}.down"])
    if m.get("shared"):
        out = out + torch.sigmoid(h @ w["shared.sg"].T) * small_expert(h, w["shared.up"], w["shared.down"])
    return out


# ---------------------------------------------------------------------------- the model


def below(tensors, prefix):
    return {name[len(prefix):]: value for name, value in tensors.items() if name.startswith(prefix)}


def run_order(config):
    """[(layer, number of the pass or None, first of its pass)]"""
    count = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return [(i, None, False) for i in range(count)]
    order = [(i, None, False) for i in range(loop["start"])]
    for t in range(loop["times"]):
        order += [(i, t, i == loop["start"]) for i in range(loop["start"], loop["stop"])]
    return order + [(i, None, False) for i in range(loop["stop"], count)]


def forward(config, tensors, tokens, positions=None):
    """(logits [T, vocab], the residual stream after every layer run [runs, T, width]), float64."""
    eps = config["norm"]["eps"]
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(len(tokens)) if positions is None else positions
    x = tensors["embed"][tokens]
    embedded = x.clone()
    streams = []
    for layer, pass_number, enters in run_order(config):
        if enters:
            x = torch.cat([x, embedded], dim=-1) @ tensors["loop.in"].T + tensors["loop.step"][pass_number]
        entry, prefix = config["layers"][layer], f"l{layer}."
        h = layer_norm(x, tensors[prefix + "norm1"], tensors[prefix + "norm1.b"], eps)
        mix = below(tensors, prefix + "mix.")
        if entry["type"] == "latent_attention":
            x = x + latent_attention(h, mix, entry["mixer"], eps, positions)
        elif entry["type"] == "delta":
            x = x + gated_delta(h, mix, entry["mixer"], eps)
        else:
            raise ValueError(entry["type"])
        if entry.get("mlp"):
            h = layer_norm(x, tensors[prefix + "norm2"], tensors[prefix + "norm2.b"], eps)
            mlp = below(tensors, prefix + "mlp.")
            x = x + (dense_feed_forward(h, mlp) if entry["mlp"]["kind"] == "dense" else routed_feed_forward(h, mlp, entry["mlp"]))
        streams.append(x.clone())
    x = layer_norm(x, tensors["final.norm"], tensors["final.norm.b"], eps)
    return x @ tensors["head"].T, torch.stack(streams)
