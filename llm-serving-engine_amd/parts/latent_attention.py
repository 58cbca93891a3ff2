"""Attention over a cached latent: keys and values of every head are products of one low-rank
vector per token, and only that vector and one rotated key part are kept in the cache."""

from __future__ import annotations

from dataclasses import dataclass

import torch

from .attention import Mixer
from .base import MIXERS, PagedKeyValue, TensorSpec
from .position import HeadLayout, YarnScaling, rotary_frequencies


@dataclass(frozen=True)
class LatentAttentionSpec:
    """Per head `dim` unrotated and `rot_dim` rotated query/key dimensions and `vdim` value dimensions.
    Queries come from a latent of `q_rank`, keys and values from one of `kv_rank`; the rotated key part
    is one vector for all heads.  Rotary turns the first `rot_dims` of the rotated part, in adjacent pairs."""

    hidden_size: int
    num_heads: int
    dim: int
    rot_dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    eps: float
    rot_dims: int
    theta: float
    scaling: YarnScaling | None = None
    kind: str = "latent_attention"


@MIXERS.register("latent_attention")
class LatentAttention(Mixer):
    """c_q = rmsnorm(W_dq x), q = W_uq c_q (head by head [dim | rot_dim]); W_dkv x = [c' | r], c = rmsnorm(c');
    head h's key is [W_uk,h c | rot(r)], its value W_uv,h c; softmax over the causal scores
    (q_nope . k_nope + rot(q_rot) . rot(r)) * scale; W_o on the heads' results.

    Since q_nope . (W_uk,h c) = (W_uk,h^T q_nope) . c and sum_j p_j W_uv,h c_j = W_uv,h sum_j p_j c_j, the
    attention runs in the latent space: every head asks with [W_uk,h^T q_nope | rot(q_rot)] for the one
    cached row [c | rot(r)] per token, which is key and value at once, and W_uv,h is applied to the
    head's weighted sum of latents.  That is attention with one kv head of size kv_rank + rot_dim, and
    the engine's paged attention kernels run it; the cache holds the row once as a key (in pieces, rows
    of a page side by side) and once as a value (transposed), as those kernels read them."""

    @classmethod
    def tensors(cls, spec: LatentAttentionSpec) -> dict[str, TensorSpec]:
        q_width = spec.num_heads * (spec.dim + spec.rot_dim)
        return {
            "dq": TensorSpec((spec.q_rank, spec.hidden_size)),
            "dq.norm": TensorSpec((spec.q_rank,), role="norm"),
            "uq": TensorSpec((q_width, spec.q_rank)),
            "dkv": TensorSpec((spec.kv_rank + spec.rot_dim, spec.hidden_size)),
            "dkv.norm": TensorSpec((spec.kv_rank,), role="norm"),
            "uk": TensorSpec((spec.num_heads * spec.dim, spec.kv_rank)),
            "uv": TensorSpec((spec.num_heads * spec.vdim, spec.kv_rank)),
            "o": TensorSpec((spec.hidden_size, spec.num_heads * spec.vdim)),
        }

    @classmethod
    def row_width(cls, spec: LatentAttentionSpec) -> int:
        return spec.kv_rank + spec.rot_dim

    @classmethod
    def cache_need(cls, spec: LatentAttentionSpec) -> PagedKeyValue:
        return PagedKeyValue(1, cls.row_width(spec), None)

    def __init__(self, spec: LatentAttentionSpec, tensors, kernels) -> None:
        super().__init__(spec, tensors, kernels)
        if spec.rot_dims > spec.rot_dim or spec.rot_dims % 2:
            raise ValueError("latent attention: the rotated dimensions are an even number within rot_dim")
        width = self.row_width(spec)
        self.layout = HeadLayout(spec.num_heads, 1, width)
        self.down = kernels.prepare_linear([tensors["dq"], tensors["dkv"]], None)
        self.q_norm, self.kv_norm = tensors["dq.norm"], tensors["dkv.norm"]
        self.up_q = kernels.prepare_linear([tensors["uq"]], None)
        # W_uk,h^T as the weight [kv_rank, dim] of head h's product over its unrotated query
        absorbed = tensors["uk"].view(spec.num_heads, spec.dim, spec.kv_rank).transpose(1, 2).contiguous()
        self.absorb = kernels.prepare_headwise_linear(absorbed)
        self.up_v = kernels.prepare_headwise_linear(tensors["uv"].view(spec.num_heads, spec.vdim, spec.kv_rank).contiguous())
        self.out = kernels.prepare_linear([tensors["o"]], None)
        shared = kernels.__dict__.setdefault("_rotary_frequencies", {})
        key = (spec.rot_dims, spec.theta, spec.scaling)
        if key not in shared:
            frequencies, magnitude = rotary_frequencies(spec.rot_dims, spec.theta, spec.scaling)
            shared[key] = (kernels.to_device(frequencies), magnitude)
        self.frequencies, self.magnitude = shared[key]

    def forward(self, x: torch.Tensor, batch, cell) -> torch.Tensor:
        kernels, spec = self.kernels, self.spec
        heads, width, per_head = spec.num_heads, self.layout.head_dim, spec.dim + spec.rot_dim
        down = kernels.linear(x, self.down)  # [T, q_rank | kv_rank | rot_dim]
        latent_q = kernels.rms_norm_columns(down, 0, self.q_norm, spec.eps)
        q = kernels.linear(latent_q, self.up_q)  # [T, heads * (dim | rot_dim)]
        table = kernels.rotary_table(batch, self.frequencies, self.magnitude)
        rows = kernels.new_rows(x.shape[0], self.layout.width)  # per token: the heads' queries, the key row, the value row
        # the key row and the value row: [c | rot(r)], twice
        kernels.rms_norm_columns(down, spec.q_rank, self.kv_norm, spec.eps, out=rows, out_first=heads * width, copies=2, copy_stride=width)
        kernels.rotate_columns(
            down, spec.q_rank + spec.kv_rank, 0, 2, spec.rot_dim, table, spec.rot_dims,
            out=rows, out_first=heads * width + spec.kv_rank, out_head_stride=width,
        )
        # the queries: [W_uk,h^T q_nope | rot(q_rot)]
        kernels.headwise_linear(q, 0, per_head, self.absorb, out=rows, out_first=0, out_head_stride=width)
        kernels.rotate_columns(q, spec.dim, per_head, heads, spec.rot_dim, table, spec.rot_dims, out=rows, out_first=spec.kv_rank, out_head_stride=width)
        mixed = kernels.rotate_store_attend(rows, self.layout, batch, cell, None, "none", spec.scale, None)  # [T, heads * width]
        values = kernels.headwise_linear(mixed, 0, width, self.up_v)  # [T, heads * vdim]
        return kernels.linear(values, self.out, out_dtype=torch.float32, partial=True)
