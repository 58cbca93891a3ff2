"""A recurrent mixer: linear attention over a matrix state per head that fades by a fixed factor a token."""

from __future__ import annotations

from dataclasses import dataclass

import torch

from .attention import Mixer
from .base import MIXERS, FixedState, TensorSpec


@dataclass(frozen=True)
class DecayAttentionSpec:
    """`num_heads` heads with queries and keys of `dim` and values of `vdim`; `decays` one factor a head;
    `activation` on the three projections; `eps` of the norm over the heads' read-outs; `gate` squashes the gate."""

    hidden_size: int
    num_heads: int
    dim: int
    vdim: int
    decays: tuple[float, ...]
    eps: float
    activation: str = "silu"
    gate: str = "sigmoid"
    kind: str = "decay_attention"


@MIXERS.register("decay_attention")
class DecayAttention(Mixer):
    """q, k, v = act(W x) head by head; token by token, per head, with S [dim, vdim] from zero:

        S = decay S + k v^T;   o = S^T q

    then the heads' o side by side / their root mean square * norm * gate(W_g x), and W_o.  S, the decays, the
    scores q . k inside a run of tokens and the read-out are float32.  Per request the cache keeps S in a state slot
    that is zero when a request begins."""

    @classmethod
    def tensors(cls, spec: DecayAttentionSpec) -> dict[str, TensorSpec]:
        qk, v = spec.num_heads * spec.dim, spec.num_heads * spec.vdim
        return {
            "q": TensorSpec((qk, spec.hidden_size)),
            "k": TensorSpec((qk, spec.hidden_size)),
            "v": TensorSpec((v, spec.hidden_size)),
            "g": TensorSpec((v, spec.hidden_size)),
            "norm": TensorSpec((v,), role="norm"),
            "o": TensorSpec((spec.hidden_size, v)),
        }

    @classmethod
    def cache_need(cls, spec: DecayAttentionSpec) -> FixedState:
        return FixedState((spec.num_heads, spec.dim, spec.vdim))

    def __init__(self, spec: DecayAttentionSpec, tensors, kernels) -> None:
        super().__init__(spec, tensors, kernels)
        if len(spec.decays) != spec.num_heads:
            raise ValueError("decay attention: one decay a head")
        self.inputs = kernels.prepare_linear([tensors[name] for name in ("q", "k", "v", "g")], None)
        self.decays = kernels.to_device(torch.tensor(spec.decays, dtype=torch.float64).to(torch.float32))
        self.norm = tensors["norm"]
        self.out = kernels.prepare_linear([tensors["o"]], None)

    def forward(self, x: torch.Tensor, batch, cell) -> torch.Tensor:
        kernels, spec = self.kernels, self.spec
        qk, v = spec.num_heads * spec.dim, spec.num_heads * spec.vdim
        projected = kernels.linear(x, self.inputs)  # [T, q | k | v | g]
        read = kernels.decay_attention(
            projected, 0, qk, 2 * qk, spec.num_heads, spec.dim, spec.vdim, self.decays, spec.activation, batch, cell.state
        )  # float32 [T, heads * vdim]
        # one norm over all heads: a single "head" as wide as the row
        gated = kernels.gated_head_norm(read, projected, 2 * qk + v, self.norm, spec.eps, 1, v, spec.gate)
        return kernels.linear(gated, self.out, out_dtype=torch.float32, partial=True)
