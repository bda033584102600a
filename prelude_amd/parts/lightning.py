"""Linear attention with a decaying state ("lightning attention"): a mixer whose memory is of fixed size.

Per head, with q, k [dim] and v [vdim] passed through an activation (SiLU):

    S_t = a_h S_(t-1) + k_t v_t^T          S [dim, vdim], from zero at a request's start
    o_t = S_t^T q_t

and no other scale.  The heads' outputs side by side are brought to unit RMS together, scaled by a weight,
multiplied by sigmoid(W_g h) and projected.  S is 32-bit and lives in a state slot of the request
(``StateSpec``), carried from step to step; the decays a_h are the model's constants.  Queries, keys, values and
the gate come from one merged product.
"""
from __future__ import annotations

from typing import Sequence

import torch

from ..ops import kernels as K
from .base import MATRIX, NORM, Mixer, PartError, StateSpec, TensorReq, register_part


@register_part("mixer", "lightning_attention")
class LightningAttention(Mixer):
    LAUNCHES = 4   # merged projection, the recurrence, norm and gate, output projection
    GRAPH_SAFE_PORTIONS = True   # launches follow the step's shape alone; rows and state slots are read on the device

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, value_dim: int, decay: Sequence[float],
                 norm_eps: float, activation: str = "silu"):
        for name, v in (("hidden_size", hidden_size), ("num_heads", num_heads), ("head_dim", head_dim), ("value_dim", value_dim)):
            if int(v) <= 0:
                raise PartError(f"lightning_attention: {name} {v} must be positive")
        self.hidden_size, self.num_heads = int(hidden_size), int(num_heads)
        self.head_dim, self.value_dim = int(head_dim), int(value_dim)
        self.decay = tuple(float(a) for a in decay)
        if len(self.decay) != self.num_heads or not all(0.0 <= a <= 1.0 for a in self.decay):
            raise PartError(f"lightning_attention: {len(self.decay)} decays {self.decay} for {self.num_heads} heads; each "
                            f"must lie in [0, 1]")
        if self.head_dim > 256:
            raise PartError(f"lightning_attention: a key width of {self.head_dim} is more than the 256 the kernels take")
        if activation not in K.LIGHTNING_ACTIVATIONS:
            raise PartError(f"lightning_attention: activation {activation!r} is not known")
        self.norm_eps, self.activation = float(norm_eps), activation
        self.w_in = self.w_o = self.out_norm = self.decays = None

    def cache_spec(self):
        return StateSpec((("s", (self.num_heads, self.head_dim, self.value_dim), torch.float32),))

    def tensors(self):
        h, qk, vv = self.hidden_size, self.num_heads * self.head_dim, self.num_heads * self.value_dim
        return {"q": TensorReq((qk, h), MATRIX), "k": TensorReq((qk, h), MATRIX), "v": TensorReq((vv, h), MATRIX),
                "g": TensorReq((vv, h), MATRIX), "o": TensorReq((h, vv), MATRIX), "norm": TensorReq((vv,), NORM)}

    def load(self, tensors, dtype, device):
        # one product for queries, keys, values and the gate: rows [q | k | v | g]
        self.w_in = K.prepare_weight(torch.cat([tensors[n] for n in ("q", "k", "v", "g")], dim=0).contiguous())
        self.w_o = K.prepare_weight(tensors["o"])
        self.out_norm = tensors["norm"]
        self.decays = torch.tensor(self.decay, dtype=torch.float32, device=device)

    def forward(self, x, step, cache, write_cache=True):
        if not write_cache:
            raise PartError("lightning_attention: a run cannot read another run's state; every run keeps its own")
        nh, d, vd = self.num_heads, self.head_dim, self.value_dim
        qk, vv = nh * d, nh * vd
        p = K.linear(x, self.w_in)
        o = K.lightning_attention(p, 0, qk, 2 * qk, self.decays, cache.tensors["s"], step, nh, d, vd, self.activation)
        y = K.gated_rmsnorm(o.view(-1, vv), p[:, 2 * qk + vv:], self.out_norm, self.norm_eps)
        return K.linear(y, self.w_o, slices_ok=True)
