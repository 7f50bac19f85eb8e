"""A matrix memory that fades by a constant a head (linear attention with a fixed decay).

q = silu(W_q h), k = silu(W_k h) (heads x key size), v = silu(W_v h) (heads x value size). Per head, with the state
S [key size, value size] zero at a request's start: S <- d_h S + k v^T, o = S^T q (the read-out sees the token's own
write; no other scale). The concatenated read-outs are RMS-normed together, times a plain weight and
sigmoid(W_g h), then W_o. One product makes [q | k | v | g]; the silu is applied in float as the scan reads its
operands; the state and the read-out are float, the state lives in the request's slot.
"""
from __future__ import annotations

from typing import Dict, List

import torch

from .. import kernels
from ..config.schema import MixerSpec
from ..weights import VECTOR, ParamDecl
from .base import LayerCache, StateNeed
from .registry import register_mixer


@register_mixer("decay_memory")
class DecayMemory:
    graph_safe = True       # the kernels read the step's shape from device arrays and leave state slot -1 alone

    @classmethod
    def declare_params(cls, spec: MixerSpec, prefix: str) -> List[ParamDecl]:
        p = spec.params
        nk, nv, w = p.heads * p.key_dim, p.heads * p.value_dim, spec.hidden
        return [ParamDecl(prefix + "q", (nk, w)), ParamDecl(prefix + "k", (nk, w)), ParamDecl(prefix + "v", (nv, w)),
                ParamDecl(prefix + "g", (nv, w)), ParamDecl(prefix + "o", (w, nv)),
                ParamDecl(prefix + "norm", (nv,), init="norm", role=VECTOR)]

    def __init__(self, spec: MixerSpec, weights: Dict[str, torch.Tensor], prefix: str, dtype: torch.dtype,
                 device: torch.device):
        p = spec.params
        if p is None:
            raise ValueError("decay_memory: the sizes come in MixerSpec.params (DecayMemorySpec)")
        if len(p.decays) != p.heads:
            raise ValueError(f"decay_memory: {len(p.decays)} decay factors for {p.heads} heads")
        self.spec, self.dtype = spec, dtype
        self.heads, self.key_dim, self.value_dim = int(p.heads), int(p.key_dim), int(p.value_dim)
        self.norm_eps = float(p.norm_eps)
        self.width = int(spec.hidden)
        self.w_in = torch.cat([weights[prefix + s] for s in ("q", "k", "v", "g")], dim=0).contiguous()
        self.w_o = weights[prefix + "o"]
        self.norm_weight = weights[prefix + "norm"].float().contiguous()
        self.decays = torch.tensor([float(d) for d in p.decays], dtype=torch.float32, device=device)
        self.state_floats = int(kernels.current().scan_state_floats("decay_memory", self.heads, self.key_dim,
                                                                    self.value_dim))

    def cache_need(self) -> StateNeed:
        return StateNeed((self.state_floats,), torch.float32)

    def forward(self, x, batch, cache: LayerCache):
        ops = kernels.current()
        T = x.shape[0]
        nk, nv = self.heads * self.key_dim, self.heads * self.value_dim
        proj = torch.empty((T, 2 * nk + 2 * nv), dtype=self.dtype, device=x.device)
        ops.linear(x, self.w_in, proj)
        read = torch.empty((T, nv), dtype=torch.float32, device=x.device)
        ops.decay_scan(proj, 0, nk, 2 * nk, self.decays, cache.state, batch, self.heads, self.key_dim, self.value_dim,
                       read)
        act = torch.empty((T, nv), dtype=self.dtype, device=x.device)
        # one norm over all heads' read-outs: a single "head" as wide as all of them
        ops.head_norm_gate(read, self.norm_weight, True, proj[:, 2 * nk + nv:], "sigmoid", self.norm_eps, 1, nv, act)
        out = torch.empty((T, self.width), dtype=torch.float32, device=x.device)     # enters a float sum as it is
        ops.linear(act, self.w_o, out)
        return out
