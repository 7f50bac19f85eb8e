"""A per-head matrix state whose decay depends on the input, one factor a key channel and token (RWKV-style
time mixing) as a token mixer.

With h the mixer's input row and h' the row of the token before (zeros for a request's first token), each of
r, k, v, g, w reads a mix of its own, m_s = h + (h' - h) * mu_s. Then r = W_r m_r, k = W_k m_k, v = W_v m_v
(heads x dim each), gate = silu(W_g m_g), and the decay

    w = exp(-exp(W_w2 tanh(W_w1 m_w) + w0))          one factor a head and key channel, in (0, 1).

Per head, with S [dim, dim] zero at a request's start and u a stored bonus a key channel:

    o_t = (S_{t-1} + diag(u) k_t v_t^T)^T r_t        the bonus for the current token alone
    S_t = diag(w_t) S_{t-1} + k_t v_t^T

Each head's o is divided by its root mean square, the heads side by side are multiplied by a weight and by the
gate, and W_o maps them back to the width. The five mixes are one kernel; the decay's pre-activation is a float
result of its product, and from there to the read-out's norm everything is float in either dtype. A request's
state slot holds S in the scan kernel's layout and, behind it, the last input row, so a prompt may be cut
anywhere.
"""
from __future__ import annotations

from typing import Dict, List

import torch

from .. import kernels
from ..config.schema import MixerSpec
from ..weights import VECTOR, ParamDecl
from .base import LayerCache, StateNeed
from .registry import register_mixer

_MIXES = ("r", "k", "v", "g", "w")


@register_mixer("wkv")
class WKV:
    graph_safe = True       # the kernels read the step's shape from device arrays and leave state slot -1 alone

    @classmethod
    def declare_params(cls, spec: MixerSpec, prefix: str) -> List[ParamDecl]:
        p = spec.params
        n, w = p.heads * p.dim, spec.hidden
        out = [ParamDecl(prefix + "mu." + s, (w,), role=VECTOR) for s in _MIXES]
        out += [ParamDecl(prefix + s, (n, w)) for s in ("r", "k", "v", "g")]
        out += [ParamDecl(prefix + "w1", (p.decay_rank, w)), ParamDecl(prefix + "w2", (n, p.decay_rank)),
                ParamDecl(prefix + "w0", (n,), init="zeros", role=VECTOR),
                ParamDecl(prefix + "u", (p.heads, p.dim), role=VECTOR),
                ParamDecl(prefix + "norm", (n,), init="norm", role=VECTOR),
                ParamDecl(prefix + "o", (w, n))]
        return out

    def __init__(self, spec: MixerSpec, weights: Dict[str, torch.Tensor], prefix: str, dtype: torch.dtype,
                 device: torch.device):
        p = spec.params
        if p is None:
            raise ValueError("wkv: the sizes come in MixerSpec.params (WKVSpec)")
        self.spec, self.dtype = spec, dtype
        self.heads, self.dim, self.decay_rank = int(p.heads), int(p.dim), int(p.decay_rank)
        self.norm_eps = float(p.norm_eps)
        self.width = int(spec.hidden)
        # the five mixing vectors as rows of one matrix, in the order of the mixes
        self.mu = torch.stack([weights[prefix + "mu." + s].to(dtype) for s in _MIXES], dim=0).contiguous()
        self.w_r, self.w_k, self.w_v, self.w_g = (weights[prefix + s] for s in ("r", "k", "v", "g"))
        self.w_1, self.w_2 = weights[prefix + "w1"], weights[prefix + "w2"]
        self.w0 = weights[prefix + "w0"].float().contiguous()
        self.u = weights[prefix + "u"].float().reshape(-1).contiguous()
        self.norm_weight = weights[prefix + "norm"].float().contiguous()
        self.w_o = weights[prefix + "o"]
        self.scan_floats = int(kernels.current().scan_state_floats("wkv", self.heads, self.dim, self.dim))
        self.state_floats = self.scan_floats + self.width

    def cache_need(self) -> StateNeed:
        return StateNeed((self.state_floats,), torch.float32)

    def forward(self, x, batch, cache: LayerCache):
        ops = kernels.current()
        T, w = x.shape
        n = self.heads * self.dim
        mixes = torch.empty((T, len(_MIXES) * w), dtype=self.dtype, device=x.device)
        ops.token_shift(x, self.mu, cache.state, self.scan_floats, batch, mixes)
        # [r | k | v | g]: four products, each over its own mix, side by side in one buffer
        proj = torch.empty((T, 4 * n), dtype=self.dtype, device=x.device)
        for j, wt in enumerate((self.w_r, self.w_k, self.w_v, self.w_g)):
            ops.linear(mixes[:, j * w:(j + 1) * w], wt, proj[:, j * n:(j + 1) * n])
        low = torch.empty((T, self.decay_rank), dtype=self.dtype, device=x.device)
        ops.linear(mixes[:, 4 * w:], self.w_1, low)
        ops.tanh_rows(low)
        decay = torch.empty((T, n), dtype=torch.float32, device=x.device)      # pre-activation, kept in float
        ops.linear(low, self.w_2, decay)
        read = torch.empty((T, n), dtype=torch.float32, device=x.device)
        ops.wkv_scan(proj, 0, n, 2 * n, decay, self.w0, self.u, cache.state, batch, self.heads, self.dim, read)
        act = torch.empty((T, n), dtype=self.dtype, device=x.device)
        ops.head_norm_gate(read, self.norm_weight, True, proj[:, 3 * n:], "silu", self.norm_eps, self.heads,
                           self.dim, act)
        out = torch.empty((T, self.width), dtype=self.dtype, device=x.device)
        ops.linear(act, self.w_o, out)
        return out
