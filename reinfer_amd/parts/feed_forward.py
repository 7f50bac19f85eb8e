"""Dense SwiGLU feed-forward: down( silu(gate(x)) * up(x) ), no bias.

crates/cuda/src/engine.rs:4288-4303; silu(g) = g / (1 + exp(-g))
(crates/cuda/kernels/dense_kernels.cu:202-213). gate and up are one product:
their rows are interleaved in runs of 8 at load (8 gate rows, the 8 up rows of
the same features, ...), so that for few tokens the product's epilogue applies
the gate itself and for many the gate kernel reads both from one cache line.
A width that is no multiple of 8 keeps [gate; up] and the separate gate kernel.
The option ``act`` names another gate activation ("gelu_tanh": 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)));
"swish_bounded" with the option ``limit``: g <- min(gate, limit), u <- clamp(up, -limit, limit),
g sigmoid(1.702 g) (u + 1)); it is applied by the gate kernel behind the product.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import kernels
from ..config.schema import FeedForwardSpec
from ..weights import ParamDecl
from .base import NormTarget, split_input
from .registry import register_feed_forward


@register_feed_forward("swiglu")
class SwiGLU:
    graph_safe = True       # no host-side state: a decode step with it can be captured
    adds_in_place = True    # forward(..., resid=) may add the down projection into the stream
    takes_row_scaled = True     # x may be RowScaled: the gate/up product applies the row factor
    emits_for_norm = True       # forward(..., emit=) may fill a NormTarget from the down projection
    adds_scaled = True          # forward(..., resid=, resid_scale=) adds resid_scale times the result

    @staticmethod
    def _names(spec: FeedForwardSpec):
        """Tensor names of gate, up and down behind the prefix (the option ``names`` where they differ)."""
        return tuple(dict(spec.extra).get("names", ("gate_proj.weight", "up_proj.weight", "down_proj.weight")))

    @classmethod
    def declare_params(cls, spec: FeedForwardSpec, prefix: str) -> List[ParamDecl]:
        g, u, d = cls._names(spec)
        return [ParamDecl(prefix + g, (spec.intermediate, spec.hidden)),
                ParamDecl(prefix + u, (spec.intermediate, spec.hidden)),
                ParamDecl(prefix + d, (spec.hidden, spec.intermediate))]

    def __init__(self, spec: FeedForwardSpec, weights: Dict[str, torch.Tensor], prefix: str,
                 dtype: torch.dtype, device: torch.device):
        self.spec = spec
        self.dtype = dtype
        gn, un, dn = self._names(spec)
        gate, up = weights[prefix + gn], weights[prefix + un]
        I, h = spec.intermediate, spec.hidden
        self.group = getattr(kernels.current(), "GATE_GROUP", 0)
        if self.group and I % self.group == 0:
            g = self.group
            self.w_gate_up = torch.stack([gate.view(I // g, g, h), up.view(I // g, g, h)], dim=1) \
                .reshape(2 * I, h).contiguous()
        else:
            self.group = 0
            self.w_gate_up = torch.cat([gate, up], dim=0).contiguous()
        self.w_down = weights[prefix + dn]
        self.act = str(dict(spec.extra).get("act", "silu"))
        if self.act not in ("silu", "gelu_tanh", "swish_bounded"):
            raise ValueError(f"swiglu: gate activation {self.act!r}; built: silu, gelu_tanh, swish_bounded")
        self.limit = float(dict(spec.extra).get("limit", 0.0))
        if self.act == "swish_bounded" and not self.limit > 0.0:
            raise ValueError("swiglu: the bounded activation needs a positive limit")

    def forward(self, x, batch, resid: Optional[torch.Tensor] = None, emit: Optional[NormTarget] = None,
                resid_scale: float = 1.0):
        ops = kernels.current()
        x, row_sums = split_input(x)
        T = x.shape[0]
        I = self.spec.intermediate
        act = torch.empty((T, I), dtype=self.dtype, device=x.device)
        if self.act != "silu":
            # the products' gated epilogue is silu: another activation runs as the gate kernel
            gu = torch.empty((T, 2 * I), dtype=self.dtype, device=x.device)
            if row_sums is None:
                ops.linear(x, self.w_gate_up, gu)
            else:
                ops.linear_skinny(x, self.w_gate_up, gu, row_sums=row_sums)
            if self.act == "swish_bounded":
                ops.silu_mul(gu, act, self.group, act=self.act, limit=self.limit)
            else:
                ops.silu_mul(gu, act, self.group, act=self.act)
        elif self.group:
            if row_sums is None:
                ops.gated_linear(x, self.w_gate_up, act)
            else:
                ops.gated_linear(x, self.w_gate_up, act, row_sums=row_sums)
        else:
            gu = torch.empty((T, 2 * I), dtype=self.dtype, device=x.device)
            if row_sums is None:
                ops.linear(x, self.w_gate_up, gu)
            else:
                ops.linear_skinny(x, self.w_gate_up, gu, row_sums=row_sums)
            ops.silu_mul(gu, act)
        can_add = getattr(ops, "can_accumulate", None)
        if resid is not None and can_add and can_add(act, self.w_down):
            if resid_scale != 1.0:
                ops.linear_skinny(act, self.w_down, resid, accumulate=True, alpha=resid_scale)
                return None
            # x += act . Wd^T in the epilogue, which can also prepare the norm that follows
            if emit is not None and emit.finished:
                done = ops.linear_skinny(act, self.w_down, resid, accumulate=True, finish=emit.finish)
                return emit if done else None
            if emit is not None:
                written = ops.linear_skinny(act, self.w_down, resid, accumulate=True, emit=emit.emit)
                emit.ss = emit.ss[:written]          # as many partial sums a row as the kernel that ran has workgroups
                return emit
            ops.linear_skinny(act, self.w_down, resid, accumulate=True)
            return None
        out = torch.empty((T, self.spec.hidden), dtype=self.dtype, device=x.device)
        ops.linear(act, self.w_down, out)
        return out
