"""Several mixers on one input, averaged: y = (1/n) sum_i rms(mixer_i(h)) * w_i; or, with ``combine``
"scaled_sum", added up with a constant each: y = sum_i s_i mixer_i(h), no norms and no weights.

Each member reads the same normed input and keeps what it needs itself (keys and values in pages, a recurrent
state in the request's slot); the layer's cache need is the members' needs side by side
(:class:`JointNeed`). A member's output is divided by its root mean square over the model width and
multiplied by a plain weight of its own before the mean, all in float, one kernel.
"""
from __future__ import annotations

from typing import Dict, List

import torch

from .. import kernels
from ..config.schema import MixerSpec
from ..weights import VECTOR, ParamDecl
from .base import JointNeed, LayerCache, ScaledTerms
from .registry import lookup, register_mixer


@register_mixer("side_by_side")
class SideBySide:
    @classmethod
    def declare_params(cls, spec: MixerSpec, prefix: str) -> List[ParamDecl]:
        p = spec.params
        out: List[ParamDecl] = []
        for sub, m in p.members:
            out += lookup("mixer", m.kind).declare_params(m, prefix + sub)
        if getattr(p, "combine", "normed_mean") == "normed_mean":
            for sub, _ in p.members:
                out.append(ParamDecl(prefix + sub + p.out_name, (spec.hidden,), init="norm", role=VECTOR))
        return out

    def __init__(self, spec: MixerSpec, weights: Dict[str, torch.Tensor], prefix: str, dtype: torch.dtype,
                 device: torch.device):
        p = spec.params
        if p is None or not p.members:
            raise ValueError("side_by_side: the members come in MixerSpec.params (SideBySideSpec)")
        self.spec, self.dtype = spec, dtype
        self.eps = float(p.norm_eps)
        self.members = [lookup("mixer", m.kind)(m, weights, prefix + sub, dtype, device) for sub, m in p.members]
        self.combine = str(getattr(p, "combine", "normed_mean"))
        if self.combine == "scaled_sum":
            self.scales = [float(v) for v in p.scales]
            if len(self.scales) != len(self.members):
                raise ValueError(f"side_by_side: {len(self.scales)} factors for {len(self.members)} mixers")
            self.adds_scaled = False
            self.returns_terms = True      # forward(..., terms_ok=True) may hand back the addends with their factors
            return
        if self.combine != "normed_mean":
            raise ValueError(f"side_by_side: combine {self.combine!r}; built: normed_mean, scaled_sum")
        self.out_weights = [weights[prefix + sub + p.out_name].float().contiguous() for sub, _ in p.members]

    @property
    def graph_safe(self) -> bool:
        return all(bool(getattr(m, "graph_safe", False)) for m in self.members)

    def cache_need(self) -> JointNeed:
        return JointNeed(tuple(m.cache_need() if hasattr(m, "cache_need") else None for m in self.members))

    def plan_captured_step(self, batch, num_rows: int, ctx_cap: int) -> None:
        for m in self.members:
            hook = getattr(m, "plan_captured_step", None)
            if hook is not None:
                hook(batch, num_rows, ctx_cap)

    adds_scaled = True      # forward(..., resid=, resid_scale=) adds the mean into the float stream itself

    def forward(self, x, batch, cache: LayerCache, resid=None, resid_scale: float = 1.0, terms_ok: bool = False):
        outs = [m.forward(x, batch, cache.members[i]) for i, m in enumerate(self.members)]
        if self.combine == "scaled_sum":
            if terms_ok:
                # the caller adds the sum up itself (in the kernel that norms it and adds it to the stream)
                return ScaledTerms(outs, list(self.scales))
            out = torch.empty_like(outs[0])
            kernels.current().sum_norm_add(outs, self.scales, None, 0.0, copy=out)
            return out
        if resid is not None:
            kernels.current().normed_mean(outs, self.out_weights, self.eps, resid=resid, scale=resid_scale)
            return None
        out = torch.empty_like(outs[0])
        kernels.current().normed_mean(outs, self.out_weights, self.eps, out=out)
        return out
