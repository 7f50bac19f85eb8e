"""Mixture-of-experts feed-forward: a router picks ``top`` of ``experts`` small feed-forward layers a token.

Router logits z = W_r h in float; the ``top`` largest are chosen and weighted by the softmax over the chosen
logits alone; an expert is W_down act(W_up h) with act = relu squared, no bias; the output is the weighted
sum of the chosen experts' outputs.

The experts' up projections are laid side by side as one [experts * ff, width] matrix and their down
projections as one [width, experts * ff] matrix. A step computes every expert's up projection in one product,
applies the activation and the routing weight in one kernel (0 for experts a token did not choose), and one
product with the down matrix is then the weighted sum: with few experts of which a good share is chosen, two
dense products at the matrix cores' rate cost less than gathering tokens by expert would. A step of so few
tokens that most experts are not asked for at all (one or two requests decoding) reads only the chosen experts'
rows instead, a wave a row.

A second form of the same part (``activation`` "silu_gated", ``weights`` "sigmoid"): an expert is
W_down (silu(W_gate h) * (W_up h)); a token's score for expert e is sigmoid(z_e); where the experts form
groups of neighbours, a group's score is the sum of its largest scores (two of them) and only experts of the
best groups can be chosen; the chosen experts' weights are their scores times a constant, not renormalised;
a shared expert of the same form may run for every token. Here every expert's [gate; up] rows lie one
after the other in one matrix, the shared expert's behind them, one kernel applies the gate and the
routing weight (1 for the shared expert, 0 for experts not chosen), and one product with all down
projections side by side is the sum. A step of few tokens reads only the chosen experts' rows and the shared
expert's, as the first form does.

A third form (``activation`` "silu_gated", ``weights`` "softmax"): scores are the softmax of the router's logits
over all its outputs; the choice is by score + a stored correction, inside the best groups (a group's score is
its largest choice score); the weights are the chosen scores over their sum. The router's last ``identity``
outputs stand for experts without matrices whose output is the token's input row; the shared expert's result is
multiplied by the sigmoid of one more logit a token (its weight row lies behind the router's, so the same float
product makes it). The experts' matrices and the two products are those of the second form.

A fourth form (``activation`` "silu_gated", ``weights`` "table"): no router. An integer table [vocabulary, top]
gives each token id its experts (the entries of a row differ), each weighing 1 / top; a kernel looks the step's
token ids up, and everything behind the choice is the second form's.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import kernels
from ..config.schema import FeedForwardSpec
from ..weights import INT_TABLE, VECTOR, ParamDecl
from .registry import register_feed_forward


@register_feed_forward("moe")
class MixtureOfExperts:
    graph_safe = True       # routing stays on the device: a decode step with it can be captured
    adds_in_place = True    # forward(..., resid=) may add the down projection into the stream
    adds_scaled = True      # forward(..., resid=, resid_scale=) adds resid_scale times the result

    @classmethod
    def declare_params(cls, spec: FeedForwardSpec, prefix: str) -> List[ParamDecl]:
        p = spec.params
        out = []
        gated = p.activation == "silu_gated"
        for e in range(p.experts):
            if gated:
                out.append(ParamDecl(f"{prefix}e{e}.gate", (spec.intermediate, spec.hidden)))
            out += [ParamDecl(f"{prefix}e{e}.up", (spec.intermediate, spec.hidden)),
                    ParamDecl(f"{prefix}e{e}.down", (spec.hidden, spec.intermediate))]
        if p.weights == "table":
            out.append(ParamDecl(prefix + "table", (int(dict(spec.extra)["vocab"]), p.top), init=f"distinct:{p.experts}",
                                 role=INT_TABLE))
        else:
            out.append(ParamDecl(prefix + "router", (p.experts + p.identity, spec.hidden)))
        if p.correction:
            out.append(ParamDecl(prefix + "correction", (p.experts + p.identity,), init="zeros", role=VECTOR))
        if p.shared:
            if gated:
                out.append(ParamDecl(prefix + "shared.gate", (p.shared, spec.hidden)))
            out += [ParamDecl(prefix + "shared.up", (p.shared, spec.hidden)),
                    ParamDecl(prefix + "shared.down", (spec.hidden, p.shared))]
            if p.shared_gated:
                out.append(ParamDecl(prefix + "shared.sg", (1, spec.hidden)))
        return out

    def __init__(self, spec: FeedForwardSpec, weights: Dict[str, torch.Tensor], prefix: str,
                 dtype: torch.dtype, device: torch.device):
        p = spec.params
        if p is None:
            raise ValueError("moe: the routing comes in FeedForwardSpec.params (MoESpec)")
        if (p.activation, p.weights) not in (("relu2", "softmax_chosen"), ("silu_gated", "sigmoid"),
                                             ("silu_gated", "softmax"), ("silu_gated", "table")):
            raise ValueError(f"moe: activation {p.activation!r} with weights {p.weights!r} is not built")
        self.spec = spec
        self.dtype = dtype
        self.experts, self.top, self.ff = int(p.experts), int(p.top), int(spec.intermediate)
        self.gated = p.activation == "silu_gated"
        self.routing = p
        self.identity = int(p.identity)
        routed = self.experts + self.identity             # groups are formed over experts and identity experts together
        if p.groups < 1 or routed % p.groups or not 1 <= p.groups_kept <= p.groups \
                or p.top > p.groups_kept * (routed // p.groups):
            raise ValueError(f"moe: {routed} experts in {p.groups} groups of which {p.groups_kept} are kept "
                             f"cannot give {p.top} choices")
        if p.weights != "softmax" and (p.identity or p.correction or p.shared_gated):
            raise ValueError("moe: identity experts, a correction of the choice and a gate on the shared expert "
                             "are built for the softmax router")
        if p.weights == "softmax" and p.groups > 1 and p.group_top != 1:
            raise ValueError("moe: the softmax router scores a group by its largest choice score (group_top 1)")
        if p.shared_gated and not p.shared:
            raise ValueError("moe: a gate on the shared expert needs a shared expert")
        if (p.groups > 1 or p.shared) and not self.gated:
            raise ValueError("moe: groups of experts and a shared expert are built for the gated form")
        self.table = None
        if p.weights == "table":
            if p.groups != 1 or p.top > p.experts:
                raise ValueError(f"moe: a table of {p.top} choices among {p.experts} experts in {p.groups} groups")
            self.table = weights[prefix + "table"].contiguous()
            if int(self.table.min()) < 0 or int(self.table.max()) >= self.experts:
                raise ValueError(f"moe: {prefix}table names experts outside 0..{self.experts - 1}")
        self.router = weights[prefix + "router"] if self.table is None else None      # logits are accumulated and kept in float
        self.correction = weights[prefix + "correction"].float().contiguous() if p.correction else None
        if p.shared_gated:
            # the shared expert's gate is one more row of the float product that makes the router's logits
            self.router = torch.cat([self.router, weights[prefix + "shared.sg"]], dim=0).contiguous()
        if self.gated:
            self.shared = int(p.shared)
            rows = []
            for e in range(self.experts):
                rows += [weights[f"{prefix}e{e}.gate"], weights[f"{prefix}e{e}.up"]]
            downs = [weights[f"{prefix}e{e}.down"] for e in range(self.experts)]
            if self.shared:
                rows += [weights[prefix + "shared.gate"], weights[prefix + "shared.up"]]
                downs.append(weights[prefix + "shared.down"])
            self.w_gate_up = torch.cat(rows, dim=0).contiguous()       # [2 (E ff + shared), width]
            self.w_down = torch.cat(downs, dim=1).contiguous()          # [width, E ff + shared]
            return
        self.w_up = torch.cat([weights[f"{prefix}e{e}.up"] for e in range(self.experts)], dim=0).contiguous()
        self.w_down = torch.cat([weights[f"{prefix}e{e}.down"] for e in range(self.experts)], dim=1).contiguous()

    def _forward_gated(self, x, resid, resid_scale=1.0, batch=None):
        ops = kernels.current()
        p = self.routing
        T = x.shape[0]
        n = self.experts * self.ff + self.shared
        ids = torch.empty((T, self.top), dtype=torch.int32, device=x.device)
        weights = torch.empty((T, self.top), dtype=torch.float32, device=x.device)
        routed = self.experts + self.identity
        shared_logit = None
        if p.weights == "table":
            ops.moe_table_route(batch.token_ids, self.table, ids, weights)
        elif p.weights == "softmax":
            logits = ops.moe_route(x, self.router, self.top, ids, weights, scoring="softmax", groups=int(p.groups),
                                   groups_kept=int(p.groups_kept), correction=self.correction,
                                   norm_eps=float(p.norm_eps), outputs=routed)
            if p.shared_gated:
                shared_logit = logits[:, routed]
        else:
            ops.moe_route(x, self.router, self.top, ids, weights, scoring="sigmoid", scale=float(p.weight_scale),
                          groups=int(p.groups), groups_kept=int(p.groups_kept), group_top=int(p.group_top))
        chosen = getattr(ops, "moe_reads_chosen", None)
        if chosen is not None and hasattr(ops, "moe_gate_up_chosen") and chosen(T, self.top, routed):
            # so few tokens that most experts are not asked for: only the chosen experts' rows and the shared
            # expert's are read; the identity experts' share is added behind the down projection's sum
            act = torch.empty((T, self.top * self.ff + self.shared), dtype=self.dtype, device=x.device)
            ops.moe_gate_up_chosen(x, self.w_gate_up, ids, weights, act, self.experts, self.ff, self.shared,
                                   shared_logit=shared_logit)
            out = torch.empty((T, self.spec.hidden), dtype=self.dtype, device=x.device)
            ops.moe_down_gated_chosen(act, self.w_down, ids, weights, x, out, self.experts, self.ff, self.shared)
            return out
        gu = torch.empty((T, 2 * n), dtype=self.dtype, device=x.device)
        ops.linear(x, self.w_gate_up, gu)
        act = torch.empty((T, n), dtype=self.dtype, device=x.device)
        if shared_logit is not None:
            ops.moe_silu_gate_scale(gu, act, ids, weights, self.experts, self.ff, self.shared, shared_logit=shared_logit)
        else:
            ops.moe_silu_gate_scale(gu, act, ids, weights, self.experts, self.ff, self.shared)
        if self.identity:
            # the chosen identity experts' share, weight times the input row, is added to the product's result
            out = torch.empty((T, self.spec.hidden), dtype=self.dtype, device=x.device)
            ops.linear(act, self.w_down, out)
            ops.moe_identity_add(out, x, ids, weights, self.experts)
            return out
        can_add = getattr(ops, "can_accumulate", None)
        if resid is not None and can_add and can_add(act, self.w_down):
            if resid_scale != 1.0:
                ops.linear_skinny(act, self.w_down, resid, accumulate=True, alpha=resid_scale)
            else:
                ops.linear_skinny(act, self.w_down, resid, accumulate=True)
            return None
        out = torch.empty((T, self.spec.hidden), dtype=self.dtype, device=x.device)
        ops.linear(act, self.w_down, out)
        return out

    def forward(self, x, batch, resid: Optional[torch.Tensor] = None, resid_scale: float = 1.0):
        if self.gated:
            return self._forward_gated(x, resid, resid_scale, batch)
        if resid_scale != 1.0:
            resid = None                    # the ungated form adds its result as it is: the caller scales it
        ops = kernels.current()
        T = x.shape[0]
        n = self.experts * self.ff
        ids = torch.empty((T, self.top), dtype=torch.int32, device=x.device)
        weights = torch.empty((T, self.top), dtype=torch.float32, device=x.device)
        ops.moe_route(x, self.router, self.top, ids, weights)
        chosen = getattr(ops, "moe_reads_chosen", None)
        if chosen is not None and chosen(T, self.top, self.experts):
            # so few tokens that most experts are not asked for: only the chosen experts' rows are read
            act = torch.empty((T * self.top, self.ff), dtype=self.dtype, device=x.device)
            ops.moe_up_chosen(x, self.w_up, ids, weights, act, self.ff)
            if resid is not None:
                ops.moe_down_chosen(act, self.w_down, ids, self.ff, resid=resid)
                return None
            out = torch.empty((T, self.spec.hidden), dtype=self.dtype, device=x.device)
            ops.moe_down_chosen(act, self.w_down, ids, self.ff, out=out)
            return out
        up = torch.empty((T, n), dtype=self.dtype, device=x.device)
        ops.linear(x, self.w_up, up)
        act = torch.empty((T, n), dtype=self.dtype, device=x.device)
        ops.moe_relu2_scale(up, act, ids, weights, self.experts, self.ff)
        can_add = getattr(ops, "can_accumulate", None)
        if resid is not None and can_add and can_add(act, self.w_down):
            ops.linear_skinny(act, self.w_down, resid, accumulate=True)
            return None
        out = torch.empty((T, self.spec.hidden), dtype=self.dtype, device=x.device)
        ops.linear(act, self.w_down, out)
        return out
