"""Attention over a cached low-rank latent, inside an optional sliding window.

With h the mixer's input, per token: q = W_q h (heads of [head_dim unrotated | rot_width rotated]),
(c_raw | kr) = W_dkv h, c = rms(c_raw) * w_c. Head a has keys W_uk,a c and values W_uv,a c, one rotated key
part kr for all heads, score scale * (q_a . k_a + rot(qr_a) . rot(kr)), softmax over the window, and the
concatenated heads, times sigmoid(W_g h) where the mixer is gated, go through W_o.

Only c and the rotated key part are cached. Since a head's keys and values are linear in c,

    q_a . (W_uk,a c) = (W_uk,a^T q_a) . c        and        sum_j p_j W_uv,a c_j = W_uv,a (sum_j p_j c_j),

the attention itself runs over the cached rows [c | rot(kr)] as ONE shared KV head of size
Dp = rank + rot_width (rounded up to the cache's tile of 16) for all query heads, through the same paged
kernels as grouped-query attention: queries [W_uk,a^T q_a | rot(qr_a)], values the same rows (the columns
behind ``rank`` of the result are not used). What is new here are the kernel that norms, rotates and writes
the cache row (``latent_prep``) and the products head by head before and after (``head_linear``).
q, the latent and the gate come from one fused product.

Two options. ``q_rank`` > 0: the queries come through a latent of their own, q = W_uq (rms(W_dq h) * w_q): the
fused product then makes [latent of q | latent | key part | gate], a row norm and a second product make q.
``head_gate``: the gate is one number a head, sigmoid(W_g h)_a with W_g [heads, width], not one a value entry.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import kernels
from ..config.schema import MixerSpec
from ..weights import VECTOR, ParamDecl
from .base import KVNeed, LayerCache
from .registry import lookup, register_mixer


def _round16(n: int) -> int:
    return -(-n // 16) * 16


@register_mixer("latent_attention")
class LatentAttention:
    graph_safe = True       # no host-side state: a decode step with it can be captured
    adds_in_place = True    # forward(..., resid=) may add the output projection into the stream

    @classmethod
    def declare_params(cls, spec: MixerSpec, prefix: str) -> List[ParamDecl]:
        p = spec.params
        H, D, R = spec.num_heads, spec.head_dim, p.rot_width
        if p.q_rank:
            out = [ParamDecl(prefix + "dq", (p.q_rank, spec.hidden)),
                   ParamDecl(prefix + "dq.norm", (p.q_rank,), init="norm", role=VECTOR),
                   ParamDecl(prefix + "uq", (H * (D + R), p.q_rank))]
        else:
            out = [ParamDecl(prefix + "q", (H * (D + R), spec.hidden))]
        out += [ParamDecl(prefix + "dkv", (p.rank + R, spec.hidden)),
               ParamDecl(prefix + "dkv.norm", (p.rank,), init="norm", role=VECTOR),
               ParamDecl(prefix + "uk", (H * D, p.rank)),
               ParamDecl(prefix + "uv", (H * p.value_dim, p.rank))]
        if p.gated:
            out.append(ParamDecl(prefix + "g", (H if p.head_gate else H * p.value_dim, spec.hidden)))
        out.append(ParamDecl(prefix + "o", (spec.hidden, H * p.value_dim)))
        return out

    def __init__(self, spec: MixerSpec, weights: Dict[str, torch.Tensor], prefix: str,
                 dtype: torch.dtype, device: torch.device):
        p = spec.params
        if p is None:
            raise ValueError("latent_attention: the mixer's sizes come in MixerSpec.params (LatentAttentionSpec)")
        self.spec = spec
        self.dtype = dtype
        self.num_heads, self.head_dim = int(spec.num_heads), int(spec.head_dim)
        self.rank, self.rot_width, self.value_dim = int(p.rank), int(p.rot_width), int(p.value_dim)
        self.gated = bool(p.gated)
        self.head_gate = bool(p.head_gate)
        self.q_rank = int(p.q_rank)
        self.eps = float(p.norm_eps)
        self.scale = float(spec.scale)
        self.window = int(spec.window)
        self.cache_dim = _round16(self.rank + self.rot_width)
        H, D, R, Dv = self.num_heads, self.head_dim, self.rot_width, self.value_dim
        # one product for everything that reads the mixer's input: rows of q (or of its latent), of the latent,
        # of the gate. The buffer's row always starts with the H query heads, which a second product fills
        # where the queries go through a latent of their own; every part starts at a multiple of 8 columns
        # (16-byte pieces for the kernels that read them).
        def pad8(n: int) -> int:
            return -(-n // 8) * 8

        def zeros(n: int):
            return torch.zeros((n, spec.hidden), dtype=self.w_dtype, device=weights[prefix + "dkv"].device)
        self.w_dtype = weights[prefix + "dkv"].dtype
        self.gate_width = (H if self.head_gate else H * Dv) if self.gated else 0
        self.q_off = 0
        self.dkv_off = pad8(H * (D + R))
        self.gate_off = self.dkv_off + pad8(self.rank + R)
        self.dq_off = self.gate_off + pad8(self.gate_width)
        self.proj_width = self.dq_off + pad8(self.q_rank)
        parts = [(self.dkv_off, weights[prefix + "dkv"])]
        if self.gated:
            parts.append((self.gate_off, weights[prefix + "g"]))
        if self.q_rank:
            parts.append((self.dq_off, weights[prefix + "dq"]))
            self.in_off = self.dkv_off          # the fused product fills the row from here on
            self.w_uq = weights[prefix + "uq"]
            self.q_norm = weights[prefix + "dq.norm"]
        else:
            parts.insert(0, (0, weights[prefix + "q"]))
            self.in_off = 0
        rows, at = [], self.in_off
        for off, w in parts:
            if off > at:
                rows.append(zeros(off - at))
            rows.append(w)
            at = off + int(w.shape[0])
        if self.proj_width > at:
            rows.append(zeros(self.proj_width - at))
        self.w_in = torch.cat(rows, dim=0).contiguous()
        self.c_norm = weights[prefix + "dkv.norm"]
        # head products, [heads, N, K] with K contiguous: queries through the key matrices, W_uk[a, d, r] transposed
        # to [a, r, d]; results through the value matrices, W_uv[a, v, r] as stored
        self.w_absorb = weights[prefix + "uk"].view(H, D, self.rank).transpose(1, 2).contiguous()
        self.w_values = weights[prefix + "uv"].view(H, Dv, self.rank).contiguous()
        self.w_o = weights[prefix + "o"]
        self.position = lookup("position", spec.position.kind)(spec.position, device)
        if self.position.rotary_dim > R:
            raise ValueError("the rotated width cannot exceed the rotated part of a head")

    def cache_need(self) -> KVNeed:
        return KVNeed(1, self.cache_dim, self.window)

    def plan_captured_step(self, batch, num_rows: int, ctx_cap: int) -> None:
        hook = getattr(kernels.current(), "plan_captured_step", None)
        if hook is not None:
            hook(batch, num_rows, ctx_cap)

    def _head_groups(self, ops, cache: LayerCache):
        """(first head, heads) of each attention call: all heads at once where the kernels take that many
        query heads on one KV head, else even groups of as many as they take."""
        H = self.num_heads
        groups = getattr(self, "_groups", None)
        if groups is None:
            limit = 0
            ask = getattr(ops, "shared_head_limit", None)
            if ask is not None and self.dtype == torch.bfloat16:
                limit = int(ask(self.cache_dim, cache.k.shape[2] * 16))
            if limit <= 0 or H <= limit:
                groups = [(0, H)]
            else:
                n = -(-H // limit)
                base, extra = divmod(H, n)
                groups, a = [], 0
                for i in range(n):
                    g = base + (1 if i < extra else 0)
                    groups.append((a, g))
                    a += g
            self._groups = groups
        return groups

    def forward(self, x, batch, cache: LayerCache, resid: Optional[torch.Tensor] = None):
        ops = kernels.current()
        T = x.shape[0]
        H, D, Dv, Dp = self.num_heads, self.head_dim, self.value_dim, self.cache_dim
        slots = batch.slots[cache.group] if cache.writes else batch.no_slots
        proj = torch.empty((T, self.proj_width), dtype=self.dtype, device=x.device)
        ops.linear(x, self.w_in, proj[:, self.in_off:])
        if self.q_rank:
            # the queries' latent, normed in float over its own width, then up to the heads
            cq = torch.empty((T, self.q_rank), dtype=self.dtype, device=x.device)
            ops.rows_rmsnorm(proj[:, self.dq_off:self.dq_off + self.q_rank], self.q_norm, self.eps, cq)
            ops.linear(cq, self.w_uq, proj[:, :H * (D + self.rot_width)])
        q_lat = torch.empty((T, H, Dp), dtype=self.dtype, device=x.device)
        ops.latent_prep(proj, self.q_off, self.dkv_off, self.c_norm, self.eps, batch.positions,
                        self.position.inv_freq, self.position.rotary_dim, self.rot_width, self.rank, H, D,
                        q_lat, slots, cache.k, cache.v)
        q_rows = q_lat.view(T, H * Dp)
        if D > 0:
            ops.head_linear(proj[:, self.q_off:], D + self.rot_width, self.w_absorb, q_rows, Dp)
        else:
            q_lat[:, :, :self.rank].zero_()
        o_lat = torch.empty((T, H * Dp), dtype=self.dtype, device=x.device)
        for a, g in self._head_groups(ops, cache):
            # heads a .. a + g - 1 against the one cached row a token: column ranges of the same buffers
            ops.attention(q_rows[:, a * Dp:], H * Dp, o_lat[:, a * Dp:(a + g) * Dp], cache.k, cache.v, batch, g, 1,
                          Dp, self.scale, self.window, cache.group)
        heads = torch.empty((T, H * Dv), dtype=self.dtype, device=x.device)
        ops.head_linear(o_lat, Dp, self.w_values, heads, Dv,
                        gate=proj[:, self.gate_off:self.gate_off + self.gate_width] if self.gated else None,
                        gate_per_head=self.head_gate)
        can_add = getattr(ops, "can_accumulate", None)
        if resid is not None and can_add and can_add(heads, self.w_o):
            ops.linear_skinny(heads, self.w_o, resid, accumulate=True)
            return None
        out = torch.empty((T, self.spec.hidden), dtype=self.dtype, device=x.device)
        ops.linear(heads, self.w_o, out)
        return out
