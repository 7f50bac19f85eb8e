"""Grouped-query attention over the paged cache.

q/k/v projections (one fused product), optional per-head RMSNorm of q and k,
rotation, cache write, attention over the request's block table, output
projection. Order and formulas: crates/cuda/src/engine.rs:4090-4281 (decode) and
:5462-5621 (whole prompt); the reference has separate kernels for head norm,
rotation, scale and cache write and separate calls for prompts and decoding,
here one fused kernel and one call serve any mix of both. The scale multiplies
the float score, not q (the reference scales and re-rounds q, engine.rs:4150-4160).

A value head may have a size of its own (``MixerSpec.value_dim``), and head sizes need not be multiples of
16: the cache and the kernels work on heads of one size D, the larger of the two rounded up to 16, and the
projections are laid out for it at load (rows of zeros behind each head of W_q, W_k and W_v, columns of zeros
in W_o). Zeros in q and k add nothing to a score, zeros in v give zeros that W_o's zero columns meet, so
the result is the attention of the sizes given. Tensor names other than ``q_proj.weight`` ... come as the
option ``names`` = (q, k, v, o); ``bias_suffix`` names the biases after their matrices (``q`` + suffix) and
``norm_names`` = (q, k) the head-norm weights.

Further options (fields of the ``MixerSpec``), each with kernels of its own around the same paged attention:
``qk_norm_whole`` (q and k are RMS-normed over all their heads at once, with weights of that size), ``softcap``
and ``distance_bias`` (the score is capped by a tanh, and r1_h ln(1 + r2_h (i - j)) is taken off it, tensors
``r1`` and ``r2`` with one number a query head), ``rotate_values`` (a value is turned by its own position over
its whole size before it is cached, pair m by position * theta^(-2m / size) in the pair layout of the mixer's
rotation, and a head's result is turned back by the query's position), ``out_gate`` (the concatenated heads times
sigmoid(W_g h), tensor ``g``) and ``kv_shared`` (no key and value tensors: the layer reads another layer's cache
with queries of its own). With a head norm and heads that are padded with zeros the norm's mean is taken over
the true size: the kernel's mean over D entries with eps * size / D inside the root, times sqrt(size / D) folded
into the weight, is the same number.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import kernels
from ..config.schema import MixerSpec
from ..weights import MATRIX, VECTOR, ParamDecl
from .base import KVNeed, LayerCache, NormTarget, split_input
from .registry import lookup, register_mixer


@register_mixer("gqa_attention")
class GroupedQueryAttention:
    graph_safe = True       # no host-side state: a decode step with it can be captured
    adds_in_place = True    # forward(..., resid=) may add the output projection into the stream
    takes_row_scaled = True     # x may be RowScaled: the q/k/v product applies the row factor
    emits_for_norm = True       # forward(..., emit=) may fill a NormTarget from the output projection

    @staticmethod
    def _names(spec: MixerSpec):
        return tuple(spec.option("names", ("q_proj.weight", "k_proj.weight", "v_proj.weight", "o_proj.weight")))

    @classmethod
    def _bias_names(cls, spec: MixerSpec):
        suffix = spec.option("bias_suffix")
        if suffix is None:
            return ("q_proj.bias", "k_proj.bias", "v_proj.bias")
        q, k, v, _ = cls._names(spec)
        return (q + suffix, k + suffix, v + suffix)

    @staticmethod
    def _norm_names(spec: MixerSpec):
        return tuple(spec.option("norm_names", ("q_norm.weight", "k_norm.weight")))

    @staticmethod
    def _extended(spec: MixerSpec) -> bool:
        return bool(spec.qk_norm_whole or spec.softcap or spec.distance_bias or spec.rotate_values or spec.out_gate
                    or spec.kv_shared)

    @classmethod
    def declare_params(cls, spec: MixerSpec, prefix: str) -> List[ParamDecl]:
        nq = spec.num_heads * spec.head_dim
        nkv = spec.num_kv_heads * spec.head_dim
        vd = spec.value_dim or spec.head_dim
        q, k, v, o = cls._names(spec)
        own_kv = not spec.kv_shared
        out = [ParamDecl(prefix + q, (nq, spec.hidden))]
        if own_kv:
            out += [ParamDecl(prefix + k, (nkv, spec.hidden)),
                    ParamDecl(prefix + v, (spec.num_kv_heads * vd, spec.hidden))]
        out.append(ParamDecl(prefix + o, (spec.hidden, spec.num_heads * vd)))
        if spec.bias:
            bq, bk, bv = cls._bias_names(spec)
            out.append(ParamDecl(prefix + bq, (nq,), init="zeros", role=MATRIX))
            if own_kv:
                out += [ParamDecl(prefix + bk, (nkv,), init="zeros", role=MATRIX),
                        ParamDecl(prefix + bv, (spec.num_kv_heads * vd,), init="zeros", role=MATRIX)]
        if spec.qk_norm or spec.qk_norm_whole:
            nq_name, nk_name = cls._norm_names(spec)
            out.append(ParamDecl(prefix + nq_name, (nq if spec.qk_norm_whole else spec.head_dim,), init="norm", role=VECTOR))
            if own_kv:
                out.append(ParamDecl(prefix + nk_name, (nkv if spec.qk_norm_whole else spec.head_dim,), init="norm",
                                     role=VECTOR))
        if spec.distance_bias:
            out += [ParamDecl(prefix + "r1", (spec.num_heads,), init="norm", role=VECTOR),
                    ParamDecl(prefix + "r2", (spec.num_heads,), init="norm", role=VECTOR)]
        if spec.out_gate:
            out.append(ParamDecl(prefix + "g", (spec.num_heads * vd, spec.hidden)))
        return out

    def __init__(self, spec: MixerSpec, weights: Dict[str, torch.Tensor], prefix: str,
                 dtype: torch.dtype, device: torch.device):
        if spec.num_heads <= 0 or spec.num_kv_heads <= 0 or spec.num_heads % spec.num_kv_heads:
            raise ValueError(f"{spec.num_heads} query heads do not divide into {spec.num_kv_heads} groups")
        self.spec = spec
        self.dtype = dtype
        key_dim, value_dim = spec.head_dim, spec.value_dim or spec.head_dim
        # the one head size the cache and the kernels work with
        D = -(-max(key_dim, value_dim) // 16) * 16
        self.num_heads, self.num_kv_heads, self.head_dim = spec.num_heads, spec.num_kv_heads, D
        self.key_dim, self.value_dim = key_dim, value_dim
        self.scale = float(spec.scale)
        self.window = int(spec.window)
        self.qkv_width = (spec.num_heads + 2 * spec.num_kv_heads) * D
        qn, kn, vn, on = self._names(spec)
        H, G = spec.num_heads, spec.num_kv_heads
        self.own_kv = not spec.kv_shared
        self.extended = self._extended(spec)
        if self.extended:
            # the further options run as kernels of their own around the attention: no norm rides on this
            # mixer's products, and its result goes back to the caller
            self.adds_in_place = self.takes_row_scaled = self.emits_for_norm = False
        if (key_dim != D or value_dim != D) and (spec.qk_norm or spec.bias) and not self.extended:
            raise ValueError(f"attention: heads of {key_dim} / {value_dim} are laid out with zeros behind them, which a "
                             "head norm or a bias takes only on the path of the further options: without those, head "
                             "sizes go in steps of 16")
        if spec.qk_norm and spec.qk_norm_whole:
            raise ValueError("attention: q and k are normed per head or over their whole projection, not both")

        def heads_of(w, n, d):           # [n * d, ...] -> [n * D, ...], zeros behind each head
            if d == D:
                return w
            out = torch.zeros((n, D, *w.shape[1:]), dtype=w.dtype, device=w.device)
            out[:, :d] = w.view(n, d, *w.shape[1:])
            return out.view(n * D, *w.shape[1:])
        # rows of q, k, v one after the other: stays [out, in], K contiguous
        rows = [heads_of(weights[prefix + qn], H, key_dim)]
        if self.own_kv:
            rows += [heads_of(weights[prefix + kn], G, key_dim), heads_of(weights[prefix + vn], G, value_dim)]
        self.w_qkv = torch.cat(rows, dim=0).contiguous()
        self.b_qkv = None
        if spec.bias:
            bq, bk, bv = self._bias_names(spec)
            rows = [heads_of(weights[prefix + bq], H, key_dim)]
            if self.own_kv:
                rows += [heads_of(weights[prefix + bk], G, key_dim), heads_of(weights[prefix + bv], G, value_dim)]
            self.b_qkv = torch.cat(rows, dim=0).to(dtype).contiguous()
        self.w_o = weights[prefix + on]
        if value_dim != D:
            wo = torch.zeros((spec.hidden, H, D), dtype=self.w_o.dtype, device=self.w_o.device)
            wo[:, :, :value_dim] = self.w_o.view(spec.hidden, H, value_dim)
            self.w_o = wo.view(spec.hidden, H * D).contiguous()
        self.eps = float(spec.qk_norm_eps)
        self.q_norm = self.k_norm = self.q_whole = self.k_whole = None
        nq_name, nk_name = self._norm_names(spec)
        if spec.qk_norm:
            self.q_norm = weights[prefix + nq_name]
            self.k_norm = weights[prefix + nk_name] if self.own_kv else self.q_norm
            if key_dim != D:
                # the kernel's mean runs over D entries of which key_dim carry values
                fold = (key_dim / D) ** 0.5
                pad = lambda w: torch.cat([w.float() * fold, torch.zeros(D - key_dim, dtype=torch.float32, device=w.device)])
                self.q_norm, self.k_norm = pad(self.q_norm).contiguous(), pad(self.k_norm).contiguous()
                self.eps = self.eps * key_dim / D
        if spec.qk_norm_whole:
            self.q_whole = heads_of(weights[prefix + nq_name].float(), H, key_dim).contiguous()
            if self.own_kv:
                self.k_whole = heads_of(weights[prefix + nk_name].float(), G, key_dim).contiguous()
        self.position = lookup("position", spec.position.kind)(spec.position, device)
        if self.position.rotary_dim > key_dim:
            raise ValueError("the rotated width cannot exceed the head size")
        self.softcap = float(spec.softcap)
        self.distance = None
        if spec.distance_bias:
            self.distance = (weights[prefix + "r1"].float().contiguous(), weights[prefix + "r2"].float().contiguous())
        self.value_inv_freq = None
        if spec.rotate_values:
            if value_dim % 2:
                raise ValueError(f"attention: values of {value_dim} entries do not turn in pairs")
            m = torch.arange(value_dim // 2, dtype=torch.float64)
            theta = torch.tensor(float(spec.position.theta), dtype=torch.float64)
            self.value_inv_freq = torch.pow(theta, -2.0 * m / value_dim).to(torch.float32).to(device)
        self.w_gate = None
        if spec.out_gate:
            self.w_gate = heads_of(weights[prefix + "g"], H, value_dim).contiguous()

    def cache_need(self) -> KVNeed:
        return KVNeed(self.num_kv_heads, self.head_dim, self.window)

    def plan_captured_step(self, batch, num_rows: int, ctx_cap: int) -> None:
        # the attention kernels pick their grids by host-side numbers of the step: the kernel set fixes them
        hook = getattr(kernels.current(), "plan_captured_step", None)
        if hook is not None:
            hook(batch, num_rows, ctx_cap)

    def _forward_extended(self, x, batch, cache: LayerCache):
        """The mixer with any of its further options; the result is float (it enters a float sum as it is)."""
        ops = kernels.current()
        T = x.shape[0]
        H, G, D = self.num_heads, self.num_kv_heads, self.head_dim
        # a layer without keys of its own makes queries alone; where the head kernel must still run over them (a
        # head norm, a rotation) the key and value parts it expects are zeros that nothing stores
        head_kernel = self.own_kv or self.q_norm is not None or self.position.rotary_dim > 0
        width = (H + 2 * G) * D if head_kernel else H * D
        if self.own_kv:
            qkv = torch.empty((T, width), dtype=self.dtype, device=x.device)
            ops.linear(x, self.w_qkv, qkv, self.b_qkv)
        elif head_kernel:
            qkv = torch.zeros((T, width), dtype=self.dtype, device=x.device)
            q_only = torch.empty((T, H * D), dtype=self.dtype, device=x.device)
            ops.linear(x, self.w_qkv, q_only, self.b_qkv)
            qkv[:, :H * D] = q_only
        else:
            qkv = torch.empty((T, width), dtype=self.dtype, device=x.device)
            ops.linear(x, self.w_qkv, qkv, self.b_qkv)
        if self.q_whole is not None:
            spans = [(0, H * D, self.q_whole, H * self.key_dim)]
            if self.own_kv:
                spans.append((H * D, G * D, self.k_whole, G * self.key_dim))
            ops.span_rmsnorm(qkv, spans, self.eps)
        if self.value_inv_freq is not None and self.own_kv:
            ops.turn_heads(qkv[:, (H + G) * D:], G, D, self.value_dim, self.position.style, batch.positions,
                           self.value_inv_freq, 1.0)
        slots = batch.slots[cache.group] if (cache.writes and self.own_kv) else batch.no_slots
        if head_kernel:
            ops.qk_norm_rope_cache(qkv, self.q_norm, self.k_norm, self.eps, batch.positions, self.position.inv_freq,
                                   self.position.rotary_dim, self.position.style, slots, cache.k, cache.v, H, G, D)
        attn = torch.empty((T, H * D), dtype=self.dtype, device=x.device)
        ops.attention(qkv, width, attn, cache.k, cache.v, batch, H, G, D, self.scale, self.window, cache.group,
                      softcap=self.softcap, distance=self.distance)
        if self.value_inv_freq is not None or self.w_gate is not None:
            gate = None
            if self.w_gate is not None:
                gate = torch.empty((T, H * D), dtype=self.dtype, device=x.device)
                ops.linear(x, self.w_gate, gate)
            turned = self.value_dim if self.value_inv_freq is not None else 0
            ops.turn_heads(attn, H, D, turned, self.position.style, batch.positions, self.value_inv_freq, -1.0,
                           gate=gate, gate_stride=D)
        out = torch.empty((T, self.spec.hidden), dtype=torch.float32, device=x.device)
        ops.linear(attn, self.w_o, out)
        return out

    def forward(self, x, batch, cache: LayerCache, resid: Optional[torch.Tensor] = None,
                emit: Optional[NormTarget] = None):
        if self.extended:
            return self._forward_extended(split_input(x)[0], batch, cache)
        ops = kernels.current()
        x, row_sums = split_input(x)
        T = x.shape[0]
        slots = batch.slots[cache.group] if cache.writes else batch.no_slots
        # a product that the kernels cut into K ranges may hand them over unadded: the kernel behind it
        # adds them as it reads, which saves the adding kernel (and applies a carried norm's row factor)
        in_ranges = getattr(ops, "linear_ranges", None)
        ranges = in_ranges(x, self.w_qkv) if in_ranges is not None and self.b_qkv is None else None
        if ranges is not None:
            q_rows, q_stride = torch.empty((T, self.num_heads * self.head_dim), dtype=self.dtype, device=x.device), \
                self.num_heads * self.head_dim
            ops.qk_norm_rope_cache_ranges(ranges, row_sums, q_rows, self.q_norm, self.k_norm, self.eps,
                                          batch.positions, self.position.inv_freq, self.position.rotary_dim,
                                          self.position.style, slots, cache.k, cache.v, self.num_heads,
                                          self.num_kv_heads, self.head_dim)
        else:
            q_rows, q_stride = torch.empty((T, self.qkv_width), dtype=self.dtype, device=x.device), self.qkv_width
            if row_sums is None:
                ops.linear(x, self.w_qkv, q_rows, self.b_qkv)
            else:
                ops.linear_skinny(x, self.w_qkv, q_rows, self.b_qkv, row_sums=row_sums)
            ops.qk_norm_rope_cache(q_rows, self.q_norm, self.k_norm, self.eps, batch.positions,
                                   self.position.inv_freq, self.position.rotary_dim, self.position.style,
                                   slots, cache.k, cache.v, self.num_heads, self.num_kv_heads, self.head_dim)
        attn = torch.empty((T, self.num_heads * self.head_dim), dtype=self.dtype, device=x.device)
        ops.attention(q_rows, q_stride, attn, cache.k, cache.v, batch, self.num_heads,
                      self.num_kv_heads, self.head_dim, self.scale, self.window, cache.group)
        can_add = getattr(ops, "can_accumulate", None)
        if resid is not None and can_add and can_add(attn, self.w_o):
            # x += attn . Wo^T in the epilogue, which can also prepare the norm that follows
            if emit is not None and emit.finished:
                done = ops.linear_skinny(attn, self.w_o, resid, accumulate=True, finish=emit.finish)
                return emit if done else None
            if emit is not None:
                written = ops.linear_skinny(attn, self.w_o, resid, accumulate=True, emit=emit.emit)
                emit.ss = emit.ss[:written]          # as many partial sums a row as the kernel that ran has workgroups
                return emit
            ops.linear_skinny(attn, self.w_o, resid, accumulate=True)
            return None
        out = torch.empty((T, self.spec.hidden), dtype=self.dtype, device=x.device)
        ops.linear(attn, self.w_o, out)
        return out
