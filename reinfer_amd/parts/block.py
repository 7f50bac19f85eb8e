"""How norm, mixer and feed-forward are arranged in a layer.

"outnorm": x += norm1(mixer(x)); x += norm2(ffn(x)): the parts read the stream itself and the norm stands on
each part's result alone (a layer may have no feed-forward).

"prenorm": x += mixer(norm(x)); x += ffn(norm(x))
(crates/cuda/src/engine.rs:4075-4314); with ``residual_scale`` s both addends enter times s, and a layer
may have no feed-forward (then it has no second norm either). The residual stream is float. A block
gets the stream and the previous block's last addend, not yet added, so that
the add and the norm are one kernel (the reference fuses the same pair for the
o-projection, dense_kernels.cu:257-274); it returns its own last addend, or
None if its last part added it into the stream itself.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..config.schema import BlockSpec
from ..weights import VECTOR, ParamDecl
from .base import JointNeed, LayerCache, ScaledTerms, StateNeed, StreamCopy
from .registry import lookup, register_block


@register_block("prenorm")
class PreNormBlock:
    @classmethod
    def declare_params(cls, spec: BlockSpec) -> List[ParamDecl]:
        p = spec.prefix
        out = lookup("norm", spec.mixer_norm.kind).declare_params(spec.mixer_norm, p + spec.mixer_norm_name)
        out += lookup("mixer", spec.mixer.kind).declare_params(spec.mixer, p + spec.mixer_prefix)
        if spec.ffn is not None:
            out += lookup("norm", spec.ffn_norm.kind).declare_params(spec.ffn_norm, p + spec.ffn_norm_name)
            out += lookup("feed_forward", spec.ffn.kind).declare_params(spec.ffn, p + spec.ffn_prefix)
        return out

    def __init__(self, spec: BlockSpec, weights: Dict[str, torch.Tensor], dtype: torch.dtype,
                 device: torch.device):
        missing = [n for n in ("mixer", "mixer_norm") if getattr(spec, n) is None]
        if spec.ffn is not None and spec.ffn_norm is None:
            missing.append("ffn_norm")
        if missing:
            raise ValueError(f"a prenorm block is made of a mixer with a norm before it and at most a feed-forward "
                             f"with a norm before it; block {spec.prefix!r} names no {', '.join(missing)}")
        p = spec.prefix
        self.spec = spec
        self.mixer_norm = lookup("norm", spec.mixer_norm.kind)(spec.mixer_norm, weights,
                                                               p + spec.mixer_norm_name, dtype, device)
        self.mixer = lookup("mixer", spec.mixer.kind)(spec.mixer, weights, p + spec.mixer_prefix, dtype, device)
        self.ffn_norm = self.ffn = None
        if spec.ffn is not None:
            self.ffn_norm = lookup("norm", spec.ffn_norm.kind)(spec.ffn_norm, weights,
                                                               p + spec.ffn_norm_name, dtype, device)
            self.ffn = lookup("feed_forward", spec.ffn.kind)(spec.ffn, weights, p + spec.ffn_prefix, dtype, device)
        self.residual_scale = float(spec.residual_scale)
        # the norm-on-products hand-over is for the plain form: both parts there, addends entering as they are
        self.passes_emit = self.ffn is not None and self.residual_scale == 1.0

    @property
    def graph_safe(self) -> bool:
        return bool(getattr(self.mixer, "graph_safe", False)
                    and (self.ffn is None or getattr(self.ffn, "graph_safe", False)))

    def cache_need(self):
        """What this layer keeps between steps: its mixer's need."""
        return self.mixer.cache_need() if hasattr(self.mixer, "cache_need") else None

    def parts(self):
        """The parts this arrangement is made of (for whoever asks every part something)."""
        return tuple(p for p in (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn) if p is not None)

    def entry_target(self, resid: torch.Tensor):
        """A NormTarget for this block's first norm, for the part that runs before the block, or
        None if the norm or the mixer behind it cannot use one."""
        if not hasattr(self.mixer_norm, "emit_target"):
            return None
        return self.mixer_norm.emit_target(resid, getattr(self.mixer, "takes_row_scaled", False))

    def forward(self, resid: torch.Tensor, delta, batch, cache: Optional[LayerCache], emit=None):
        # A part that declares ``adds_in_place`` also gets the residual stream: where its last
        # product can add into it, it does and returns None; any other part returns its addend.
        # Where that product can also prepare the norm that follows (the part ``emits_for_norm``,
        # the norm offers a target, and the part behind the norm ``takes_row_scaled``), the norm
        # costs no kernel: its column weight is applied by the product before it, its row
        # factor by the product after it.
        mixer, ffn = self.mixer, self.ffn
        if ffn is None or self.residual_scale != 1.0:
            return self._forward_scaled(resid, delta, batch, cache)
        xn = self._norm(self.mixer_norm, resid, delta, mixer)
        if getattr(mixer, "adds_in_place", False):
            tgt = self._target(self.ffn_norm, resid, mixer, ffn)
            if tgt is not None:
                a = mixer.forward(xn, batch, cache, resid=resid, emit=tgt)
            else:
                a = mixer.forward(xn, batch, cache, resid=resid)
        else:
            a = mixer.forward(xn, batch, cache)
        xn = self._norm(self.ffn_norm, resid, a, ffn)
        if getattr(ffn, "adds_in_place", False):
            if emit is not None and getattr(ffn, "emits_for_norm", False):
                return ffn.forward(xn, batch, resid=resid, emit=emit)
            return ffn.forward(xn, batch, resid=resid)
        return ffn.forward(xn, batch)

    def _forward_scaled(self, resid: torch.Tensor, delta, batch, cache: Optional[LayerCache]):
        """x += s * mixer(norm(x)); x += s * ffn(norm(x)), the sums in the float stream. A part that declares
        ``adds_scaled`` adds s times its result into the stream itself (``forward(..., resid=, resid_scale=)``
        returns None then); any other part's addend is added by the norm that follows it, or, the block's
        last one, by the stream-add kernel: this block hands no pending addend on, since whoever adds it
        would not know its factor."""
        from .. import kernels
        s = self.residual_scale
        if not isinstance(delta, torch.Tensor) and delta is not None:
            delta = None               # a filled norm target: the sum is already in the stream
        xn = self.mixer_norm.add_norm(resid, delta)
        a = self._run(self.mixer, xn, batch, resid, s, cache)
        if self.ffn is not None:
            xn = self.ffn_norm.add_norm(resid, a, delta_scale=s) if a is not None else self.ffn_norm.add_norm(resid, None)
            a = self._run(self.ffn, xn, batch, resid, s)
        if a is not None:
            kernels.current().stream_add(resid, a, delta_scale=s)
        return None

    @staticmethod
    def _run(part, xn, batch, resid, s, *cache):
        if getattr(part, "adds_scaled", False):
            return part.forward(xn, batch, *cache, resid=resid, resid_scale=s)
        return part.forward(xn, batch, *cache)

    @staticmethod
    def _norm(norm, resid, delta, consumer):
        if hasattr(norm, "emit_target"):
            return norm.add_norm(resid, delta, scaled_ok=getattr(consumer, "takes_row_scaled", False))
        if not isinstance(delta, torch.Tensor) and delta is not None:
            delta = None               # a filled target: the sum is already in the stream
        return norm.add_norm(resid, delta)

    @staticmethod
    def _target(norm, resid, producer, consumer):
        if not (getattr(producer, "emits_for_norm", False) and hasattr(norm, "emit_target")):
            return None
        return norm.emit_target(resid, getattr(consumer, "takes_row_scaled", False))


@register_block("parallel")
class ParallelBlock:
    """h = norm(x); x += mixer(h) + ffn(h): one norm, and both parts read its output. A block without a
    feed-forward (``spec.ffn`` None) is x += mixer(norm(x)). The sums are float: a part that can add its last
    product into the stream does so, any other addend goes through the stream-add kernel or, the last one,
    back to the caller, whose next norm adds it.

    Two options (``spec.params``, a :class:`ParallelSpec`). ``token_shift``: the mixer reads
    h + (h' - h) * s, h' being the normed row of the token before (zeros for a request's first token); the
    feed-forward reads h as it is. The last h of a portion is kept in the request's state, so the layer's cache
    is the mixer's and, beside it, one row of the width. ``gated``: x += sigmoid(W1 h + b1) * mixer(...) +
    sigmoid(W2 h + b2) * ffn(h); both gates come from one product over h and the sum is one float kernel."""

    @staticmethod
    def _options(spec: BlockSpec):
        o = spec.params
        return (bool(getattr(o, "token_shift", False)), bool(getattr(o, "gated", False)),
                str(getattr(o, "shift_name", "shift")), tuple(getattr(o, "gate_names", ("rg1", "rg2"))))

    @classmethod
    def declare_params(cls, spec: BlockSpec) -> List[ParamDecl]:
        p = spec.prefix
        out = lookup("norm", spec.mixer_norm.kind).declare_params(spec.mixer_norm, p + spec.mixer_norm_name)
        out += lookup("mixer", spec.mixer.kind).declare_params(spec.mixer, p + spec.mixer_prefix)
        if spec.ffn is not None:
            out += lookup("feed_forward", spec.ffn.kind).declare_params(spec.ffn, p + spec.ffn_prefix)
        shift, gated, shift_name, gate_names = cls._options(spec)
        w = spec.mixer_norm.size
        if shift:
            out.append(ParamDecl(p + shift_name, (w,), role=VECTOR))
        if gated:
            for name in gate_names[:2 if spec.ffn is not None else 1]:
                out += [ParamDecl(p + name, (w, w)), ParamDecl(p + name + ".b", (w,), init="zeros", role=VECTOR)]
        return out

    def __init__(self, spec: BlockSpec, weights: Dict[str, torch.Tensor], dtype: torch.dtype,
                 device: torch.device):
        missing = [n for n in ("mixer", "mixer_norm") if getattr(spec, n) is None]
        if missing:
            raise ValueError(f"a parallel block is made of one norm, a mixer and at most a feed-forward; "
                             f"block {spec.prefix!r} names no {', '.join(missing)}")
        p = spec.prefix
        self.spec = spec
        self.norm = lookup("norm", spec.mixer_norm.kind)(spec.mixer_norm, weights, p + spec.mixer_norm_name,
                                                         dtype, device)
        self.mixer = lookup("mixer", spec.mixer.kind)(spec.mixer, weights, p + spec.mixer_prefix, dtype, device)
        self.ffn = None
        if spec.ffn is not None:
            self.ffn = lookup("feed_forward", spec.ffn.kind)(spec.ffn, weights, p + spec.ffn_prefix, dtype, device)
        self.dtype = dtype
        self.width = int(spec.mixer_norm.size)
        self.token_shift, self.gated, shift_name, gate_names = self._options(spec)
        if self.token_shift:
            self.shift = weights[p + shift_name].to(dtype).view(1, self.width).contiguous()
        if self.gated:
            names = gate_names[:2 if self.ffn is not None else 1]
            # both gates' pre-activations from one product over h: rows of the mixer's gate, then the feed-forward's
            self.w_gates = torch.cat([weights[p + n] for n in names], dim=0).contiguous()
            self.b_gates = torch.cat([weights[p + n + ".b"] for n in names], dim=0).to(self.w_gates.dtype).contiguous()

    @property
    def graph_safe(self) -> bool:
        return bool(getattr(self.mixer, "graph_safe", False)
                    and (self.ffn is None or getattr(self.ffn, "graph_safe", False)))

    def cache_need(self):
        need = self.mixer.cache_need() if hasattr(self.mixer, "cache_need") else None
        if self.token_shift:
            # the mixer's own need and, beside it, the last normed row of the request
            return JointNeed((need, StateNeed((self.width,), torch.float32)))
        return need

    def parts(self):
        return tuple(p for p in (self.norm, self.mixer, self.ffn) if p is not None)

    def _forward_shift_gate(self, resid: torch.Tensor, h: torch.Tensor, batch, cache: Optional[LayerCache]):
        """The block with a token shift and / or gates on its addends: nothing is left pending."""
        from .. import kernels
        ops = kernels.current()
        T = h.shape[0]
        mixer_cache, hs = cache, h
        if self.token_shift:
            mixer_cache, kept = cache.members
            hs = torch.empty_like(h)
            ops.token_shift(h, self.shift, kept.state, 0, batch, hs)
        a = self.mixer.forward(hs, batch, mixer_cache)
        b = self.ffn.forward(h, batch) if self.ffn is not None else None
        if self.gated:
            gates = torch.empty((T, self.w_gates.shape[0]), dtype=self.dtype, device=h.device)
            ops.linear(h, self.w_gates, gates, self.b_gates)
            ops.gated_stream_add(resid, gates, a, b)
            return None
        ops.stream_add(resid, a)
        return b

    def forward(self, resid: torch.Tensor, delta, batch, cache: Optional[LayerCache]):
        from .. import kernels
        if not isinstance(delta, torch.Tensor) and delta is not None:
            delta = None               # a filled norm target: the sum is already in the stream
        h = self.norm.add_norm(resid, delta)          # the stream now holds everything before this block
        if self.token_shift or self.gated:
            return self._forward_shift_gate(resid, h, batch, cache)
        addends = []
        if getattr(self.mixer, "adds_in_place", False):
            a = self.mixer.forward(h, batch, cache, resid=resid)
        else:
            a = self.mixer.forward(h, batch, cache)
        if a is not None:
            addends.append(a)
        if self.ffn is not None:
            if getattr(self.ffn, "adds_in_place", False):
                b = self.ffn.forward(h, batch, resid=resid)
            else:
                b = self.ffn.forward(h, batch)
            if b is not None:
                addends.append(b)
        for a in addends[:-1]:
            kernels.current().stream_add(resid, a)
        return addends[-1] if addends else None


@register_block("outnorm")
class OutNormBlock:
    """x <- x + norm1(mixer(x)); x <- x + norm2(ffn(x)): both parts read the residual stream itself (in the
    activations' type for their products), and each result is normed before it enters. The stream and the norms
    are float. One kernel forms the part's result (a sum of scaled terms where the mixer hands back several),
    norms it, adds it into the stream and writes the new stream in the activations' type for the part that reads
    it next; the last copy is handed on to the next block (:class:`StreamCopy`). A block without a feed-forward
    (``spec.ffn`` None) has no second norm."""

    @classmethod
    def declare_params(cls, spec: BlockSpec) -> List[ParamDecl]:
        p = spec.prefix
        out = lookup("norm", spec.mixer_norm.kind).declare_params(spec.mixer_norm, p + spec.mixer_norm_name)
        out += lookup("mixer", spec.mixer.kind).declare_params(spec.mixer, p + spec.mixer_prefix)
        if spec.ffn is not None:
            out += lookup("norm", spec.ffn_norm.kind).declare_params(spec.ffn_norm, p + spec.ffn_norm_name)
            out += lookup("feed_forward", spec.ffn.kind).declare_params(spec.ffn, p + spec.ffn_prefix)
        return out

    def __init__(self, spec: BlockSpec, weights: Dict[str, torch.Tensor], dtype: torch.dtype,
                 device: torch.device):
        missing = [n for n in ("mixer", "mixer_norm") if getattr(spec, n) is None]
        if spec.ffn is not None and spec.ffn_norm is None:
            missing.append("ffn_norm")
        if missing:
            raise ValueError(f"an outnorm block is made of a mixer with a norm behind it and at most a feed-forward "
                             f"with a norm behind it; block {spec.prefix!r} names no {', '.join(missing)}")
        p = spec.prefix
        self.spec, self.dtype = spec, dtype
        self.mixer_norm = lookup("norm", spec.mixer_norm.kind)(spec.mixer_norm, weights, p + spec.mixer_norm_name,
                                                               dtype, device)
        self.mixer = lookup("mixer", spec.mixer.kind)(spec.mixer, weights, p + spec.mixer_prefix, dtype, device)
        self.ffn_norm = self.ffn = None
        if spec.ffn is not None:
            self.ffn_norm = lookup("norm", spec.ffn_norm.kind)(spec.ffn_norm, weights, p + spec.ffn_norm_name,
                                                               dtype, device)
            self.ffn = lookup("feed_forward", spec.ffn.kind)(spec.ffn, weights, p + spec.ffn_prefix, dtype, device)
        for n in (self.mixer_norm, self.ffn_norm):
            if n is not None and getattr(n, "groups", 1) != 1:
                raise ValueError("an outnorm block norms a part's result over the whole width")

    @property
    def graph_safe(self) -> bool:
        return bool(getattr(self.mixer, "graph_safe", False)
                    and (self.ffn is None or getattr(self.ffn, "graph_safe", False)))

    def cache_need(self):
        return self.mixer.cache_need() if hasattr(self.mixer, "cache_need") else None

    def parts(self):
        return tuple(p for p in (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn) if p is not None)

    @staticmethod
    def _norm_weight(norm):
        """The norm's weight as the kernel takes it: one float number, or a float vector over the width."""
        w = getattr(norm, "scalar", None)
        if w is None:
            w = norm.weight if norm.weight.dtype == torch.float32 else norm.weight.float()
        return w

    def _enter(self, ops, resid, y, norm, want_copy: bool):
        """resid += norm(y); -> the new stream in the activations' type (the stream itself where that is float)."""
        if isinstance(y, ScaledTerms):
            terms, scales = y.terms, y.scales
        else:
            terms, scales = [y], [1.0]
        copy = None
        if want_copy and self.dtype != torch.float32:
            copy = torch.empty(resid.shape, dtype=self.dtype, device=resid.device)
        ops.sum_norm_add(terms, scales, self._norm_weight(norm), norm.eps, resid=resid, copy=copy)
        return copy if copy is not None else resid

    def forward(self, resid: torch.Tensor, delta, batch, cache: Optional[LayerCache]):
        from .. import kernels
        ops = kernels.current()
        if isinstance(delta, StreamCopy) and delta.x.dtype == self.dtype and delta.x.shape == resid.shape:
            h = delta.x                       # the block before left the stream in the activations' type
        else:
            if isinstance(delta, torch.Tensor):
                ops.stream_add(resid, delta)
            if self.dtype == torch.float32:
                h = resid
            else:
                h = torch.empty(resid.shape, dtype=self.dtype, device=resid.device)
                ops.stream_cast(resid, h)
        if getattr(self.mixer, "returns_terms", False):
            a = self.mixer.forward(h, batch, cache, terms_ok=True)
        else:
            a = self.mixer.forward(h, batch, cache)
        h = self._enter(ops, resid, a, self.mixer_norm, True)
        if self.ffn is not None:
            b = self.ffn.forward(h, batch)
            h = self._enter(ops, resid, b, self.ffn_norm, True)
        return StreamCopy(h) if h is not resid else None
