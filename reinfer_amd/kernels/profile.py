"""Per-kernel-class GPU time of a step, measured with events around every call
into the kernel set.

    timed = TimedKernels(kernels.current())
    timed.name_weight(block.mixer.w_qkv, "qkv")          # products are classed by their weight
    with kernels.use(timed):
        timed.hold_back(20.0)                            # the GPU busy elsewhere while the step is queued
        runner.step(entries)
    rows = timed.report()                                # class -> calls, milliseconds

The reference brackets the segments of its decode step the same way, with
events on the stream (crates/cuda/src/engine.rs:1146-1408) and prints them with
``--perf`` (bin/reinfer/src/main.rs:706-727). Two things make the figures mean
what a captured step costs: the step is queued behind work that keeps the GPU
busy meanwhile (``hold_back``), so that no kernel waits for the host between
its two events; and an event pair costs the stream about a microsecond, which
``report`` measures on an empty pair and takes off every class.
"""
from __future__ import annotations

from typing import Any, Callable, Dict, List, Optional, Tuple

import torch

# methods of the kernel set that launch work, and how their calls are classed
_ROWS = {"embed": "embedding", "add_rmsnorm": "norm", "silu_mul": "gate", "sample": "sampler",
         "filter_logits": "sampler"}
_QK = {"qk_norm_rope_cache", "qk_norm_rope_cache_ranges"}
_ATTN = {"attention", "attention_plain", "attention_decode", "attention_prefill"}
_LINEAR = {"linear", "linear_plain", "linear_skinny", "gated_linear", "linear_ranges"}
# kernels of further mechanisms, each a class of its own
_OTHER = {"latent_prep": "latent norm + rotation + cache write", "head_linear": "products head by head",
          "moe_route": "router", "moe_relu2_scale": "expert activation",
          "moe_up_chosen": "chosen experts up", "moe_down_chosen": "chosen experts down",
          "moe_gate_up_chosen": "chosen experts up", "moe_down_gated_chosen": "chosen experts down", "stream_add": "stream add",
          "pair_hash_add": "embedding", "tanh_cap": "logit cap",
          "matrix_memory_scan": "matrix memory scan", "delta_rule_prepare": "filter + unit norms",
          "delta_rule_scan": "delta rule scan", "head_norm_gate": "head norm + gate",
          "normed_mean": "mean of normed mixers", "moe_silu_gate_scale": "expert activation",
          "wkv_scan": "wkv scan", "token_shift": "mix with the row before", "gated_stream_add": "gated stream add",
          "rows_rmsnorm": "row norm", "tanh_rows": "tanh", "moe_identity_add": "identity experts",
          "stream_cast": "stream as operand", "sum_norm_add": "sum + norm + stream add",
          "span_rmsnorm": "projection norm", "turn_heads": "turn of heads (+ gate)", "decay_scan": "decay scan",
          "moe_table_route": "router"}


class TimedKernels:
    """A kernel set that times every call of the set it wraps."""

    def __init__(self, inner):
        self._inner = inner
        self._names: Dict[int, str] = {}
        self._spans: List[Tuple[str, torch.cuda.Event, torch.cuda.Event, int, int]] = []
        self._filler: Optional[torch.Tensor] = None
        self.name = getattr(inner, "name", "timed")

    def name_weight(self, weight: torch.Tensor, role: str) -> None:
        self._names[weight.data_ptr()] = role

    def _label(self, method: str, args, kwargs) -> str:
        if method in _ROWS:
            return _ROWS[method]
        if method in _QK:
            return "head norm + rotation + cache write"
        if method in _ATTN:
            return "attention"
        if method in _OTHER:
            return _OTHER[method]
        if method in _LINEAR:
            w = args[1] if len(args) > 1 else kwargs.get("weight")
            role = self._names.get(w.data_ptr()) if isinstance(w, torch.Tensor) else None
            return role or f"product {w.shape[0]}x{w.shape[1]}"
        return method

    def __getattr__(self, attr: str) -> Any:
        target = getattr(self._inner, attr)
        if not callable(target) or not (attr in _ROWS or attr in _QK or attr in _ATTN or attr in _LINEAR
                                        or attr in _OTHER):
            return target

        def timed_call(*args, **kwargs):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            out = target(*args, **kwargs)
            e1.record()
            # what a product must read (its weight) and compute, for pricing the class against the machine
            nbytes = flops = 0
            w = None
            if attr in _LINEAR:
                w = args[1] if len(args) > 1 else kwargs.get("weight")
            elif attr == "head_linear":
                w = args[2] if len(args) > 2 else kwargs.get("weight")
            if isinstance(w, torch.Tensor) and isinstance(args[0], torch.Tensor):
                nbytes = w.numel() * w.element_size()
                flops = 2 * args[0].shape[0] * w.numel()
            if attr == "linear_ranges" and out is None:
                return out                # it declined (the caller runs the whole product next): nothing was launched
            self._spans.append((self._label(attr, args, kwargs), e0, e1, nbytes, flops))
            return out
        return timed_call

    def hold_back(self, milliseconds: float, device="cuda:0") -> None:
        """Queue about this much reading of a large buffer, so that the host can queue a whole step
        behind it (the step's kernels then run back to back, as in a replayed graph)."""
        size = 2 << 30
        if self._filler is None:
            self._filler = torch.empty(size // 4, dtype=torch.int32, device=device).random_()
            self._sink = torch.zeros(1, dtype=torch.int32, device=device)
        from . import library
        reads = max(1, int(milliseconds / (size / 5.5e12 * 1e3)))
        for _ in range(reads):
            library.call("ra_stream_read", self._filler.data_ptr(), size, self._sink.data_ptr(),
                         torch.cuda.current_stream().cuda_stream)

    def report(self) -> Dict[str, Dict[str, float]]:
        """class -> {"calls", "ms", "bytes", "flops"} (the last two for products: weight bytes read, flops);
        clears what was recorded."""
        pairs = []
        for _ in range(16):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            e1.record()
            pairs.append((e0, e1))
        torch.cuda.synchronize()
        empty = sorted(a.elapsed_time(b) for a, b in pairs)[len(pairs) // 2]
        out: Dict[str, Dict[str, float]] = {}
        for label, e0, e1, nbytes, flops in self._spans:
            row = out.setdefault(label, {"calls": 0, "ms": 0.0, "bytes": 0, "flops": 0})
            row["calls"] += 1
            row["ms"] += max(0.0, e0.elapsed_time(e1) - empty)
            row["bytes"] += nbytes
            row["flops"] += flops
        self._spans = []
        return out
