"""Tiny Gibavik configurations and model folders for the tests.

The configurations differ in every size and option: layer order (a side-by-side layer first or last, attention
layers alone), width (a multiple of 8 or not), query heads in groups of 1, 2 and 8 a key head, key sizes that are no
multiple of 16 with value sizes above and below them, a layer that reads the keys of an earlier one (next to it or
further back), windows of 5, 21 and 40 and none, rotation over a whole head or part of one, memories of one and
several heads with key sizes on either side of the scan kernels' switch of lanes a column, experts looked up by
twos, all of them, or one of one, layers with no feed-forward, caps, factors and scales present and absent.

Random weights are drawn so that attention scores are of order one: softmax weights are uneven, and a wrong key, a
window that is one off or a lost state changes the logits visibly.
"""
from __future__ import annotations

import json
import os
from typing import Dict, Optional

import torch

from reinfer_amd.config import config_from_dict
from reinfer_amd.models import declare_params
from reinfer_amd.weights import random_tensors
from reinfer_amd.weights.safetensors_io import write_safetensors


def _attn(heads, kv, dim, vdim, scale=None, kv_from=None, window=None):
    m = {"dim": dim, "heads": heads, "kv_heads": kv, "scale": dim ** -0.5 if scale is None else scale, "vdim": vdim}
    if kv_from is not None:
        m["kv_from"] = kv_from
    if window:
        m["mask"] = {"size": window}
    return m


def _left(heads, kv, dim, vdim, window, dims, base=10000.0, cap=25.0, scale=None):
    m = {"dim": dim, "heads": heads, "kv_heads": kv, "scale": dim ** -0.5 if scale is None else scale, "vdim": vdim}
    if window:
        m["mask"] = {"size": window}
    if dims:
        m["rot"] = {"base": base, "dims": dims}
    if cap:
        m["softcap"] = cap
    return m


def _right(heads, dim, vdim, decay):
    return {"decay": list(decay), "dim": dim, "heads": heads, "vdim": vdim}


def _pair(left, right, ls=None, rs=None):
    m = {"left": left, "right": right}
    if ls is not None:
        m["left_scale"] = ls
    if rs is not None:
        m["right_scale"] = rs
    return m


def _moe(experts, top, ff):
    return {"expert": {"ff": ff}, "kind": "moe", "router": {"experts": experts, "top": top}}


def _dense(ff, limit):
    return {"ff": ff, "kind": "dense", "limit": limit}


GB_A = {
    "architecture": "Gibavik", "vocab": 300, "width": 64, "norm": {"eps": 1e-5}, "embedding": {"scale": 4.0},
    "logit_softcap": 12.0,
    "layers": [
        {"type": "parallel", "mixer": _pair(_left(4, 2, 24, 16, 21, 12, cap=6.0), _right(3, 20, 12, (0.5, 0.9, 0.99)),
                                            0.7, 1.1),
         "mlp": _moe(6, 2, 24)},
        {"type": "attention", "mixer": _attn(4, 2, 24, 40), "mlp": _dense(96, 0.8)},
        {"type": "attention", "mixer": _attn(4, 2, 24, 40, scale=0.3, kv_from=1), "mlp": None},
        {"type": "parallel", "mixer": _pair(_left(2, 2, 16, 8, 5, 16, base=500.0, scale=0.3),
                                            _right(1, 40, 8, (0.97,)), 1.3, 0.4),
         "mlp": _moe(3, 3, 16)},
    ],
}
# attention layers alone, one query head a key head, a width that is no multiple of 8, no scale and no cap given
GB_B = {
    "architecture": "Gibavik", "vocab": 131, "width": 36, "norm": {"eps": 3e-6},
    "layers": [
        {"type": "attention", "mixer": _attn(3, 3, 8, 8), "mlp": _dense(40, 2.0)},
        {"type": "attention", "mixer": _attn(5, 1, 12, 20), "mlp": None},
        {"type": "attention", "mixer": _attn(3, 3, 8, 8, kv_from=0), "mlp": _dense(24, 0.5)},
    ],
}
# for bfloat16: head sizes the matrix-core kernels take as they are; eight query heads on one key head
GB_C = {
    "architecture": "Gibavik", "vocab": 257, "width": 96, "norm": {"eps": 1e-6}, "embedding": {"scale": 6.0},
    "logit_softcap": 30.0,
    "layers": [
        {"type": "attention", "mixer": _attn(8, 1, 32, 16), "mlp": _moe(4, 2, 32)},
        {"type": "parallel", "mixer": _pair(_left(8, 4, 32, 32, 40, 8, base=100000.0), _right(2, 32, 48, (0.8, 0.995)),
                                            0.5, 1.0),
         "mlp": _dense(128, 1.5)},
        {"type": "attention", "mixer": _attn(8, 1, 32, 16, kv_from=0), "mlp": _moe(4, 4, 16)},
        {"type": "parallel", "mixer": _pair(_left(3, 3, 48, 16, 17, 48), _right(4, 16, 16, (0.3, 0.6, 0.9, 0.999)),
                                            1.0, 1.0),
         "mlp": None},
    ],
}
# whatever may be absent is absent: no window, no rotation (the values then do not turn), no caps, no factors, no
# embedding scale; one expert of one; a side-by-side layer first
GB_D = {
    "architecture": "Gibavik", "vocab": 90, "width": 40, "norm": {"eps": 1e-6},
    "layers": [
        {"type": "parallel", "mixer": {"left": {"dim": 16, "heads": 5, "kv_heads": 5, "vdim": 8},
                                       "right": _right(3, 8, 16, (0.9, 0.8, 0.7))},
         "mlp": _moe(1, 1, 24)},
        {"type": "attention", "mixer": {"dim": 8, "heads": 2, "kv_heads": 1, "vdim": 24}, "mlp": _dense(56, 1.0)},
    ],
}
CONFIGS = {"A": (GB_A, 31), "B": (GB_B, 32), "C": (GB_C, 33), "D": (GB_D, 34)}

# deviation of the random matrices by the last part of their name
STD = {"embed": 0.5, "head": 0.3, "b": 0.3, "default": 0.15}


def draw_weights(raw: dict, seed: int, dtype: torch.dtype = torch.float32, scales: Optional[Dict[str, float]] = None,
                 shifts: Optional[Dict[str, float]] = None):
    """name -> tensor of the random model of ``raw`` and ``seed``. The distance term's second number is drawn
    small (0.1 to 0.5 a token); ``scales`` multiplies and ``shifts`` adds to named tensors (a name's last part,
    or its last two, stand for every layer's tensor)."""
    cfg = config_from_dict(raw)
    out = {}
    g = torch.Generator().manual_seed(seed)
    for d in declare_params(cfg.to_spec()):
        if d.optional:
            continue
        last = d.name.rsplit(".", 1)[-1]
        t = random_tensors([d], seed, torch.float32, std=STD.get(d.name if d.name in STD else last, STD["default"]))[d.name]
        if last == "r2":
            t = 0.1 + 0.4 * torch.rand(d.shape, generator=g)
        elif last == "r1":
            t = 0.3 + 1.2 * torch.rand(d.shape, generator=g)
        out[d.name] = t
    for table, f in ((scales, lambda t, v: t * v), (shifts, lambda t, v: t + v)):
        for name, v in (table or {}).items():
            hit = [n for n in out if n == name or n.endswith("." + name)]
            assert hit, name
            for n in hit:
                out[n] = f(out[n], v)
    return {n: (t.to(dtype) if t.is_floating_point() else t) for n, t in out.items()}


def write_folder(out: str, raw: dict, weights: Dict[str, torch.Tensor]) -> str:
    os.makedirs(out, exist_ok=True)
    with open(os.path.join(out, "config.json"), "w", encoding="utf-8") as f:
        json.dump(raw, f, indent=1)
    write_safetensors(os.path.join(out, "model.safetensors"), weights, metadata={"format": "pt"})
    return out


def make_folder(tmp_path, which: str, dtype: str = "bfloat16", scales=None, shifts=None, tag: str = "") -> str:
    raw, seed = CONFIGS[which]
    out = os.path.join(str(tmp_path), f"gibavik_{which}_{dtype}{tag}")
    if not os.path.isdir(out):
        tdtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[dtype]
        write_folder(out, raw, draw_weights(raw, seed, tdtype, scales, shifts))
    return out


def read_folder(path: str, dtype=torch.float64):
    """(raw config dict, name -> CPU tensor: floats in ``dtype``, integer tables as they are) for the plain
    implementation."""
    from reinfer_amd.weights import SafetensorsFile
    with open(os.path.join(path, "config.json")) as f:
        raw = json.load(f)
    with SafetensorsFile(os.path.join(path, "model.safetensors")) as sf:
        weights = {}
        for n in sf.names():
            t = sf.tensor(n).clone()
            weights[n] = t.to(dtype) if t.is_floating_point() else t
    return raw, weights
