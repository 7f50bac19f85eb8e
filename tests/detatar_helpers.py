"""Tiny Detatar configurations and model folders for the tests.

The configurations differ in every size and option: layer order (attention first or a wkv layer first, wkv layers
alone), a layer that runs an earlier layer's tensors again (a wkv layer, an attention layer), width (a multiple of 8
or not), the norm in 1, 2 and 3 groups, the embedding's scale (also absent), attention heads whose unrotated, rotated
and value sizes all differ, rotation on all or on part of the rotated entries, latents of queries and of keys of other
ranks, wkv heads of sizes on either side of the scan kernels' switch from 8 to 16 lanes a column, decays of several
ranks, experts in groups (2 of 4 kept, 1 of 2), in one group, all chosen, with 0, 1 and 2 identity experts, with and
without a shared expert, layers with no feed-forward.

Random weights are drawn so that attention scores, gates, decays and router logits are of order one: softmax weights
are uneven, the decays sit between 0.1 and 0.9, and a wrong key or a lost state changes the logits visibly.
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


def _latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, dims=None, base=10000.0, scale=None):
    out = {"dim": dim, "heads": heads, "kv_rank": kv_rank, "q_rank": q_rank, "rot_dim": rot_dim,
           "scale": (dim + rot_dim) ** -0.5 if scale is None else scale, "vdim": vdim}
    if rot_dim:
        out["rot"] = {"base": base, "dims": rot_dim if dims is None else dims}
    return out


def _wkv(heads, dim):
    return {"dim": dim, "heads": heads}


def _moe(experts, top, ff, identity=None, groups=None, shared=0):
    router = {"experts": experts, "top": top}
    if identity is not None:
        router["identity"] = identity
    if groups:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    out = {"expert": {"ff": ff}, "kind": "moe", "router": router}
    if shared:
        out["shared"] = {"ff": shared}
    return out


def _dense(ff):
    return {"ff": ff, "kind": "dense"}


# ``decay_ranks`` (the rows of a wkv layer's first decay matrix) stands in these dictionaries because a random
# model has no tensors yet to read it from; the config.json that make_folder writes leaves it out
DT_A = {
    "architecture": "Detatar", "vocab": 300, "width": 64, "norm": {"eps": 1e-5, "groups": 2},
    "embedding": {"scale": 2.5}, "decay_ranks": [0, 12, 0, 0],
    "layers": [
        {"type": "latent_attention", "mixer": _latent(3, 16, 8, 24, 40, 24),
         "mlp": _moe(6, 2, 24, identity=2, groups=(4, 2), shared=40)},
        {"type": "wkv", "mixer": _wkv(2, 20), "mlp": _dense(96)},
        {"type": "latent_attention", "mixer": _latent(5, 8, 16, 8, 24, 16, dims=12, base=500.0, scale=0.3),
         "mlp": None},
        {"type": "wkv", "mixer": _wkv(2, 20), "mlp": _dense(96), "weights_of": 1},
    ],
}
# wkv layers alone: no keys, so no block pool; a width that is no multiple of 8; three norm groups; no embedding
# scale; one expert chosen of three, no identity experts, no groups, no shared expert
DT_B = {
    "architecture": "Detatar", "vocab": 131, "width": 36, "norm": {"eps": 3e-6, "groups": 3}, "decay_ranks": [5, 8],
    "layers": [
        {"type": "wkv", "mixer": _wkv(4, 9), "mlp": _dense(40)},
        {"type": "wkv", "mixer": _wkv(1, 40), "mlp": _moe(3, 1, 16, identity=0)},
    ],
}
# for bfloat16: no comparison rests on which of two nearly equal scores is the larger after rounding (every expert
# and identity expert of the one group is chosen); eight heads on one cached row; a wkv layer first
DT_C = {
    "architecture": "Detatar", "vocab": 257, "width": 96, "norm": {"eps": 1e-6, "groups": 1},
    "embedding": {"scale": 2.0}, "decay_ranks": [16, 0, 0],
    "layers": [
        {"type": "wkv", "mixer": _wkv(3, 32), "mlp": _moe(3, 4, 32, identity=1, shared=16)},
        {"type": "latent_attention", "mixer": _latent(8, 16, 32, 48, 64, 40, base=100000.0), "mlp": _dense(128)},
        {"type": "latent_attention", "mixer": _latent(8, 16, 32, 48, 64, 40, base=100000.0), "mlp": _dense(128),
         "weights_of": 1},
    ],
}
# whatever may be absent is absent: no embedding scale, no norm groups, no identity key, no router groups, no shared
# expert; one expert of one; an attention layer first, a head with rotated entries alone
DT_D = {
    "architecture": "Detatar", "vocab": 90, "width": 40, "norm": {"eps": 1e-6}, "decay_ranks": [0, 4],
    "layers": [
        {"type": "latent_attention", "mixer": _latent(5, 0, 16, 8, 16, 8),
         "mlp": {"expert": {"ff": 24}, "kind": "moe", "router": {"experts": 1, "top": 1}}},
        {"type": "wkv", "mixer": _wkv(5, 8), "mlp": _moe(4, 2, 8, identity=2, groups=(2, 1))},
    ],
}
CONFIGS = {"A": (DT_A, 31), "B": (DT_B, 32), "C": (DT_C, 33), "D": (DT_D, 34)}

# deviation of the random matrices by the last part of their name
STD = {"embed": 0.5, "router": 0.5, "sg": 0.3, "w1": 0.3, "w2": 0.5, "u": 0.5, "rg1": 0.1, "rg2": 0.1, "default": 0.15}


def draw_weights(raw: dict, seed: int, dtype: torch.dtype = torch.float32, scales: Optional[Dict[str, float]] = None,
                 shifts: Optional[Dict[str, float]] = None):
    """name -> tensor of the random model of ``raw`` and ``seed``. Mixing factors are drawn between 0 and 1, the
    decays' biases so that the decays spread over (0.1, 0.9), gate biases and router corrections away from zero;
    ``scales`` multiplies and ``shifts`` adds to named tensors (a name's last part stands for every layer's tensor)."""
    cfg = config_from_dict(raw)
    out = {}
    g = torch.Generator().manual_seed(seed)
    for d in declare_params(cfg.to_spec()):
        if d.optional:
            continue
        parts = d.name.split(".")
        last = parts[-1]
        t = random_tensors([d], seed, torch.float32, std=STD.get(d.name if d.name in STD else last, STD["default"]))[d.name]
        if last == "shift" or (len(parts) >= 2 and parts[-2] == "mu"):
            t = torch.rand(d.shape, generator=g)
        elif last == "w0":
            t = torch.rand(d.shape, generator=g) * 3.0 - 2.2          # decays exp(-exp(w0)) from 0.9 down to 0.1
        elif last == "b":
            t = torch.randn(d.shape, generator=g) * 0.5
        elif last == "correction":
            t = torch.randn(d.shape, generator=g) * 0.1
        out[d.name] = t
    for table, f in ((scales, lambda t, v: t * v), (shifts, lambda t, v: t + v)):
        for name, v in (table or {}).items():
            hit = [n for n in out if n == name or n.endswith("." + name)]
            assert hit, name
            for n in hit:
                out[n] = f(out[n], v)
    return {n: t.to(dtype) for n, t in out.items()}


def config_json(raw: dict) -> dict:
    """``raw`` as a model folder holds it: the sizes that the tensors give are not written."""
    return {k: v for k, v in raw.items() if k != "decay_ranks"}


def make_folder(tmp_path, which: str, dtype: str = "bfloat16", scales=None, shifts=None, tag: str = "") -> str:
    raw, seed = CONFIGS[which]
    return write_folder(os.path.join(str(tmp_path), f"detatar_{which}_{dtype}{tag}"), raw, seed, dtype, scales, shifts)


def write_folder(out: str, raw: dict, seed: int, dtype: str = "bfloat16", scales=None, shifts=None) -> str:
    if not os.path.isdir(out):
        os.makedirs(out)
        tdtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[dtype]
        with open(os.path.join(out, "config.json"), "w", encoding="utf-8") as f:
            json.dump(config_json(raw), f, indent=1)
        write_safetensors(os.path.join(out, "model.safetensors"), draw_weights(raw, seed, tdtype, scales, shifts),
                          metadata={"format": "pt"})
    return out


def read_folder(path: str, dtype=torch.float64):
    """(raw config dict, name -> CPU tensor in ``dtype``) for the plain implementation."""
    from reinfer_amd.weights import SafetensorsFile
    with open(os.path.join(path, "config.json")) as f:
        raw = json.load(f)
    with SafetensorsFile(os.path.join(path, "model.safetensors")) as sf:
        weights = {n: sf.tensor(n).to(dtype) for n in sf.names()}
    return raw, weights
