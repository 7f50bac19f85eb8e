"""Gibavik, slowly and plainly: one function per mechanism, loops over tokens and keys, double precision on the
CPU. It shares no code with the package; the engine is compared with it.

Notation. x: the residual stream, read by both sublayers as it is; a sublayer's result y enters as
x <- x + y / sqrt(mean y^2 + eps) * g with one number g. Weights are [out, in]. A model is (raw config dict,
name -> tensor).

  rms(x)               x / sqrt(mean x^2 + eps)
  biased_attention     q, k RMS-normed over their whole projection; score - r1 ln(1 + r2 (i - j)); causal softmax;
                       a layer may read the keys and values of an earlier layer
  turn_halves          entries (i, i + n/2) of the first n of a head turned by p base^(-2i/n)
  window_attention     per-head q/k norm, rotation, values turned by their own position and the result turned back by
                       the query's, capped scores, a sliding window, a sigmoid gate before the output projection
  decay_memory         S <- d_h S + k v^T, o = S^T q with silu on q, k, v; norm over all heads, sigmoid gate
  clamped_ff           min / clamp, g sigmoid(1.702 g) (u + 1)
  table_moe            experts looked up by token id, each weighing 1 / top
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import torch

D = torch.float64


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def silu(z):
    return z * torch.sigmoid(z)


def add_normed(x, y, g, eps):
    """x + rms(y) * g, g one number."""
    return x + rms(y, eps) * g


# ------------------------------------------------------------------ attention with a distance bias
def biased_attention(h, w, p, cfg, eps, shared=None, keep=None):
    """h [T, width] -> [T, width]. ``shared`` = (k, v) of the layer whose keys this layer reads; ``keep``: a list
    that receives this layer's own (k, v)."""
    H, G, dk, dv = cfg["heads"], cfg["kv_heads"], cfg["dim"], cfg["vdim"]
    T = h.shape[0]
    q = rms(h @ w[p + "q"].T + w[p + "q.b"], eps) * w[p + "q.norm"]          # over all H dk entries at once
    if shared is None:
        k = rms(h @ w[p + "k"].T + w[p + "k.b"], eps) * w[p + "k.norm"]
        v = h @ w[p + "v"].T + w[p + "v.b"]
        k, v = k.view(T, G, dk), v.view(T, G, dv)
    else:
        k, v = shared
    if keep is not None:
        keep.append((k, v))
    q = q.view(T, H, dk)
    window = int((cfg.get("mask") or {}).get("size", 0))
    out = torch.zeros(T, H, dv, dtype=D)
    for a in range(H):
        g = a // (H // G)
        r1, r2 = float(w[p + "r1"][a]), float(w[p + "r2"][a])
        for i in range(T):
            lo = max(0, i - window + 1) if window else 0
            dist = (i - torch.arange(lo, i + 1)).to(D)
            s = (k[lo:i + 1, g] @ q[i, a]) * cfg.get("scale", dk ** -0.5) - r1 * torch.log(1.0 + r2 * dist)
            pr = torch.softmax(s, dim=0)
            out[i, a] = (pr[:, None] * v[lo:i + 1, g]).sum(0)
    return out.reshape(T, H * dv) @ w[p + "o"].T


# ------------------------------------------------------------------ windowed attention with turned values
def turn_halves(x: torch.Tensor, pos: torch.Tensor, n: int, base: float, sign: float = 1.0) -> torch.Tensor:
    """x [T, heads, d]; entry i < n/2 and entry i + n/2 are a pair (u, v) -> (u cos a - v sin a, v cos a + u sin a),
    a = sign * pos * base^(-2i/n); entries from n on pass."""
    if n == 0:
        return x
    out = x.clone()
    half = n // 2
    i = torch.arange(half, dtype=D)
    ang = sign * pos.to(D)[:, None] * base ** (-2.0 * i / n)[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u, v = x[..., :half], x[..., half:n]
    out[..., :half] = u * c - v * s
    out[..., half:n] = v * c + u * s
    return out


def window_attention(h, w, p, cfg, eps):
    H, G, dk, dv = cfg["heads"], cfg["kv_heads"], cfg["dim"], cfg["vdim"]
    T = h.shape[0]
    pos = torch.arange(T)
    rot = cfg.get("rot")
    q = (h @ w[p + "q"].T + w[p + "q.b"]).view(T, H, dk)
    k = (h @ w[p + "k"].T + w[p + "k.b"]).view(T, G, dk)
    v = (h @ w[p + "v"].T + w[p + "v.b"]).view(T, G, dv)
    q = rms(q, eps) * w[p + "q.norm"]                       # per head, one weight for all heads
    k = rms(k, eps) * w[p + "k.norm"]
    if rot:
        q = turn_halves(q, pos, rot["dims"], rot["base"])
        k = turn_halves(k, pos, rot["dims"], rot["base"])
        v = turn_halves(v, pos, dv, rot["base"])            # a value is turned by its own position, over all of vdim
    cap = cfg.get("softcap")
    window = int((cfg.get("mask") or {}).get("size", 0))
    out = torch.zeros(T, H, dv, dtype=D)
    for a in range(H):
        g = a // (H // G)
        for i in range(T):
            lo = max(0, i - window + 1) if window else 0
            s = (k[lo:i + 1, g] @ q[i, a]) * cfg.get("scale", dk ** -0.5)
            if cap:
                s = cap * torch.tanh(s / cap)
            out[i, a] = (torch.softmax(s, dim=0)[:, None] * v[lo:i + 1, g]).sum(0)
    if rot:
        out = turn_halves(out, pos, dv, rot["base"], sign=-1.0)      # back by the query's position
    out = out.reshape(T, H * dv) * torch.sigmoid(h @ w[p + "g"].T)
    return out @ w[p + "o"].T


# ------------------------------------------------------------------ the decaying matrix memory
def decay_memory(h, w, p, cfg, eps):
    H, dk, dv = cfg["heads"], cfg["dim"], cfg["vdim"]
    T = h.shape[0]
    q = silu(h @ w[p + "q"].T).view(T, H, dk)
    k = silu(h @ w[p + "k"].T).view(T, H, dk)
    v = silu(h @ w[p + "v"].T).view(T, H, dv)
    out = torch.zeros(T, H, dv, dtype=D)
    for a in range(H):
        S = torch.zeros(dk, dv, dtype=D)
        d = float(cfg["decay"][a])
        for t in range(T):
            S = d * S + torch.outer(k[t, a], v[t, a])
            out[t, a] = S.T @ q[t, a]
    o = rms(out.reshape(T, H * dv), eps) * w[p + "norm"]    # all heads together
    o = o * torch.sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


def parallel_mixers(h, w, p, cfg, eps):
    return cfg.get("left_scale", 1.0) * window_attention(h, w, p + "left.", cfg["left"], eps) \
        + cfg.get("right_scale", 1.0) * decay_memory(h, w, p + "right.", cfg["right"], eps)


# ------------------------------------------------------------------ feed-forwards
def clamped_ff(h, w, p, limit: float):
    g = torch.clamp(h @ w[p + "gate"].T, max=limit)
    u = torch.clamp(h @ w[p + "up"].T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[p + "down"].T


def table_moe(h, w, p, cfg, tokens: Sequence[int]):
    top = cfg["router"]["top"]
    table = w[p + "table"]
    y = torch.zeros(h.shape[0], w[p + "e0.down"].shape[0], dtype=D)
    for t, tok in enumerate(tokens):
        for j in range(top):
            e = int(table[tok, j])
            a = silu(h[t] @ w[f"{p}e{e}.gate"].T) * (h[t] @ w[f"{p}e{e}.up"].T)
            y[t] += (a @ w[f"{p}e{e}.down"].T) / top
    return y


# ------------------------------------------------------------------ the model
def forward(raw: dict, w: Dict[str, torch.Tensor], tokens: Sequence[int], layers_out: Optional[list] = None):
    """Logits [T, vocab] of one sequence from its start; ``layers_out`` collects the stream behind every layer."""
    w = {k: (v.to(D) if v.is_floating_point() else v) for k, v in w.items()}
    eps = float(raw["norm"]["eps"])
    x = w["embed"][torch.tensor(list(tokens))] * float((raw.get("embedding") or {}).get("scale", 1.0))
    kept: Dict[int, tuple] = {}
    for i, L in enumerate(raw["layers"]):
        p = f"l{i}."
        m = L["mixer"]
        if L["type"] == "attention":
            mine: list = []
            src = m.get("kv_from")
            y = biased_attention(x, w, p + "mix.", m, eps, shared=kept[src] if src is not None else None, keep=mine)
            kept[i] = mine[0]
        elif L["type"] == "parallel":
            y = parallel_mixers(x, w, p + "mix.", m, eps)
        else:
            raise ValueError(L["type"])
        x = add_normed(x, y, w[p + "norm1"], eps)
        f = L.get("mlp")
        if f is not None:
            if f["kind"] == "dense":
                y = clamped_ff(x, w, p + "mlp.", float(f["limit"]))
            else:
                y = table_moe(x, w, p + "mlp.", f, tokens)
            x = add_normed(x, y, w[p + "norm2"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    logits = (rms(x, eps) * w["final.norm"]) @ w["head"].T
    cap = raw.get("logit_softcap")
    if cap:
        logits = cap * torch.tanh(logits / cap)
    return logits


def greedy_generate(raw, w, prompt: Sequence[int], n: int) -> List[int]:
    toks, out = list(prompt), []
    for _ in range(n):
        row = forward(raw, w, toks)[-1]
        t = int(torch.nonzero(row == row.max())[0])
        out.append(t)
        toks.append(t)
    return out
