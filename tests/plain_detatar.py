"""Detatar, slowly and plainly: one function per mechanism, a loop over tokens wherever the design has a
recurrence, double precision on the CPU. It shares no code with the package; the engine is compared with it.

Notation. x: the residual stream; h: a layer's normed row; hs: h after the layer's token shift (what the mixer
reads). Weights are [out, in]. A model is (raw config dict, name -> tensor).

  group_norm        the row in equal consecutive parts, each over its own root mean square, then times w
  token_shift       hs_t = h_t + (h_{t-1} - h_t) * s, zeros before the first token
  wkv               per head o_t = (S + diag(u) k v^T)^T r; S <- diag(w_t) S + k v^T, decays from the input
  rotate_half       entry i paired with i + dims/2, turned by p * base^(-2i/dims)
  latent_attention  queries through a normed latent, keys and values from a normed latent, one shared rotated
                    key part, causal softmax, a sigmoid gate a head
  dense_ff          down(gelu_tanh(gate h) * up h)
  moe_ff            softmax router over experts and identity experts, choice by score + correction inside the
                    best groups, weights renormalised, a shared expert behind a sigmoid
  layer             x + sigmoid(rg1 h + b1) * mixer(hs) + sigmoid(rg2 h + b2) * ff(h)
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence

import torch

D = torch.float64


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def group_norm(x: torch.Tensor, w: torch.Tensor, groups: int, eps: float) -> torch.Tensor:
    T, n = x.shape
    return rms(x.view(T, groups, n // groups), eps).reshape(T, n) * w


def silu(z):
    return z * torch.sigmoid(z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def previous_rows(h: torch.Tensor) -> torch.Tensor:
    """Row t holds h[t - 1]; zeros for the first token."""
    return torch.cat([torch.zeros_like(h[:1]), h[:-1]], dim=0)


def token_shift(h: torch.Tensor, s: torch.Tensor) -> torch.Tensor:
    return h + (previous_rows(h) - h) * s


# ------------------------------------------------------------------ wkv
def wkv(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, cfg: dict, eps: float) -> torch.Tensor:
    """h [T, width] (the mixer's input) -> [T, width]. State per head: S [dim, dim], zero at the start."""
    H, d = cfg["heads"], cfg["dim"]
    T = h.shape[0]
    prev = previous_rows(h)

    def mix(name):
        return h + (prev - h) * w[p + "mu." + name]

    r = (mix("r") @ w[p + "r"].T).view(T, H, d)
    k = (mix("k") @ w[p + "k"].T).view(T, H, d)
    v = (mix("v") @ w[p + "v"].T).view(T, H, d)
    gate = silu(mix("g") @ w[p + "g"].T)
    decay = torch.exp(-torch.exp(torch.tanh(mix("w") @ w[p + "w1"].T) @ w[p + "w2"].T + w[p + "w0"])).view(T, H, d)
    u = w[p + "u"].view(H, d)
    out = torch.zeros(T, H, d, dtype=D)
    for a in range(H):
        S = torch.zeros(d, d, dtype=D)
        for t in range(T):
            kv = torch.outer(k[t, a], v[t, a])
            out[t, a] = (S + u[a][:, None] * kv).T @ r[t, a]
            S = decay[t, a][:, None] * S + kv
    o = rms(out, eps).reshape(T, H * d) * w[p + "norm"] * gate
    return o @ w[p + "o"].T


# ------------------------------------------------------------------ latent attention
def rotate_half(x: torch.Tensor, pos: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """x [T, ..., n]: the first ``dims`` entries, i paired with i + dims/2, turned by pos * base^(-2i/dims)."""
    if dims == 0:
        return x
    half = dims // 2
    i = torch.arange(half, dtype=D)
    ang = pos.to(D)[:, None] * base ** (-2.0 * i / dims)[None, :]
    c, s = torch.cos(ang), torch.sin(ang)
    while c.dim() < x.dim():
        c, s = c.unsqueeze(1), s.unsqueeze(1)
    out = x.clone()
    a, b = x[..., :half], x[..., half:dims]
    out[..., :half] = a * c - b * s
    out[..., half:dims] = b * c + a * s
    return out


def latent_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, cfg: dict, eps: float) -> torch.Tensor:
    H, d, R, dv, rank = cfg["heads"], cfg["dim"], cfg["rot_dim"], cfg["vdim"], cfg["kv_rank"]
    rot = cfg.get("rot") or {"dims": 0, "base": 1.0}
    T = h.shape[0]
    pos = torch.arange(T)
    cq = rms(h @ w[p + "dq"].T, eps) * w[p + "dq.norm"]
    q = (cq @ w[p + "uq"].T).view(T, H, d + R)
    q_plain, q_rot = q[..., :d], rotate_half(q[..., d:], pos, rot["dims"], rot["base"])
    down = h @ w[p + "dkv"].T
    c = rms(down[:, :rank], eps) * w[p + "dkv.norm"]
    k_rot = rotate_half(down[:, rank:], pos, rot["dims"], rot["base"])          # [T, R], one for all heads
    k_plain = (c @ w[p + "uk"].T).view(T, H, d)
    v = (c @ w[p + "uv"].T).view(T, H, dv)
    gate = torch.sigmoid(h @ w[p + "g"].T)                                      # [T, H]
    out = torch.zeros(T, H, dv, dtype=D)
    hidden = torch.triu(torch.ones(T, T, dtype=torch.bool), 1)
    for a in range(H):
        s = (q_plain[:, a] @ k_plain[:, a].T + q_rot[:, a] @ k_rot.T) * cfg["scale"]
        s = s.masked_fill(hidden, float("-inf"))
        out[:, a] = (torch.softmax(s, dim=-1) @ v[:, a]) * gate[:, a:a + 1]
    return out.reshape(T, H * dv) @ w[p + "o"].T


# ------------------------------------------------------------------ feed-forwards
def gated_ff(h, w, p, act) -> torch.Tensor:
    return (act(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def dense_ff(h, w, p) -> torch.Tensor:
    return gated_ff(h, w, p, gelu_tanh)


def route(choice: torch.Tensor, top: int, groups: int, keep: int) -> List[List[int]]:
    """The chosen experts of every row of ``choice`` [T, E]: the ``top`` largest among the experts of the
    ``keep`` groups (of ``groups`` equal runs of neighbours) whose largest entry is highest."""
    T, E = choice.shape
    size = E // groups
    out = []
    for t in range(T):
        s = choice[t].tolist()
        best = sorted(range(groups), key=lambda g: (-max(s[g * size:(g + 1) * size]), g))[:keep]
        allowed = [e for e in range(E) if e // size in best]
        out.append(sorted(allowed, key=lambda e: (-s[e], e))[:top])
    return out


def moe_ff(h, w, p, cfg) -> torch.Tensor:
    r = cfg["router"]
    E, ident = r["experts"], r.get("identity", 0)
    groups = r.get("groups") or {"count": 1, "keep": 1}
    s = torch.softmax(h @ w[p + "router"].T, dim=-1)                             # [T, E + ident]
    chosen = route(s + w[p + "correction"], r["top"], groups["count"], groups["keep"])
    y = torch.zeros_like(h)
    for t, es in enumerate(chosen):
        total = sum(float(s[t, e]) for e in es) + 1e-20
        for e in es:
            weight = float(s[t, e]) / total
            y[t] += weight * (gated_ff(h[t:t + 1], w, f"{p}e{e}.", silu)[0] if e < E else h[t])
    if cfg.get("shared") is not None:
        y = y + torch.sigmoid(h @ w[p + "shared.sg"].T) * gated_ff(h, w, p + "shared.", silu)
    return y


# ------------------------------------------------------------------ the model
def layer(x, w, p: str, L: dict, groups: int, eps: float) -> torch.Tensor:
    """One run of a layer whose tensors start with ``p`` over a whole sequence from its start."""
    h = group_norm(x, w[p + "norm1"], groups, eps)
    hs = token_shift(h, w[p + "shift"])
    if L["type"] == "wkv":
        y = wkv(hs, w, p + "mix.", L["mixer"], eps)
    elif L["type"] == "latent_attention":
        y = latent_attention(hs, w, p + "mix.", L["mixer"], eps)
    else:
        raise ValueError(L["type"])
    x = x + torch.sigmoid(h @ w[p + "rg1"].T + w[p + "rg1.b"]) * y
    if L.get("mlp") is not None:
        f = dense_ff(h, w, p + "mlp.") if L["mlp"]["kind"] == "dense" else moe_ff(h, w, p + "mlp.", L["mlp"])
        x = x + torch.sigmoid(h @ w[p + "rg2"].T + w[p + "rg2.b"]) * f
    return x


def forward(raw: dict, w: Dict[str, torch.Tensor], tokens: Sequence[int], layers_out: Optional[list] = None):
    """Logits [T, vocab] of one sequence from its start; ``layers_out`` collects the stream behind every layer."""
    w = {k: v.to(D) for k, v in w.items()}
    eps = float(raw["norm"]["eps"])
    groups = int(raw["norm"].get("groups", 1))
    x = w["embed"][torch.tensor(list(tokens))] * float((raw.get("embedding") or {}).get("scale", 1.0))
    for i, L in enumerate(raw["layers"]):
        x = layer(x, w, f"l{L.get('weights_of', i)}.", L, groups, eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return group_norm(x, w["final.norm"], groups, eps) @ w["head"].T


def greedy_generate(raw, w, prompt: Sequence[int], n: int) -> List[int]:
    toks, out = list(prompt), []
    for _ in range(n):
        row = forward(raw, w, toks)[-1]
        t = int(torch.nonzero(row == row.max())[0])
        out.append(t)
        toks.append(t)
    return out
