"""The plain Gibavik implementation pinned by numbers worked out by hand and by closed forms of one and two tokens,
each chosen so that a plausible misreading of a mechanism fails it."""
import math

import torch

import plain_gibavik as plain

D = torch.float64


def t(*v):
    return torch.tensor(v, dtype=D)


def test_rms_has_eps_inside_the_root_and_the_norm_takes_one_number():
    x = t(3.0, 4.0)
    assert torch.allclose(plain.rms(x, 0.5), x / math.sqrt(12.5 + 0.5))
    y = plain.add_normed(t(1.0, 1.0), t(3.0, 4.0), torch.tensor(2.0, dtype=D), 0.5)
    assert torch.allclose(y, t(1.0, 1.0) + 2.0 * x / math.sqrt(13.0))


def test_turn_halves_pairs_entries_half_a_width_apart():
    x = t(1.0, 2.0, 3.0, 4.0, 5.0).view(1, 1, 5)
    pos = torch.tensor([3])
    y = plain.turn_halves(x, pos, 4, 100.0)[0, 0]
    a0, a1 = 3.0, 3.0 * 100.0 ** -0.5                     # pair 0: entries 0 and 2; pair 1: entries 1 and 3
    want = t(1 * math.cos(a0) - 3 * math.sin(a0), 2 * math.cos(a1) - 4 * math.sin(a1),
             3 * math.cos(a0) + 1 * math.sin(a0), 4 * math.cos(a1) + 2 * math.sin(a1), 5.0)
    assert torch.allclose(y, want)
    back = plain.turn_halves(y.view(1, 1, 5), pos, 4, 100.0, sign=-1.0)[0, 0]
    assert torch.allclose(back, x[0, 0])


def _biased_model(H, G, dk, dv, width):
    g = torch.Generator().manual_seed(1)
    r = lambda *s: torch.randn(*s, generator=g, dtype=D)
    return {"m.q": r(H * dk, width), "m.q.b": r(H * dk), "m.k": r(G * dk, width), "m.k.b": r(G * dk),
            "m.v": r(G * dv, width), "m.v.b": r(G * dv), "m.q.norm": r(H * dk), "m.k.norm": r(G * dk),
            "m.r1": torch.rand(H, generator=g, dtype=D) + 0.5, "m.r2": torch.rand(H, generator=g, dtype=D) + 0.1,
            "m.o": r(width, H * dv)}


def test_biased_attention_two_tokens_by_hand():
    H, G, dk, dv, width, eps, scale = 2, 1, 3, 2, 4, 1e-5, 0.7
    w = _biased_model(H, G, dk, dv, width)
    h = torch.randn(2, width, generator=torch.Generator().manual_seed(2), dtype=D)
    cfg = {"heads": H, "kv_heads": G, "dim": dk, "vdim": dv, "scale": scale}
    got = plain.biased_attention(h, w, "m.", cfg, eps)
    q = h @ w["m.q"].T + w["m.q.b"]
    q = q / torch.sqrt((q * q).mean(-1, keepdim=True) + eps) * w["m.q.norm"]          # over all six entries at once
    k = h @ w["m.k"].T + w["m.k.b"]
    k = k / torch.sqrt((k * k).mean(-1, keepdim=True) + eps) * w["m.k.norm"]
    v = h @ w["m.v"].T + w["m.v.b"]
    heads = []
    for a in range(H):
        qa = q[1, a * dk:(a + 1) * dk]
        s0 = float(qa @ k[0]) * scale - float(w["m.r1"][a]) * math.log(1.0 + float(w["m.r2"][a]) * 1.0)
        s1 = float(qa @ k[1]) * scale                                                   # distance 0: nothing taken off
        p0 = 1.0 / (1.0 + math.exp(s1 - s0))
        heads.append(p0 * v[0] + (1.0 - p0) * v[1])
    want = torch.cat(heads) @ w["m.o"].T
    assert torch.allclose(got[1], want, atol=1e-12)
    # the first token sees itself alone: its value, whatever the scores
    first = torch.cat([v[0], v[0]]) @ w["m.o"].T
    assert torch.allclose(got[0], first, atol=1e-12)


def test_a_layer_that_reads_another_layers_keys_uses_them_as_they_were_normed():
    H, G, dk, dv, width, eps = 2, 1, 3, 2, 4, 1e-5
    w = _biased_model(H, G, dk, dv, width)
    h = torch.randn(5, width, generator=torch.Generator().manual_seed(3), dtype=D)
    h2 = torch.randn(5, width, generator=torch.Generator().manual_seed(4), dtype=D)
    cfg = {"heads": H, "kv_heads": G, "dim": dk, "vdim": dv, "scale": 0.5}
    kept = []
    plain.biased_attention(h, w, "m.", cfg, eps, keep=kept)
    # a reader with the same query tensors on another input: the keys and values of the first call, not of its input
    reader = {n: v for n, v in w.items() if not n.startswith(("m.k", "m.v"))}
    got = plain.biased_attention(h2, reader, "m.", cfg, eps, shared=kept[0])
    w2 = dict(w)
    own = plain.biased_attention(h2, w2, "m.", cfg, eps)
    assert not torch.allclose(got, own)
    k, v = kept[0]
    q = plain.rms(h2 @ w["m.q"].T + w["m.q.b"], eps) * w["m.q.norm"]
    a = 1
    s = torch.stack([(q[4, a * dk:(a + 1) * dk] @ k[j, 0]) * 0.5 - w["m.r1"][a] * torch.log(1 + w["m.r2"][a] * (4 - j))
                     for j in range(5)])
    o = (torch.softmax(s, 0)[:, None] * v[:, 0]).sum(0)
    full = got[4]
    a0 = 0
    s0 = torch.stack([(q[4, :dk] @ k[j, 0]) * 0.5 - w["m.r1"][a0] * torch.log(1 + w["m.r2"][a0] * (4 - j)) for j in range(5)])
    o0 = (torch.softmax(s0, 0)[:, None] * v[:, 0]).sum(0)
    assert torch.allclose(full, torch.cat([o0, o]) @ w["m.o"].T, atol=1e-12)


def _window_model(H, G, dk, dv, width, seed=5):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g, dtype=D)
    return {"m.q": r(H * dk, width), "m.q.b": r(H * dk), "m.k": r(G * dk, width), "m.k.b": r(G * dk),
            "m.v": r(G * dv, width), "m.v.b": r(G * dv), "m.q.norm": r(dk), "m.k.norm": r(dk),
            "m.g": r(H * dv, width), "m.o": r(width, H * dv)}


def test_window_of_one_gives_the_tokens_own_value_unturned_times_the_gate():
    H, G, dk, dv, width, eps = 2, 2, 4, 4, 6, 1e-5
    w = _window_model(H, G, dk, dv, width)
    h = torch.randn(7, width, generator=torch.Generator().manual_seed(6), dtype=D)
    cfg = {"heads": H, "kv_heads": G, "dim": dk, "vdim": dv, "scale": 0.5, "softcap": 3.0, "mask": {"size": 1},
           "rot": {"base": 50.0, "dims": 2}}
    got = plain.window_attention(h, w, "m.", cfg, eps)
    v = h @ w["m.v"].T + w["m.v.b"]                        # turned by j and back by i = j
    want = (v * torch.sigmoid(h @ w["m.g"].T)) @ w["m.o"].T
    assert torch.allclose(got, want, atol=1e-12)


def test_values_turn_with_their_own_position_and_back_with_the_querys():
    """Zero queries give equal weights; with two tokens the second result is half of (the first value turned back by
    one position) plus half of its own value."""
    H, G, dk, dv, width, eps = 1, 1, 4, 4, 5, 1e-5
    w = _window_model(H, G, dk, dv, width, seed=7)
    w["m.q"].zero_()
    w["m.q.b"].zero_()
    w["m.g"].zero_()                                       # the gate is one half
    w["m.o"] = torch.eye(4, dtype=D)[:, :4].contiguous()
    w["m.o"] = torch.cat([torch.eye(4, dtype=D), torch.zeros(1, 4, dtype=D)], 0)      # [width 5, 4]: the heads come out as they are
    h = torch.randn(2, width, generator=torch.Generator().manual_seed(8), dtype=D)
    cfg = {"heads": H, "kv_heads": G, "dim": dk, "vdim": dv, "scale": 1.0, "softcap": 50.0, "mask": {"size": 8},
           "rot": {"base": 9.0, "dims": 2}}
    got = plain.window_attention(h, w, "m.", cfg, eps)[1, :4]
    v = h @ w["m.v"].T + w["m.v.b"]
    f = [1.0, 9.0 ** -0.5]                                  # pair m of the value: base^(-2m/4), whatever dims is
    v0 = v[0].clone()
    for m in range(2):
        c, s = math.cos(-f[m]), math.sin(-f[m])
        v0[m], v0[m + 2] = v[0, m] * c - v[0, m + 2] * s, v[0, m + 2] * c + v[0, m] * s
    assert torch.allclose(got, 0.5 * (0.5 * v0 + 0.5 * v[1]), atol=1e-12)


def test_scores_are_capped_before_the_softmax_and_the_window_counts_the_token_itself():
    H, G, dk, dv, width, eps = 1, 1, 2, 2, 3, 1e-5
    w = _window_model(H, G, dk, dv, width, seed=9)
    w["m.g"].zero_()
    w["m.o"] = torch.cat([torch.eye(2, dtype=D), torch.zeros(1, 2, dtype=D)], 0)
    h = torch.randn(4, width, generator=torch.Generator().manual_seed(10), dtype=D) * 3
    cfg = {"heads": H, "kv_heads": G, "dim": dk, "vdim": dv, "scale": 2.0, "softcap": 1.5, "mask": {"size": 2}}
    got = plain.window_attention(h, w, "m.", cfg, eps)[3, :2]
    q = plain.rms(h @ w["m.q"].T + w["m.q.b"], eps) * w["m.q.norm"]
    k = plain.rms(h @ w["m.k"].T + w["m.k.b"], eps) * w["m.k.norm"]
    v = h @ w["m.v"].T + w["m.v.b"]
    s = [1.5 * math.tanh(float(q[3] @ k[j]) * 2.0 / 1.5) for j in (2, 3)]          # a window of 2: itself and one before
    p2 = 1.0 / (1.0 + math.exp(s[1] - s[0]))
    assert torch.allclose(got, 0.5 * (p2 * v[2] + (1 - p2) * v[3]), atol=1e-12)


def test_decay_memory_first_two_tokens_in_closed_form():
    H, dk, dv, width, eps = 2, 3, 2, 4, 1e-5
    g = torch.Generator().manual_seed(11)
    r = lambda *s: torch.randn(*s, generator=g, dtype=D)
    w = {"m.q": r(H * dk, width), "m.k": r(H * dk, width), "m.v": r(H * dv, width), "m.g": r(H * dv, width),
         "m.o": r(width, H * dv), "m.norm": r(H * dv)}
    h = r(2, width)
    cfg = {"heads": H, "dim": dk, "vdim": dv, "decay": [0.5, 0.9]}
    got = plain.decay_memory(h, w, "m.", cfg, eps)
    silu = lambda z: z / (1 + torch.exp(-z))
    q, k, v = silu(h @ w["m.q"].T), silu(h @ w["m.k"].T), silu(h @ w["m.v"].T)
    o = []
    for a, d in enumerate(cfg["decay"]):
        qa, ka, va = q[:, a * dk:(a + 1) * dk], k[:, a * dk:(a + 1) * dk], v[:, a * dv:(a + 1) * dv]
        # o_1 = (q_1 . k_1) v_1 + d (q_1 . k_0) v_0: the read-out sees the token's own write, and no other scale
        o.append((qa[1] @ ka[1]) * va[1] + d * (qa[1] @ ka[0]) * va[0])
    o = torch.cat(o)
    o = o / torch.sqrt((o * o).mean() + eps) * w["m.norm"]                          # all heads together
    want = (o * torch.sigmoid(h[1] @ w["m.g"].T)) @ w["m.o"].T
    assert torch.allclose(got[1], want, atol=1e-12)


def test_clamped_feed_forward_by_hand():
    w = {"f.gate": t(2.0, -3.0).view(2, 1), "f.up": t(5.0, -0.25).view(2, 1), "f.down": t(1.0, 10.0).view(1, 2)}
    y = plain.clamped_ff(t(1.0).view(1, 1), w, "f.", 1.5)
    g0, u0 = 1.5, 1.5                                       # 2 and 5 are cut from above
    g1, u1 = -3.0, -0.25                                    # the gate has no bound from below
    want = g0 / (1 + math.exp(-1.702 * g0)) * (u0 + 1) + 10 * g1 / (1 + math.exp(-1.702 * g1)) * (u1 + 1)
    assert abs(float(y) - want) < 1e-12
    y2 = plain.clamped_ff(t(-1.0).view(1, 1), w, "f.", 1.5)  # up = -5 is cut to -1.5: u + 1 = -0.5
    want2 = -2.0 / (1 + math.exp(1.702 * 2.0)) * (-0.5) + 10 * 1.5 / (1 + math.exp(-1.702 * 1.5)) * 1.25
    assert abs(float(y2) - want2) < 1e-12


def test_table_experts_weigh_one_over_top_each():
    g = torch.Generator().manual_seed(12)
    r = lambda *s: torch.randn(*s, generator=g, dtype=D)
    w = {"f.table": torch.tensor([[0, 2], [1, 0], [2, 1]], dtype=torch.int32)}
    for e in range(3):
        w.update({f"f.e{e}.gate": r(4, 3), f"f.e{e}.up": r(4, 3), f"f.e{e}.down": r(3, 4)})
    h = r(2, 3)
    y = plain.table_moe(h, w, "f.", {"router": {"experts": 3, "top": 2}}, [2, 0])
    silu = lambda z: z / (1 + torch.exp(-z))
    ex = lambda e, x: (silu(x @ w[f"f.e{e}.gate"].T) * (x @ w[f"f.e{e}.up"].T)) @ w[f"f.e{e}.down"].T
    assert torch.allclose(y[0], 0.5 * (ex(2, h[0]) + ex(1, h[0])), atol=1e-12)       # token id 2: experts 2 and 1
    assert torch.allclose(y[1], 0.5 * (ex(0, h[1]) + ex(2, h[1])), atol=1e-12)


def test_the_parts_read_the_stream_itself_and_the_head_is_capped():
    """One attention layer without a feed-forward, one token: x1 = x0 + g rms(W_o (W_v x0 + b_v)); logits =
    cap tanh(head (g_f rms(x1)) / cap)."""
    from gibavik_helpers import draw_weights
    raw = {"architecture": "Gibavik", "vocab": 20, "width": 8, "norm": {"eps": 1e-5}, "embedding": {"scale": 3.0},
           "logit_softcap": 2.0,
           "layers": [{"type": "attention", "mlp": None, "mixer": {"dim": 4, "heads": 2, "kv_heads": 1, "vdim": 6,
                                                                   "scale": 0.5}}]}
    w = {n: v.double() for n, v in draw_weights(raw, 1).items()}
    got = plain.forward(raw, w, [7])[0]
    x0 = w["embed"][7] * 3.0
    v = w["l0.mix.v"] @ x0 + w["l0.mix.v.b"]
    y = w["l0.mix.o"] @ torch.cat([v, v])
    x1 = x0 + w["l0.norm1"] * y / torch.sqrt((y * y).mean() + 1e-5)
    z = w["head"] @ (w["final.norm"] * x1 / torch.sqrt((x1 * x1).mean() + 1e-5))
    assert torch.allclose(got, 2.0 * torch.tanh(z / 2.0), atol=1e-12)
