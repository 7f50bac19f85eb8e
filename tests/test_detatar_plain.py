"""The plain implementation of Detatar, pinned mechanism by mechanism: by numbers worked out by hand, by closed
forms of one or two tokens written out here from the equations, and by cases that reduce to something simpler.
Each is chosen so that a plausible misreading fails it (one norm over the whole row, the shift applied to what the
feed-forward reads, the bonus kept in the state, the decay applied before the read-out, pairs (2i, 2i + 1), a
rotated key a head, the correction in the weights, a group scored by a sum, masked groups counted as zero, identity
experts outside the softmax)."""
import math

import torch

import plain_detatar as plain

D = torch.float64


def rnd(*shape, seed=0, std=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=D) * std


def test_norm_in_groups():
    x = torch.tensor([[3.0, 4.0, 0.5, 0.5]], dtype=D)
    w = torch.tensor([1.0, 2.0, 1.0, 3.0], dtype=D)
    out = plain.group_norm(x, w, 2, 0.0)
    r0, r1 = math.sqrt(12.5), 0.5
    assert torch.allclose(out, torch.tensor([[3 / r0, 8 / r0, 0.5 / r1, 1.5 / r1]], dtype=D))
    # one group: the whole row; eps inside the root
    one = plain.group_norm(x, w, 1, 0.25)
    r = math.sqrt((9 + 16 + 0.25 + 0.25) / 4 + 0.25)
    assert torch.allclose(one, x / r * w)
    assert not torch.allclose(one, out)


def test_token_shift_reads_the_row_before():
    h = torch.tensor([[1.0, 10.0], [2.0, 20.0], [4.0, 40.0]], dtype=D)
    s = torch.tensor([0.25, 1.0], dtype=D)
    out = plain.token_shift(h, s)
    # first token: zeros before it; factor 1 hands the row before on as it was (not its shifted form)
    assert torch.allclose(out, torch.tensor([[0.75, 0.0], [1.75, 10.0], [3.5, 20.0]], dtype=D))


def _wkv_weights(H, d, width, rank, seed):
    n = H * d
    w = {"mu." + s: torch.rand(width, generator=torch.Generator().manual_seed(seed + i), dtype=D)
         for i, s in enumerate("rkvgw")}
    w.update({"r": rnd(n, width, seed=seed + 10), "k": rnd(n, width, seed=seed + 11), "v": rnd(n, width, seed=seed + 12),
              "g": rnd(n, width, seed=seed + 13), "w1": rnd(rank, width, seed=seed + 14), "w2": rnd(n, rank, seed=seed + 15),
              "w0": rnd(n, seed=seed + 16) - 1.0, "u": rnd(H, d, seed=seed + 17), "norm": torch.ones(n, dtype=D),
              "o": torch.eye(n, dtype=D)})
    return w


def test_wkv_first_two_tokens_in_closed_form():
    H, d, width, rank, eps = 2, 3, 6, 2, 1e-5
    w = _wkv_weights(H, d, width, rank, 40)
    h = rnd(2, width, seed=41)
    got = plain.wkv(h, w, "", {"heads": H, "dim": d}, eps).view(2, H, d)
    prev = [torch.zeros(width, dtype=D), h[0]]
    mix = lambda t, s: h[t] + (prev[t] - h[t]) * w["mu." + s]
    for a in range(H):
        rows = slice(a * d, (a + 1) * d)
        r = [w["r"][rows] @ mix(t, "r") for t in range(2)]
        k = [w["k"][rows] @ mix(t, "k") for t in range(2)]
        v = [w["v"][rows] @ mix(t, "v") for t in range(2)]
        gate = [plain.silu(w["g"][rows] @ mix(t, "g")) for t in range(2)]
        dec0 = torch.exp(-torch.exp(w["w2"][rows] @ torch.tanh(w["w1"] @ mix(0, "w")) + w["w0"][rows]))
        u = w["u"][a]
        # token 0: an empty state, the bonus alone: o = v (u * k . r)
        o0 = v[0] * float((u * k[0]) @ r[0])
        # token 1: the state holds k0 v0^T once, without bonus and without a decay (the decay of token 0 is applied
        # after its write, and token 1's own only after token 1's read-out)
        o1 = v[0] * float(k[0] @ r[1]) + v[1] * float((u * k[1]) @ r[1])
        for t, o in ((0, o0), (1, o1)):
            want = o / torch.sqrt((o * o).mean() + eps) * gate[t]
            assert torch.allclose(got[t, a], want), (a, t)
        assert float(dec0.min()) > 0 and float(dec0.max()) < 1
    # a third token sees token 0 through token 1's decay, channel by channel
    h3 = rnd(3, width, seed=42)
    w["norm"] = torch.ones(H * d, dtype=D)
    got3 = plain.wkv(h3, w, "", {"heads": H, "dim": d}, 0.0).view(3, H, d)
    prev = [torch.zeros(width, dtype=D), h3[0], h3[1]]
    mix = lambda t, s: h3[t] + (prev[t] - h3[t]) * w["mu." + s]
    a, rows = 1, slice(d, 2 * d)
    r2 = w["r"][rows] @ mix(2, "r")
    k = [w["k"][rows] @ mix(t, "k") for t in range(3)]
    v = [w["v"][rows] @ mix(t, "v") for t in range(3)]
    dec1 = torch.exp(-torch.exp(w["w2"][rows] @ torch.tanh(w["w1"] @ mix(1, "w")) + w["w0"][rows]))
    o2 = v[0] * float((dec1 * k[0]) @ r2) + v[1] * float(k[1] @ r2) + v[2] * float((w["u"][a] * k[2]) @ r2)
    gate2 = plain.silu(w["g"][rows] @ mix(2, "g"))
    assert torch.allclose(got3[2, a], o2 / torch.sqrt((o2 * o2).mean()) * gate2)


def test_rotate_half_pairs_and_angles():
    x = torch.tensor([[[1.0, 2.0, 3.0, 4.0, 5.0, 6.0]]], dtype=D).repeat(2, 1, 1)       # two positions, one head
    out = plain.rotate_half(x, torch.tensor([0, 3]), 4, 100.0)
    assert torch.equal(out[0], x[0])                                                    # position 0: unchanged
    a0, a1 = 3 * 1.0, 3 * 100.0 ** -0.5                                                 # f_i = base^(-2i/dims)
    # entry i with entry i + 2
    want = [1 * math.cos(a0) - 3 * math.sin(a0), 2 * math.cos(a1) - 4 * math.sin(a1),
            3 * math.cos(a0) + 1 * math.sin(a0), 4 * math.cos(a1) + 2 * math.sin(a1), 5.0, 6.0]
    assert torch.allclose(out[1, 0], torch.tensor(want, dtype=D))


def test_latent_attention_by_hand():
    H, d, R, dv, rank, qr, width, T, eps = 3, 4, 2, 5, 6, 3, 7, 5, 1e-5
    cfg = {"heads": H, "dim": d, "rot_dim": R, "vdim": dv, "kv_rank": rank, "q_rank": qr, "scale": 0.41,
           "rot": {"dims": R, "base": 30.0}}
    w = {"dq": rnd(qr, width, seed=1), "dq.norm": rnd(qr, seed=2), "uq": rnd(H * (d + R), qr, seed=3),
         "dkv": rnd(rank + R, width, seed=4), "dkv.norm": rnd(rank, seed=5), "uk": rnd(H * d, rank, seed=6),
         "uv": rnd(H * dv, rank, seed=7), "g": rnd(H, width, seed=8), "o": torch.eye(H * dv, dtype=D)}
    h = rnd(T, width, seed=9)
    out = plain.latent_attention(h, w, "", cfg, eps).view(T, H, dv)
    down = h @ w["dkv"].T
    c = down[:, :rank] / torch.sqrt((down[:, :rank] ** 2).mean(-1, keepdim=True) + eps) * w["dkv.norm"]
    v = (c @ w["uv"].T).view(T, H, dv)
    gate = torch.sigmoid(h @ w["g"].T)
    # the first token sees itself alone: its value times its head's gate
    for a in range(H):
        assert torch.allclose(out[0, a], v[0, a] * gate[0, a])
    # token 3, head 2, by hand; the rotated key part is not normed and is the same for every head
    cq = h @ w["dq"].T
    cq = cq / torch.sqrt((cq * cq).mean(-1, keepdim=True) + eps) * w["dq.norm"]
    q = (cq @ w["uq"].T).view(T, H, d + R)
    t, a = 3, 2

    def turn(x, p):
        ang = p * 1.0
        return torch.stack([x[0] * math.cos(ang) - x[1] * math.sin(ang), x[1] * math.cos(ang) + x[0] * math.sin(ang)])
    s = []
    for j in range(t + 1):
        kj = w["uk"][a * d:(a + 1) * d] @ c[j]
        s.append((float(q[t, a, :d] @ kj) + float(turn(q[t, a, d:], t) @ turn(down[j, rank:], j))) * 0.41)
    s = torch.tensor(s, dtype=D)
    p = torch.exp(s - s.max()) / torch.exp(s - s.max()).sum()
    assert torch.allclose(out[t, a], (p @ v[:t + 1, a]) * gate[t, a])


def test_dense_feed_forward_uses_the_tanh_form():
    z = torch.tensor([-2.0, -0.3, 0.0, 0.7, 3.0], dtype=D)
    want = [0.5 * x * (1 + math.tanh(math.sqrt(2 / math.pi) * (x + 0.044715 * x ** 3))) for x in z.tolist()]
    assert torch.allclose(plain.gelu_tanh(z), torch.tensor(want, dtype=D))
    assert float((plain.gelu_tanh(z) - torch.nn.functional.gelu(z)).abs().max()) > 1e-5        # not the erf form
    w = {"gate": rnd(5, 3, seed=1), "up": rnd(5, 3, seed=2), "down": rnd(3, 5, seed=3)}
    h = rnd(2, 3, seed=4)
    assert torch.allclose(plain.dense_ff(h, w, ""), (plain.gelu_tanh(h @ w["gate"].T) * (h @ w["up"].T)) @ w["down"].T)


def test_choice_inside_the_best_groups():
    # six outputs in three groups of two; a group is scored by its largest entry, not by a sum:
    # group 0 has the largest sum, groups 1 and 2 the largest entries
    choice = torch.tensor([[0.30, 0.29, 0.05, 0.40, 0.35, 0.01]], dtype=D)
    assert plain.route(choice, 2, 3, 2) == [[3, 4]]
    assert plain.route(choice, 3, 3, 2) == [[3, 4, 2]]
    assert plain.route(choice, 2, 1, 1) == [[3, 4]]
    assert plain.route(choice, 3, 1, 1) == [[3, 4, 0]]
    # negative choice scores: an expert outside the kept group is never chosen, though 0 would beat -0.2
    neg = torch.tensor([[-0.1, -0.2, -0.15, -0.3]], dtype=D)
    assert plain.route(neg, 2, 2, 1) == [[0, 1]]


def test_mixture_weights_correction_and_identity():
    width, E, ident, ff = 4, 3, 2, 5
    cfg = {"expert": {"ff": ff}, "router": {"experts": E, "identity": ident, "top": 2}}
    w = {"router": rnd(E + ident, width, seed=1), "correction": torch.zeros(E + ident, dtype=D)}
    for e in range(E):
        w.update({f"e{e}.gate": rnd(ff, width, seed=10 + e), f"e{e}.up": rnd(ff, width, seed=20 + e),
                  f"e{e}.down": rnd(width, ff, seed=30 + e)})
    h = rnd(1, width, seed=5)
    s = torch.softmax(h @ w["router"].T, dim=-1)[0]                    # over experts and identity experts alike
    order = sorted(range(E + ident), key=lambda e: -float(s[e]))
    # the correction moves the choice to the two lowest scores and stays out of the weights
    w["correction"] = torch.zeros(E + ident, dtype=D)
    w["correction"][order[-1]] = 5.0
    w["correction"][order[-2]] = 4.0
    chosen = order[-2:]
    total = float(s[chosen[0]] + s[chosen[1]]) + 1e-20
    want = torch.zeros(width, dtype=D)
    for e in chosen:
        y = plain.gated_ff(h, w, f"e{e}.", plain.silu)[0] if e < E else h[0]
        want += float(s[e]) / total * y
    assert torch.allclose(plain.moe_ff(h, w, "", cfg)[0], want)
    # both identity experts chosen: the output is h itself (weights sum to one)
    w["correction"] = torch.tensor([0.0, 0.0, 0.0, 9.0, 9.0], dtype=D)
    assert torch.allclose(plain.moe_ff(h, w, "", cfg)[0], h[0])
    # a shared expert is added behind one sigmoid a token
    cfg["shared"] = {"ff": 3}
    w.update({"shared.gate": rnd(3, width, seed=41), "shared.up": rnd(3, width, seed=42),
              "shared.down": rnd(width, 3, seed=43), "shared.sg": rnd(1, width, seed=44)})
    sg = torch.sigmoid(h @ w["shared.sg"].T)
    assert sg.shape == (1, 1)
    assert torch.allclose(plain.moe_ff(h, w, "", cfg)[0], h[0] + float(sg) * plain.gated_ff(h, w, "shared.", plain.silu)[0])


def test_layer_gates_and_what_each_part_reads():
    width, T, eps = 8, 3, 1e-5
    L = {"type": "wkv", "mixer": {"heads": 2, "dim": 3}, "mlp": {"kind": "dense", "ff": 5}}
    w = {"l0.mix." + k: v for k, v in _wkv_weights(2, 3, width, 2, 70).items()}
    w["l0.mix.o"] = rnd(width, 6, seed=71)
    w.update({"l0.norm1": rnd(width, seed=72), "l0.shift": torch.rand(width, dtype=D), "l0.rg1": rnd(width, width, seed=73),
              "l0.rg1.b": rnd(width, seed=74), "l0.rg2": rnd(width, width, seed=75), "l0.rg2.b": rnd(width, seed=76),
              "l0.mlp.gate": rnd(5, width, seed=77), "l0.mlp.up": rnd(5, width, seed=78), "l0.mlp.down": rnd(width, 5, seed=79)})
    x = rnd(T, width, seed=80)
    got = plain.layer(x, w, "l0.", L, 2, eps)
    h = plain.group_norm(x, w["l0.norm1"], 2, eps)
    hs = plain.token_shift(h, w["l0.shift"])
    mixer = plain.wkv(hs, w, "l0.mix.", L["mixer"], eps)            # the mixer reads the shifted row ...
    ff = plain.dense_ff(h, w, "l0.mlp.")                            # ... the feed-forward and both gates the row itself
    want = x + torch.sigmoid(h @ w["l0.rg1"].T + w["l0.rg1.b"]) * mixer + torch.sigmoid(h @ w["l0.rg2"].T + w["l0.rg2.b"]) * ff
    assert torch.allclose(got, want)
    # without a feed-forward only the mixer's addend is there
    L2 = dict(L, mlp=None)
    assert torch.allclose(plain.layer(x, w, "l0.", L2, 2, eps), x + torch.sigmoid(h @ w["l0.rg1"].T + w["l0.rg1.b"]) * mixer)


def test_a_layer_run_again_has_a_state_of_its_own():
    """Two layers on one set of tensors: the second run starts from an empty state and its own row before."""
    raw = {"vocab": 11, "width": 8, "norm": {"eps": 1e-5, "groups": 2}, "embedding": {"scale": 1.5},
           "layers": [{"type": "wkv", "mixer": {"heads": 2, "dim": 3}, "mlp": None},
                      {"type": "wkv", "mixer": {"heads": 2, "dim": 3}, "mlp": None, "weights_of": 0}]}
    w = {"l0.mix." + k: v for k, v in _wkv_weights(2, 3, 8, 2, 90).items()}
    w["l0.mix.o"] = rnd(8, 6, seed=91)
    w.update({"l0.norm1": rnd(8, seed=92), "l0.shift": torch.rand(8, dtype=D), "l0.rg1": rnd(8, 8, seed=93),
              "l0.rg1.b": rnd(8, seed=94), "embed": rnd(11, 8, seed=95), "head": rnd(11, 8, seed=96),
              "final.norm": rnd(8, seed=97)})
    toks = [3, 7, 1, 0]
    x = w["embed"][torch.tensor(toks)] * 1.5
    for _ in range(2):
        x = plain.layer(x, w, "l0.", raw["layers"][0], 2, 1e-5)
    want = plain.group_norm(x, w["final.norm"], 2, 1e-5) @ w["head"].T
    assert torch.allclose(plain.forward(raw, w, toks), want)
