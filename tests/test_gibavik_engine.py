"""Gibavik through the engine against the plain implementation: configuration, whole prompts, prompts against
token-by-token decoding, portions down to two tokens, unequal requests in one batch with blocks and state slots that
are given back and used again, the first tokens, long decoding, keys far back, at block borders and on either side of
a window's edge, a memory that must survive hundreds of tokens, and greedy generation through the entry point and
the scheduler. Without a GPU the engine's bookkeeping runs on the CPU stand-in for the kernels (float32); the
``gpu`` tests run the same checks on the real kernels in float32 and bfloat16.
"""
import json
import os

import pytest
import torch

import plain_gibavik as plain
from gibavik_helpers import CONFIGS, GB_A, draw_weights, make_folder, read_folder, write_folder
from helpers import random_tokens, rel_err, run_plan
from kernel_double import KernelDouble
from reinfer_amd import LLMEngine, SamplingParams, kernels
from reinfer_amd.config import ConfigError, GibavikConfig, config_from_dict
from reinfer_amd.engine import ModelRunner

# float32: both sides add a few hundred float or double terms in another order over three or four layers: 2e-5 of the
# largest logit. bfloat16: one rounding is 2^-9; about a dozen storage roundings a layer, in quadrature over four
# layers: 1.3e-2 of the stream; 5e-2 is more than three deviations.
TOL = {"float32": 2e-5, "bfloat16": 5e-2}


def assert_close(got, ref, dtype, what):
    """float32: no logit further from the reference than the bound (of the largest logit). bfloat16: the same bound
    position by position, but one position in fifty (at least one) may exceed it, by up to five times: random
    weights now and then give an input at which a layer amplifies the rounding of what it reads. A lost key or state
    moves many positions, or one by far more."""
    if dtype == "float32":
        assert rel_err(got, ref) < TOL[dtype], what
        return
    got, ref = got.double().cpu(), ref.double().cpu()
    assert got.shape == ref.shape and torch.isfinite(got).all(), what
    per = (got - ref).abs().max(dim=-1).values / ref.abs().max()
    over = int((per > TOL[dtype]).sum())
    assert over <= max(1, per.numel() // 50) and float(per.max()) < 5 * TOL[dtype], (what, over, float(per.max()))


# ------------------------------------------------------------------ configuration
def test_configuration_round_trip_and_spec():
    for which, (raw, _) in CONFIGS.items():
        cfg = config_from_dict(raw)
        assert isinstance(cfg, GibavikConfig)
        assert config_from_dict(cfg.to_dict()) == cfg, which
    spec = config_from_dict(GB_A).to_spec()
    assert [b.kind for b in spec.blocks] == ["outnorm"] * 4
    assert [b.mixer.kind for b in spec.blocks] == ["side_by_side", "gqa_attention", "gqa_attention", "side_by_side"]
    assert [(e.block, e.cache_from) for e in spec.run_order] == [(0, None), (1, None), (2, 1), (3, None)]
    assert spec.blocks[2].ffn is None and spec.blocks[2].ffn_norm is None
    assert spec.final_norm.scalar and spec.blocks[0].mixer_norm.scalar
    assert not spec.tie_embeddings and spec.embed_scale == 4.0 and spec.logit_softcap == 12.0
    pair = spec.blocks[0].mixer.params
    assert pair.combine == "scaled_sum" and pair.scales == (0.7, 1.1)
    left, right = pair.members[0][1], pair.members[1][1]
    assert (left.num_heads, left.num_kv_heads, left.head_dim, left.value_dim, left.window, left.softcap) == (4, 2, 24, 16, 21, 6.0)
    assert left.qk_norm and not left.qk_norm_whole and left.rotate_values and left.out_gate and left.bias
    assert left.position.kind == "rope_neox" and left.position.rotary_dim == 12 and not left.distance_bias
    assert (right.params.heads, right.params.key_dim, right.params.value_dim, right.params.decays) == (3, 20, 12, (0.5, 0.9, 0.99))
    a, b = spec.blocks[1].mixer, spec.blocks[2].mixer
    assert a.qk_norm_whole and a.distance_bias and not a.qk_norm and not a.kv_shared and a.position.kind == "none"
    assert b.kv_shared and b.scale == 0.3 and a.window == 0
    moe = spec.blocks[0].ffn.params
    assert (moe.experts, moe.top, moe.weights, moe.activation) == (6, 2, "table", "silu_gated")
    dense = dict(spec.blocks[1].ffn.extra)
    assert dense["act"] == "swish_bounded" and dense["limit"] == 0.8
    # whatever may be absent is absent
    d = config_from_dict(CONFIGS["D"][0]).to_spec()
    assert d.embed_scale == 1.0 and d.logit_softcap == 0.0
    dl = d.blocks[0].mixer.params.members[0][1]
    assert dl.window == 0 and dl.softcap == 0.0 and not dl.rotate_values and dl.position.kind == "none" and dl.scale == 0.25
    assert d.blocks[0].mixer.params.scales == (1.0, 1.0)


def test_configuration_errors_name_the_key():
    def broken(path, value):
        raw = json.loads(json.dumps(GB_A))
        node = raw
        for k in path[:-1]:
            node = node[k]
        if value is None:
            del node[path[-1]]
        else:
            node[path[-1]] = value
        return raw
    for path, value, key in ((["width"], None, "width"), (["norm", "eps"], None, "norm.eps"),
                             (["layers", 1, "mixer", "vdim"], None, "layers[1].mixer.vdim"),
                             (["layers", 1, "mixer", "kv_heads"], 3, "layers[1].mixer.kv_heads"),
                             (["layers", 0, "mixer", "left", "rot", "dims"], 26, "layers[0].mixer.left.rot.dims"),
                             (["layers", 0, "mixer", "left", "mask", "size"], 0, "layers[0].mixer.left.mask.size"),
                             (["layers", 0, "mixer", "left", "kv_from"], 0, "layers[0].mixer.left.kv_from"),
                             (["layers", 0, "mixer", "right", "decay"], [0.5, 0.5], "layers[0].mixer.right.decay"),
                             (["layers", 0, "type"], "conv", "layers[0].type"),
                             (["layers", 0, "mlp", "router", "top"], 7, "layers[0].mlp.router.top"),
                             (["layers", 1, "mlp", "limit"], None, "layers[1].mlp.limit"),
                             (["layers", 1, "mlp", "kind"], "glu", "layers[1].mlp.kind"),
                             (["layers", 2, "mixer", "kv_from"], 2, "layers[2].mixer.kv_from"),
                             (["layers", 2, "mixer", "kv_from"], 0, "layers[2].mixer.kv_from"),
                             (["layers", 2, "mixer", "vdim"], 24, "layers[2].mixer.kv_from")):
        with pytest.raises(ConfigError) as e:
            config_from_dict(broken(path, value))
        assert e.value.key == key, (path, e.value.key)


def test_a_layer_that_reads_another_layers_keys_has_no_key_tensors(tmp_path):
    folder = make_folder(tmp_path, "A", "float32")
    _, w = read_folder(folder)
    assert {"l2.mix.q", "l2.mix.q.b", "l2.mix.q.norm", "l2.mix.r1", "l2.mix.r2", "l2.mix.o", "l2.norm1"} <= set(w)
    assert not any(n.startswith(("l2.mix.k", "l2.mix.v", "l2.mlp", "l2.norm2")) for n in w)
    assert w["l1.norm1"].shape == () and w["final.norm"].shape == ()
    assert w["l0.mlp.table"].dtype == torch.int32 and w["l0.mlp.table"].shape == (300, 2)
    assert bool((w["l0.mlp.table"][:, 0] != w["l0.mlp.table"][:, 1]).all())
    with kernels.use(KernelDouble()):
        runner = ModelRunner.from_folder(folder, dtype="float32", device="cpu", max_tokens=64)
    # three groups of block tables: all keys, a window of 5 and one of 21; the reading layer has none of its own
    assert sorted(g.window for g in runner.groups) == [0, 5, 21]
    assert runner.caches[2].k is runner.caches[1].k and not runner.caches[2].writes


# ------------------------------------------------------------------ the checks, on either device
def reference(folder, toks, cache={}):
    key = (folder, tuple(toks))
    if key not in cache:
        raw, w = read_folder(folder)
        cache[key] = plain.forward(raw, w, toks).float()
    return cache[key]


def runner_for(folder, device, dtype, **limits):
    return ModelRunner.from_folder(folder, dtype=dtype, device=device, **limits)


def vocab(which):
    return CONFIGS[which][0]["vocab"]


def check_whole_and_one_by_one(folder, which, device, dtype):
    runner = runner_for(folder, device, dtype, max_tokens=256)
    for n, seed in ((1, 5), (2, 6), (33, 3), (97, 4)):
        toks = random_tokens(n, vocab(which), seed)
        ref = reference(folder, toks)
        whole = run_plan(runner, {"r": toks}, [[("r", n)]])["r"]
        assert_close(whole, ref, dtype, (n, "whole"))
        ones = run_plan(runner, {"r": toks}, [[("r", 1)]] * n)["r"]
        assert_close(ones, ref, dtype, (n, "one by one"))
    assert all(p.num_free == p.num_blocks for p in runner.manager.pools)


def check_portions(folder, which, device, dtype):
    runner = runner_for(folder, device, dtype, max_tokens=256)
    n = 131
    toks = random_tokens(n, vocab(which), 22)
    ref = reference(folder, toks)
    for cuts in ([7, 2, 16, 3, 2, 17, 2, 31, 2, 15, 1, 16, 2, 2, 13], [64, 2, 62, 1, 1, 1], [2] * 20 + [91],
                 [100] + [1] * 31, [1, 1, 2, 1, 3, 123]):
        assert sum(cuts) == n
        got = run_plan(runner, {"r": toks}, [[("r", c)] for c in cuts])["r"]
        assert_close(got, ref, dtype, cuts[:4])


def check_mixed_with_reuse(folder, which, device, dtype):
    """Six requests in a pool of 128 tokens and four state slots: blocks and slots go back and are taken again;
    freed blocks are filled with NaN and every state slot starts out as NaN, so that a read outside a request's
    own, or a memory that is not cleared at a request's start, shows."""
    runner = runner_for(folder, device, dtype, max_tokens=128, max_seqs=4)
    lens = {"a": 30, "b": 20, "c": 30, "d": 20, "e": 40, "f": 25}
    plan = [[("a", 9), ("b", 2)],
            [("a", 1), ("b", 17), ("c", 5)],
            [("a", 20), ("b", 1), ("c", 12), ("d", 17)],
            [("c", 13), ("d", 3), ("e", 3)],
            [("e", 36), ("f", 2)],
            [("e", 1), ("f", 23)]]
    seqs = {r: random_tokens(n, vocab(which), 300 + i) for i, (r, n) in enumerate(lens.items())}
    for c in runner.paged_caches():
        for t in c.tensors.values():
            t.fill_(float("nan"))
    poisoned = 0
    for top in runner.caches:
        for c in (top.flat() if top is not None else ()):
            if c.state is not None:
                c.state.fill_(float("nan"))
                poisoned += 1
    assert poisoned == sum(L["type"] == "parallel" for L in CONFIGS[which][0]["layers"])
    runner.poison_freed_blocks()
    got = run_plan(runner, seqs, plan)
    for r, toks in seqs.items():
        assert_close(got[r], reference(folder, toks), dtype, r)
    assert all(p.num_free == p.num_blocks for p in runner.manager.pools)
    # each request alone gives the same logits as in the batch, beyond rounding
    alone = run_plan(runner, {"c": seqs["c"]}, [[("c", 30)]])["c"]
    assert rel_err(alone, got["c"]) < TOL[dtype]


def check_long_decoding(folder, which, device, dtype):
    runner = runner_for(folder, device, dtype, max_tokens=256)
    n = 150
    toks = random_tokens(n, vocab(which), 23)
    got = run_plan(runner, {"r": toks}, [[("r", 3)]] + [[("r", 1)]] * (n - 3))["r"]
    assert_close(got, reference(folder, toks), dtype, "long decoding")


def check_greedy_generation(folder, which, device, dtype):
    raw, w = read_folder(folder)
    prompts = [random_tokens(n, vocab(which), 40 + n) for n in (5, 17, 33)]
    want = [plain.greedy_generate(raw, w, p, 12) for p in prompts]
    eng = LLMEngine(folder, dtype=dtype, device=device, num_blocks=32)
    outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12))
    assert [o.token_ids for o in outs] == want
    # portions of eight beside decoding requests, two state slots for three requests, and so few blocks that
    # requests wait or are recomputed
    small = LLMEngine(folder, dtype=dtype, device=device, num_blocks=8, max_num_batched_tokens=8, max_num_seqs=2,
                      admission="blocks")
    outs2 = small.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12))
    assert [o.token_ids for o in outs2] == want
    assert small.cache_stats()["blocks_free"] == small.cache_stats()["blocks_total"]


CHECKS = [check_whole_and_one_by_one, check_portions, check_mixed_with_reuse, check_long_decoding]


# ------------------------------------------------------------------ CPU: bookkeeping on the stand-in
@pytest.mark.parametrize("check", CHECKS, ids=lambda f: f.__name__)
@pytest.mark.parametrize("which", ["A", "B", "C", "D"])
def test_engine_bookkeeping_cpu(tmp_path_factory, check, which):
    folder = make_folder(tmp_path_factory.getbasetemp(), which, "float32")
    with kernels.use(KernelDouble()):
        check(folder, which, "cpu", "float32")


@pytest.mark.parametrize("which", ["A", "B"])
def test_greedy_generation_cpu(tmp_path_factory, which):
    folder = make_folder(tmp_path_factory.getbasetemp(), which, "float32")
    with kernels.use(KernelDouble()):
        check_greedy_generation(folder, which, "cpu", "float32")


# ------------------------------------------------------------------ what the tests can see
SHARP = {"q.norm": 5.0}                                   # softmax rests on one or two keys, many of them far back or at an edge
LONG_MEMORY_DECAY = 0.999                                 # the memory's slowest head keeps the first token for hundreds


def with_windows(raw, delta):
    raw = json.loads(json.dumps(raw))
    for L in raw["layers"]:
        if L["type"] == "parallel" and "mask" in L["mixer"]["left"]:
            L["mixer"]["left"]["mask"]["size"] += delta
    return raw


def test_a_window_one_off_a_far_key_and_a_lost_memory_move_the_logits(tmp_path_factory):
    """That the sharp tests can see what they are for, in the plain implementation alone: with sharp queries a
    window that is one key too wide or too narrow, the distance term left out, and other tokens in the first 40
    places each change the logits of the last 200 positions by several times the wider bound; a memory that starts
    afresh 60 tokens before the end (what a lost or cleared state slot would do at a cut) changes the last 20."""
    tmp = tmp_path_factory.getbasetemp()
    raw, w = read_folder(make_folder(tmp, "A", "float32", scales=SHARP, tag="_sharp"))
    toks = random_tokens(260, vocab("A"), 77)
    full = plain.forward(raw, w, toks).float()
    for delta in (-1, 1):
        other = plain.forward(with_windows(raw, delta), w, toks).float()
        assert rel_err(other[-200:], full[-200:]) > 3 * TOL["bfloat16"], delta
    flat = {n: (torch.zeros_like(t) if n.endswith(".r1") else t) for n, t in w.items()}
    assert rel_err(plain.forward(raw, flat, toks).float()[-200:], full[-200:]) > 3 * TOL["bfloat16"]
    other = plain.forward(raw, w, random_tokens(40, vocab("A"), 5) + toks[40:]).float()
    assert rel_err(other[-200:], full[-200:]) > 3 * TOL["bfloat16"]
    # a single side-by-side layer whose attention sees five keys: what lies further back reaches the end through
    # the memory alone
    one = {"architecture": "Gibavik", "vocab": 64, "width": 32, "norm": {"eps": 1e-5},
           "layers": [{"type": "parallel", "mlp": None,
                       "mixer": {"left": {"dim": 16, "heads": 2, "kv_heads": 1, "vdim": 16, "mask": {"size": 5}},
                                 "right": {"decay": [LONG_MEMORY_DECAY, 0.99], "dim": 16, "heads": 2, "vdim": 16},
                                 "left_scale": 0.2, "right_scale": 1.5}}]}
    w1 = {n: (t.double() if t.is_floating_point() else t) for n, t in draw_weights(one, 8).items()}
    toks = random_tokens(300, 64, 78)
    a, b = plain.forward(one, w1, toks).float(), plain.forward(one, w1, toks[-60:]).float()
    assert rel_err(a[-20:], b[-20:]) > 3 * TOL["bfloat16"]


def check_sharp(tmp, which, device, dtype):
    folder = make_folder(tmp, which, dtype, scales=SHARP, tag="_sharp")
    runner = runner_for(folder, device, dtype, max_tokens=512)
    n = 260
    toks = random_tokens(n, vocab(which), 77)
    ref = reference(folder, toks)
    for cuts in ([n], [150, 20, 1, 1, 13, 8, 9, 21, 15, 17, 5], [210] + [1] * 50, [16, 16, 32, 64, 87, 1, 44]):
        assert sum(cuts) == n
        got = run_plan(runner, {"r": toks}, [[("r", c)] for c in cuts])["r"]
        assert_close(got, ref, dtype, cuts[:3])


def check_long_memory(tmp, device, dtype):
    """Config C with its memories' slowest heads at 0.999 and the attention beside them scaled down: the first
    tokens still weigh in the state after 300."""
    raw = json.loads(json.dumps(CONFIGS["C"][0]))
    for L in raw["layers"]:
        if L["type"] == "parallel":
            L["mixer"]["right"]["decay"][-1] = LONG_MEMORY_DECAY
            L["mixer"]["left_scale"], L["mixer"]["right_scale"] = 0.2, 1.5
    folder = os.path.join(str(tmp), f"gibavik_long_{dtype}")
    if not os.path.isdir(folder):
        write_folder(folder, raw, draw_weights(raw, 35, {"bfloat16": torch.bfloat16, "float32": torch.float32}[dtype]))
    runner = runner_for(folder, device, dtype, max_tokens=512)
    n = 300
    toks = random_tokens(n, raw["vocab"], 79)
    ref = reference(folder, toks)
    for cuts in ([n], [130, 2, 1, 1, 16, 50, 100], [260] + [1] * 40):
        got = run_plan(runner, {"r": toks}, [[("r", c)] for c in cuts])["r"]
        assert_close(got, ref, dtype, cuts[:3])


def test_sharp_attention_and_long_memory_cpu(tmp_path_factory):
    with kernels.use(KernelDouble()):
        check_sharp(tmp_path_factory.getbasetemp(), "A", "cpu", "float32")
        check_long_memory(tmp_path_factory.getbasetemp(), "cpu", "float32")


def marked_key_model(tmp, dtype, window):
    """One attention layer (``window`` 0: the kind with a distance term, every earlier key; else the windowed kind of
    a side-by-side layer whose memory weighs nothing) in which the query token asks for the key of one marked token by
    a wide margin, whatever lies between: (folder, query token, marked token, filler token). A token's key and
    query depend on the token alone (no rotation); among all triples of tokens the one is taken whose smallest
    margin over the heads (the query's score for the marked key less its score for the filler's and for its own) is
    largest, and the score scale is set so that this margin is 40: with hundreds of fillers around and the distance
    term against it, the marked key still holds nearly all the weight, and losing it (a wrong block, a key masked
    at a border, a window one too narrow) changes the logits entirely."""
    H, G, d = 2, 1, 16
    if window:
        mixer = {"left": {"dim": d, "heads": H, "kv_heads": G, "vdim": 16, "mask": {"size": window}, "scale": 1.0},
                 "right": {"decay": [0.5], "dim": 8, "heads": 1, "vdim": 8}, "left_scale": 1.0, "right_scale": 0.0}
        raw = {"architecture": "Gibavik", "vocab": 48, "width": 32, "norm": {"eps": 1e-5}, "embedding": {"scale": 2.0},
               "layers": [{"type": "parallel", "mlp": None, "mixer": mixer}]}
        p = "l0.mix.left."
    else:
        raw = {"architecture": "Gibavik", "vocab": 48, "width": 32, "norm": {"eps": 1e-5}, "embedding": {"scale": 2.0},
               "layers": [{"type": "attention", "mlp": None,
                           "mixer": {"dim": d, "heads": H, "kv_heads": G, "vdim": 16, "scale": 1.0}}]}
        p = "l0.mix."
    w = {n: (t.double() if t.is_floating_point() else t) for n, t in draw_weights(raw, 5, torch.float32).items()}
    if window:
        w[p + "g"] *= 0.0                         # the gate is one half everywhere
    else:
        w[p + "r2"].fill_(0.05)
    w["l0.norm1"].fill_(3.0)                      # the mixer's addend is large beside the embedding
    x = w["embed"] * 2.0                          # one row a token of the vocabulary
    q, k = x @ w[p + "q"].T + w[p + "q.b"], x @ w[p + "k"].T + w[p + "k.b"]
    if window:
        q = plain.rms(q.view(-1, H, d), 1e-5) * w[p + "q.norm"]
        k = plain.rms(k.view(-1, G, d), 1e-5) * w[p + "k.norm"]
    else:
        q = (plain.rms(q, 1e-5) * w[p + "q.norm"]).view(-1, H, d)
        k = (plain.rms(k, 1e-5) * w[p + "k.norm"]).view(-1, G, d)
    s = torch.einsum("qhd,kd->hqk", q, k[:, 0])                                       # [head, query token, key token]
    own = torch.diagonal(s, dim1=1, dim2=2)
    margin = (s[:, :, :, None] - torch.maximum(s[:, :, None, :], own[:, :, None, None])).min(0).values
    V = margin.shape[0]
    for i in range(V):
        margin[i, i, :] = -1e9
        margin[i, :, i] = -1e9
        margin[:, i, i] = -1e9
    best = int(margin.argmax())
    qt, mt, ft = best // (V * V), (best // V) % V, best % V
    assert float(margin[qt, mt, ft]) > 0.5
    (raw["layers"][0]["mixer"]["left"] if window else raw["layers"][0]["mixer"])["scale"] = 40.0 / float(margin[qt, mt, ft])
    folder = os.path.join(str(tmp), f"gibavik_marked_{window}_{dtype}")
    if not os.path.isdir(folder):
        td = {"bfloat16": torch.bfloat16, "float32": torch.float32}[dtype]
        write_folder(folder, raw, {n: (t.to(td) if t.is_floating_point() else t) for n, t in w.items()})
    return folder, qt, mt, ft


def check_marked_key(tmp, device, dtype):
    """The marked key at the first place, on both sides of block borders and hundreds of tokens back; the queries in
    the prompt's portion, in a portion of two and decoded alone. The plain implementation with the marked token
    replaced by a filler differs by most of a logit's size, so the engine cannot pass without reading that key."""
    folder, qt, mt, ft = marked_key_model(tmp, dtype, 0)
    raw, w = read_folder(folder)
    runner = runner_for(folder, device, dtype, max_tokens=512)
    n = 400
    for place in (0, 1, 15, 16, 17, 63, 64, 127, 128, 255, 256, 383):
        toks = [ft] * n
        toks[place] = mt
        for at in (n - 1, n - 2, n - 3, n - 7):
            toks[at] = qt
        ref = plain.forward(raw, w, toks).float()
        without = plain.forward(raw, w, [ft if t == mt else t for t in toks]).float()
        assert rel_err(without[-1:], ref[-1:]) > 0.2, place
        for cuts in ([n], [n - 8, 1, 2, 2, 1, 1, 1], [place + 1, n - place - 6, 2, 1, 1, 1]):
            cuts = [c for c in cuts if c > 0]
            assert sum(cuts) == n
            got = run_plan(runner, {"r": toks}, [[("r", c)] for c in cuts])["r"]
            assert_close(got[-8:], ref[-8:], dtype, (place, cuts[:2]))


def check_window_edges(tmp, device, dtype):
    """The marked key just inside and just outside the window of each of the last queries, with the window's edge
    on a block border and off it, in prompts and in decoding: with the key at the window's last place the logits
    are the marked key's, one further back they are the fillers'."""
    for window in (16, 37):
        folder, qt, mt, ft = marked_key_model(tmp, dtype, window)
        raw, w = read_folder(folder)
        runner = runner_for(folder, device, dtype, max_tokens=256)
        n = 120
        for back in (window - 2, window - 1, window, window + 1):      # distance of the marked key from the last query
            toks = [ft] * n
            toks[n - 1 - back] = mt
            toks[n - 1] = qt
            ref = plain.forward(raw, w, toks).float()
            without = plain.forward(raw, w, [ft if t == mt else t for t in toks]).float()
            seen = rel_err(without[-1:], ref[-1:]) > 0.2
            assert seen == (back < window), (window, back)
            for cuts in ([n], [n - 1, 1], [n - 2, 2], [n - back - 1, back - 1, 1, 1], [50, 1, 1] + [2] * 33 + [1, 1]):
                assert sum(cuts) == n
                got = run_plan(runner, {"r": toks}, [[("r", c)] for c in cuts])["r"]
                assert_close(got[-3:], ref[-3:], dtype, (window, back, cuts[:2]))


def test_a_marked_key_far_back_at_block_borders_and_at_window_edges_cpu(tmp_path_factory):
    with kernels.use(KernelDouble()):
        check_marked_key(tmp_path_factory.getbasetemp(), "cpu", "float32")
        check_window_edges(tmp_path_factory.getbasetemp(), "cpu", "float32")


# ------------------------------------------------------------------ GPU: the real kernels
GPU_CASES = [("A", "float32"), ("B", "float32"), ("C", "float32"), ("D", "float32"), ("C", "bfloat16"), ("A", "bfloat16")]


@pytest.mark.gpu
@pytest.mark.parametrize("check", CHECKS, ids=lambda f: f.__name__)
@pytest.mark.parametrize("which,dtype", GPU_CASES)
def test_engine_gpu(tmp_path_factory, check, which, dtype):
    assert kernels.current().name == "hip-gfx950"
    folder = make_folder(tmp_path_factory.getbasetemp(), which, dtype)
    check(folder, which, "cuda:0", dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("which,dtype", [("A", "float32"), ("C", "float32"), ("C", "bfloat16")])
def test_sharp_attention_gpu(tmp_path_factory, which, dtype):
    check_sharp(tmp_path_factory.getbasetemp(), which, "cuda:0", dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_memory_gpu(tmp_path_factory, dtype):
    check_long_memory(tmp_path_factory.getbasetemp(), "cuda:0", dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_marked_key_far_back_at_block_borders_and_at_window_edges_gpu(tmp_path_factory, dtype):
    check_marked_key(tmp_path_factory.getbasetemp(), "cuda:0", dtype)
    check_window_edges(tmp_path_factory.getbasetemp(), "cuda:0", dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("which,dtype", [("A", "float32"), ("C", "bfloat16")])
def test_greedy_generation_gpu(tmp_path_factory, which, dtype):
    folder = make_folder(tmp_path_factory.getbasetemp(), which, dtype)
    if dtype == "float32":
        check_greedy_generation(folder, which, "cuda:0", dtype)
        return
    # bfloat16: the engine's own tokens must be the same however the requests are batched and cut
    prompts = [random_tokens(n, vocab(which), 40 + n) for n in (5, 17, 33, 64)]
    eng = LLMEngine(folder, dtype=dtype, device="cuda:0", num_blocks=64)
    a = [o.token_ids for o in eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=24))]
    alone = [eng.generate([p], SamplingParams(temperature=0.0, max_tokens=24))[0].token_ids for p in prompts]
    assert all(len(t) == 24 for t in a) and all(0 <= x < vocab(which) for t in a for x in t)
    same = sum(x == y for x, y in zip(a, alone))
    assert same >= len(prompts) - 1, "greedy tokens changed with the batch"      # a tie after rounding may flip one


@pytest.mark.gpu
@pytest.mark.parametrize("which,dtype", [("A", "float32"), ("C", "bfloat16")])
def test_captured_decode_steps_gpu(tmp_path_factory, which, dtype):
    """Decode steps replay captured graphs: the same logits as a runner without graphs, over several replays
    with eager prompt steps between them, state slots and blocks changing hands meanwhile. (bfloat16: a captured
    step cuts a token's keys into chunks by its context bucket, not by the step's longest context, so the two
    runners add the same terms in another order.)"""
    folder = make_folder(tmp_path_factory.getbasetemp(), which, dtype)
    seqs = {r: random_tokens(n, vocab(which), 500 + i) for i, (r, n) in enumerate((("a", 40), ("b", 25), ("c", 31)))}
    plan = [[("a", 10), ("b", 5)]] + [[("a", 1), ("b", 1)]] * 6 + [[("c", 9)]] + [[("a", 1), ("b", 1), ("c", 1)]] * 8 \
        + [[("a", 16), ("b", 6), ("c", 14)]]
    outs = []
    for graphs in (True, False):
        runner = runner_for(folder, "cuda:0", dtype, max_tokens=256, use_graphs=graphs)
        outs.append(run_plan(runner, seqs, plan))
        if graphs:
            assert runner.graphs is not None and runner.graphs.replays >= 14
    for r, toks in seqs.items():
        assert rel_err(outs[0][r], outs[1][r]) < (1e-6 if dtype == "float32" else 2e-2), r
        assert_close(outs[0][r], reference(folder, toks), dtype, r)


def test_command_line_init_writes_a_loadable_folder(tmp_path):
    """``reinfer init`` with this design's config.json: a folder the engine loads, every declared tensor in it."""
    from reinfer_amd import cli
    src = tmp_path / "config.json"
    src.write_text(json.dumps(GB_A))
    out = tmp_path / "model"
    assert cli.main(["init", str(src), "--seed", "3", "--out", str(out), "--dtype", "float32"]) == 0
    raw, w = read_folder(str(out))
    assert raw["architecture"] == "Gibavik" and raw["layers"][2]["mlp"] is None and raw["layers"][2]["mixer"]["kv_from"] == 1
    assert {"embed", "head", "final.norm", "l0.norm1", "l0.norm2", "l0.mix.left.q", "l0.mix.left.q.b", "l0.mix.left.k.norm",
            "l0.mix.left.g", "l0.mix.left.o", "l0.mix.right.q", "l0.mix.right.norm", "l0.mix.right.g", "l0.mix.right.o",
            "l0.mlp.e5.gate", "l0.mlp.table", "l1.mix.q.norm", "l1.mix.k.norm", "l1.mix.r1", "l1.mix.r2", "l1.mix.v.b",
            "l1.mlp.down", "l2.mix.q", "l3.mlp.e2.down"} <= set(w)
    assert "l2.mix.k" not in w and "l0.mlp.e6.gate" not in w and "l0.mlp.router" not in w
    assert w["l0.mix.left.q.norm"].shape == (24,) and w["l1.mix.q.norm"].shape == (96,) and w["l1.mix.k.norm"].shape == (48,)
    assert w["l0.mix.left.g"].shape == (64, 64) and w["l0.mix.right.norm"].shape == (36,) and w["l1.mix.r1"].shape == (4,)
    tab = w["l3.mlp.table"]
    assert tab.shape == (300, 3) and int(tab.min()) == 0 and int(tab.max()) == 2
    assert all(len(set(row)) == 3 for row in tab.tolist())
    with kernels.use(KernelDouble()):
        eng = LLMEngine(str(out), dtype="float32", device="cpu", num_blocks=16)
        toks = eng.generate([[1, 2, 3]], SamplingParams(temperature=0.0, max_tokens=4))[0].token_ids
    assert toks == plain.greedy_generate(raw, w, [1, 2, 3], 4)


@pytest.mark.gpu
def test_command_line_run_gpu(tmp_path):
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    folder = make_folder(tmp_path, "A", "float32")
    raw, w = read_folder(folder)
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "reinfer"), "run", folder, "-n", "8", "-t", "0",
                        "--dtype", "float32", "--num-blocks", "16", "--max-model-len", "128", "--", "5", "9", "200"],
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [int(t) for t in r.stdout.split()] == plain.greedy_generate(raw, w, [5, 9, 200], 8)
