"""Detatar through the engine against the plain implementation: configuration, whole prompts, prompts against
token-by-token decoding, portions down to two tokens, unequal requests in one batch with blocks and state slots that
are given back and used again, the first tokens, long decoding, keys far back and at block borders made to stand
out, a state that must survive hundreds of tokens, and greedy generation through the entry point and the scheduler.
Without a GPU the engine's bookkeeping runs on the CPU stand-in for the kernels (float32); the ``gpu`` tests run
the same checks on the real kernels in float32 and bfloat16.

bfloat16 runs use the configuration whose routers choose every expert: which of two nearly equal scores is the
larger after rounding is decided differently by any two implementations, and the choice itself is checked in
float32 and in the kernel tests."""
import json
import os

import pytest
import torch

import plain_detatar as plain
from detatar_helpers import CONFIGS, DT_A, config_json, make_folder, read_folder
from helpers import random_tokens, rel_err, run_plan
from kernel_double import KernelDouble
from reinfer_amd import LLMEngine, SamplingParams, kernels
from reinfer_amd.config import ConfigError, DetatarConfig, config_from_dict
from reinfer_amd.engine import ModelRunner

# float32: both sides add a few hundred float or double terms in another order over four layers, and the wkv state
# carries its rounding on for as long as its decays keep it: 2e-5 of the largest logit. bfloat16: one rounding is
# 2^-9; about a dozen storage roundings a layer, in quadrature over three or four layers: 1.3e-2 of the stream;
# 5e-2 is more than three deviations.
TOL = {"float32": 2e-5, "bfloat16": 5e-2}


def assert_close(got, ref, dtype, what):
    """float32: no logit further from the reference than the bound (of the largest logit). bfloat16: the same bound
    position by position, but one position in fifty (at least one) may exceed it, by up to five times: random
    weights now and then give an input at which a layer amplifies the rounding of what it reads (seen once among
    ten random configurations: one position of seventy at 0.12, the others at 0.013 in the middle, while float32
    on the same weights agreed to 2e-6 there and the engine's own bfloat16 results for the whole prompt and for
    portions agreed to 4e-3). A lost key or state moves many positions, or one by far more."""
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
        assert isinstance(cfg, DetatarConfig)
        assert config_from_dict(cfg.to_dict()) == cfg, which
        assert cfg.to_dict()["layers"] == config_from_dict(json.loads(json.dumps(cfg.to_dict()))).to_dict()["layers"]
    spec = config_from_dict(DT_A).to_spec()
    # three blocks hold tensors; the fourth layer runs the second block again
    assert [b.mixer.kind for b in spec.blocks] == ["latent_attention", "wkv", "latent_attention"]
    assert [e.block for e in spec.run_order] == [0, 1, 2, 1]
    assert all(b.kind == "parallel" and b.params.token_shift and b.params.gated for b in spec.blocks)
    assert spec.blocks[2].ffn is None
    assert not spec.tie_embeddings and spec.embed_scale == 2.5
    assert spec.final_norm.groups == 2 and spec.blocks[0].mixer_norm.groups == 2
    a = spec.blocks[0].mixer
    assert (a.num_heads, a.head_dim, a.params.rot_width, a.params.value_dim, a.params.rank, a.params.q_rank) == (3, 16, 8, 24, 40, 24)
    assert a.params.head_gate and a.position.kind == "rope_neox" and a.position.rotary_dim == 8
    c = spec.blocks[2].mixer
    assert (c.position.rotary_dim, c.position.theta, c.scale) == (12, 500.0, 0.3)
    w = spec.blocks[1].mixer.params
    assert (w.heads, w.dim, w.decay_rank) == (2, 20, 12)
    moe = spec.blocks[0].ffn.params
    assert (moe.experts, moe.identity, moe.top, moe.groups, moe.groups_kept, moe.group_top, moe.shared) == (6, 2, 2, 4, 2, 1, 40)
    assert moe.weights == "softmax" and moe.correction and moe.norm_eps == 1e-20 and moe.shared_gated
    assert dict(spec.blocks[1].ffn.extra)["act"] == "gelu_tanh"
    # whatever may be absent is absent
    d = config_from_dict(CONFIGS["D"][0]).to_spec()
    assert d.embed_scale == 1.0 and d.final_norm.groups == 1
    m = d.blocks[0].ffn.params
    assert (m.identity, m.groups, m.groups_kept, m.shared, m.shared_gated) == (0, 1, 1, 0, False)


def test_the_decay_rank_comes_from_the_tensors(tmp_path):
    folder = make_folder(tmp_path, "A", "float32")
    with open(os.path.join(folder, "config.json")) as f:
        assert "decay_ranks" not in json.load(f)
    with kernels.use(KernelDouble()):
        runner = ModelRunner.from_folder(folder, dtype="float32", device="cpu", max_tokens=64)
    assert runner.model.spec.blocks[1].mixer.params.decay_rank == 12
    with pytest.raises(ConfigError) as e:
        config_from_dict(config_json(DT_A)).to_spec()
    assert e.value.key == "layers[1].mixer"


def test_configuration_errors_name_the_key():
    def broken(path, value):
        raw = json.loads(json.dumps(DT_A))
        node = raw
        for k in path[:-1]:
            node = node[k]
        if value is None:
            del node[path[-1]]
        else:
            node[path[-1]] = value
        return raw
    for path, value, key in ((["width"], None, "width"), (["norm", "eps"], None, "norm.eps"),
                             (["norm", "groups"], 3, "norm.groups"),
                             (["layers", 0, "mixer", "vdim"], None, "layers[0].mixer.vdim"),
                             (["layers", 0, "mixer", "q_rank"], 0, "layers[0].mixer.q_rank"),
                             (["layers", 2, "mixer", "rot", "dims"], 18, "layers[2].mixer.rot.dims"),
                             (["layers", 1, "type"], "conv", "layers[1].type"),
                             (["layers", 1, "mixer", "heads"], 0, "layers[1].mixer.heads"),
                             (["layers", 0, "mlp", "router", "top"], 5, "layers[0].mlp.router.top"),
                             (["layers", 0, "mlp", "router", "groups", "count"], 3, "layers[0].mlp.router.groups.count"),
                             (["layers", 0, "mlp", "router", "groups", "keep"], 5, "layers[0].mlp.router.groups.keep"),
                             (["layers", 1, "mlp", "kind"], "glu", "layers[1].mlp.kind"),
                             (["layers", 3, "weights_of"], 3, "layers[3].weights_of"),
                             (["layers", 3, "mixer", "dim"], 24, "layers[3].weights_of")):
        with pytest.raises(ConfigError) as e:
            config_from_dict(broken(path, value))
        assert e.value.key == key, (path, e.value.key)


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
    """Six requests in a pool of 128 tokens and four state slots: blocks and slots go back and are taken
    again; freed blocks are filled with NaN and every state slot starts out as NaN (the wkv state, its row before
    and the layer's row before alike), so that a read outside a request's own, or a state that is not cleared at
    a request's start, shows."""
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
    # every layer run keeps a row before; a wkv layer a state beside it
    raw = CONFIGS[which][0]
    assert poisoned == len(raw["layers"]) + sum(L["type"] == "wkv" for L in raw["layers"])
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
SHARP = {"uq": 8.0}                                       # softmax rests on one or two keys, many of them far back
LONG_MEMORY = {"w0": -4.0}                                # decays between 0.96 and 0.998: the state lasts


def test_a_far_key_and_a_lost_state_move_the_logits(tmp_path_factory):
    """That the sharp and the long-memory tests can see what they are for, in the plain implementation alone:
    with sharp queries, other tokens in the first 40 places change the logits of the last 200 by several times
    the wider bound; with long memories, a state that starts afresh 50 tokens before the end (what a lost or
    cleared state slot would do at a cut) changes the last 20."""
    tmp = tmp_path_factory.getbasetemp()
    raw, w = read_folder(make_folder(tmp, "C", "float32", scales=SHARP, tag="_sharp"))
    # the wkv layer ahead of the attention layers forgets within a few tokens here (its decays are 0.1 to 0.9)
    toks = random_tokens(300, vocab("C"), 77)
    full = plain.forward(raw, w, toks)
    other = plain.forward(raw, w, random_tokens(40, vocab("C"), 5) + toks[40:])
    assert rel_err(other[-200:].float(), full[-200:].float()) > 3 * TOL["bfloat16"]
    raw, w = read_folder(make_folder(tmp, "B", "float32", shifts=LONG_MEMORY, tag="_long"))
    toks = random_tokens(300, vocab("B"), 78)
    a, b = plain.forward(raw, w, toks), plain.forward(raw, w, toks[-50:])         # no layer of B knows positions
    assert rel_err(a[-20:].float(), b[-20:].float()) > 4 * TOL["bfloat16"]


def test_the_row_before_moves_the_logits(tmp_path_factory):
    """A kept row that is lost at a cut (zeros instead of the token before) must show: the plain implementation
    run on a sequence's second half alone differs from the whole at that half's first token by far more than the
    bound, also for the attention layers, which have no other state."""
    raw, w = read_folder(make_folder(tmp_path_factory.getbasetemp(), "B", "float32"))
    toks = random_tokens(12, vocab("B"), 9)
    a, b = plain.forward(raw, w, toks), plain.forward(raw, w, toks[6:])
    assert rel_err(b[:1].float(), a[6:7].float()) > 4 * TOL["bfloat16"]


def check_sharp_and_long(tmp, which, device, dtype, scales, shifts, tag):
    folder = make_folder(tmp, which, dtype, scales=scales, shifts=shifts, tag=tag)
    runner = runner_for(folder, device, dtype, max_tokens=512)
    n = 300
    toks = random_tokens(n, vocab(which), 77)
    ref = reference(folder, toks)
    for cuts in ([n], [150, 20, 1, 1, 13, 8, 9, 21, 15, 17, 45], [250] + [1] * 50, [16, 16, 32, 64, 127, 1, 44]):
        assert sum(cuts) == n
        got = run_plan(runner, {"r": toks}, [[("r", c)] for c in cuts])["r"]
        assert_close(got, ref, dtype, cuts[:3])


def test_sharp_attention_and_long_memory_cpu(tmp_path_factory):
    with kernels.use(KernelDouble()):
        check_sharp_and_long(tmp_path_factory.getbasetemp(), "A", "cpu", "float32", SHARP, None, "_sharp")
        check_sharp_and_long(tmp_path_factory.getbasetemp(), "B", "cpu", "float32", None, LONG_MEMORY, "_long")


def far_key_model(tmp, dtype):
    """One attention layer in which every head of one query token asks for the key of one marked token by a wide
    margin, whatever lies between: (folder, query token, marked token, filler token). The layer's shift is zero and
    the rotated part nearly so, so a token's key and query depend on the token alone; among all triples of tokens
    the one is taken whose smallest margin over the heads (the query's score for the marked key less its score
    for the filler's and for its own) is largest, and the score scale is set so that this margin is 30: with
    hundreds of fillers around, the marked key still holds all but e^-24 of the weight, and losing it (a wrong
    block, a key masked at a border) changes the logits entirely."""
    from detatar_helpers import draw_weights, write_folder
    H, d, R, rank = 2, 8, 4, 16
    raw = {"architecture": "Detatar", "vocab": 48, "width": 32, "norm": {"eps": 1e-5, "groups": 2},
           "embedding": {"scale": 2.0},
           "layers": [{"type": "latent_attention", "mlp": None,
                       "mixer": {"dim": d, "heads": H, "kv_rank": rank, "q_rank": 8, "rot_dim": R, "scale": 1.0,
                                 "vdim": 8, "rot": {"base": 10000.0, "dims": R}}}]}
    w = {n: t.double() for n, t in draw_weights(raw, 5, torch.float32).items()}
    w["l0.shift"].zero_()
    w["l0.mix.dkv"][rank:] *= 0.01
    w["l0.rg1.b"].fill_(3.0)                  # the mixer's addend enters nearly whole, and is large beside the embedding
    w["l0.mix.o"] *= 4.0
    h = plain.group_norm(w["embed"] * 2.0, w["l0.norm1"], 2, 1e-5)                    # one row a token of the vocabulary
    q = ((plain.rms(h @ w["l0.mix.dq"].T, 1e-5) * w["l0.mix.dq.norm"]) @ w["l0.mix.uq"].T).view(-1, H, d + R)[..., :d]
    c = plain.rms((h @ w["l0.mix.dkv"].T)[:, :rank], 1e-5) * w["l0.mix.dkv.norm"]
    k = (c @ w["l0.mix.uk"].T).view(-1, H, d)
    s = torch.einsum("qhd,khd->hqk", q, k)                                            # [head, query token, key token]
    own = torch.diagonal(s, dim1=1, dim2=2)                                           # [head, query token]
    # margin[q, m, f] = min over heads of s[q, m] - max(s[q, f], s[q, q])
    margin = (s[:, :, :, None] - torch.maximum(s[:, :, None, :], own[:, :, None, None])).min(0).values
    V = margin.shape[0]
    for i in range(V):
        margin[i, i, :] = -1e9
        margin[i, :, i] = -1e9
        margin[:, i, i] = -1e9
    best = int(margin.argmax())
    qt, mt, ft = best // (V * V), (best // V) % V, best % V
    assert float(margin[qt, mt, ft]) > 0.5
    raw["layers"][0]["mixer"]["scale"] = 30.0 / float(margin[qt, mt, ft])
    folder = os.path.join(str(tmp), f"detatar_far_key_{dtype}")
    if not os.path.isdir(folder):
        os.makedirs(folder)
        from reinfer_amd.weights.safetensors_io import write_safetensors
        with open(os.path.join(folder, "config.json"), "w") as f:
            json.dump(raw, f)
        td = {"bfloat16": torch.bfloat16, "float32": torch.float32}[dtype]
        write_safetensors(os.path.join(folder, "model.safetensors"), {n: t.to(td) for n, t in w.items()},
                          metadata={"format": "pt"})
    return folder, qt, mt, ft


def check_far_key(tmp, device, dtype):
    """The marked key at the first place, on both sides of block borders and hundreds of tokens back; the queries
    in the prompt's portion, in a portion of two and decoded alone. The plain implementation with the marked token
    replaced by a filler differs by most of a logit's size, so the engine cannot pass without reading that key."""
    folder, qt, mt, ft = far_key_model(tmp, dtype)
    raw, w = read_folder(folder)
    runner = runner_for(folder, device, dtype, max_tokens=512)
    n = 400
    for place in (0, 1, 15, 16, 17, 31, 32, 63, 64, 127, 128, 255, 256, 383):
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


def test_a_marked_key_far_back_and_at_block_borders_cpu(tmp_path_factory):
    with kernels.use(KernelDouble()):
        check_far_key(tmp_path_factory.getbasetemp(), "cpu", "float32")


# ------------------------------------------------------------------ GPU: the real kernels
GPU_CASES = [("A", "float32"), ("B", "float32"), ("C", "float32"), ("D", "float32"), ("C", "bfloat16"), ("B", "bfloat16")]


@pytest.mark.gpu
@pytest.mark.parametrize("check", CHECKS, ids=lambda f: f.__name__)
@pytest.mark.parametrize("which,dtype", GPU_CASES)
def test_engine_gpu(tmp_path_factory, check, which, dtype):
    assert kernels.current().name == "hip-gfx950"
    folder = make_folder(tmp_path_factory.getbasetemp(), which, dtype)
    check(folder, which, "cuda:0", dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("which,dtype,scales,shifts,tag", [
    ("A", "float32", SHARP, None, "_sharp"), ("C", "bfloat16", SHARP, None, "_sharp"),
    ("B", "float32", None, LONG_MEMORY, "_long"), ("C", "float32", SHARP, LONG_MEMORY, "_both")])
def test_sharp_attention_and_long_memory_gpu(tmp_path_factory, which, dtype, scales, shifts, tag):
    check_sharp_and_long(tmp_path_factory.getbasetemp(), which, "cuda:0", dtype, scales, shifts, tag)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_marked_key_far_back_and_at_block_borders_gpu(tmp_path_factory, dtype):
    check_far_key(tmp_path_factory.getbasetemp(), "cuda:0", dtype)


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
def test_captured_decode_steps_gpu(tmp_path_factory):
    """Decode steps replay captured graphs: the same logits as a runner without graphs, over several replays
    with eager prompt steps between them, state slots and blocks changing hands meanwhile."""
    folder = make_folder(tmp_path_factory.getbasetemp(), "A", "float32")
    seqs = {r: random_tokens(n, vocab("A"), 500 + i) for i, (r, n) in enumerate((("a", 40), ("b", 25), ("c", 31)))}
    plan = [[("a", 10), ("b", 5)]] + [[("a", 1), ("b", 1)]] * 6 + [[("c", 9)]] + [[("a", 1), ("b", 1), ("c", 1)]] * 8 \
        + [[("a", 16), ("b", 6), ("c", 14)]]
    outs = []
    for graphs in (True, False):
        runner = runner_for(folder, "cuda:0", "float32", max_tokens=256, use_graphs=graphs)
        outs.append(run_plan(runner, seqs, plan))
        if graphs:
            assert runner.graphs is not None and runner.graphs.replays >= 14
    for r, toks in seqs.items():
        assert rel_err(outs[0][r], outs[1][r]) < 1e-6, r
        assert rel_err(outs[0][r], reference(folder, toks)) < TOL["float32"], r


def test_command_line_init_writes_a_loadable_folder(tmp_path):
    """``reinfer init`` with this design's config.json: a folder the engine loads, every declared tensor in it."""
    from reinfer_amd import cli
    src = tmp_path / "config.json"
    src.write_text(json.dumps(DT_A))
    out = tmp_path / "model"
    assert cli.main(["init", str(src), "--seed", "3", "--out", str(out), "--dtype", "float32"]) == 0
    raw, w = read_folder(str(out))
    assert raw["architecture"] == "Detatar" and raw["layers"][2]["mlp"] is None and raw["layers"][3]["weights_of"] == 1
    assert {"embed", "head", "final.norm", "l0.norm1", "l0.shift", "l0.rg1", "l0.rg2.b", "l0.mix.dq", "l0.mix.dq.norm",
            "l0.mix.uq", "l0.mix.dkv", "l0.mix.dkv.norm", "l0.mix.uk", "l0.mix.uv", "l0.mix.g", "l0.mix.o",
            "l0.mlp.e5.gate", "l0.mlp.router", "l0.mlp.correction", "l0.mlp.shared.down", "l0.mlp.shared.sg",
            "l1.mix.mu.w", "l1.mix.w1", "l1.mix.w2", "l1.mix.w0", "l1.mix.u", "l1.mix.norm", "l1.mlp.down",
            "l2.rg1.b"} <= set(w)
    assert not any(n.startswith("l3.") for n in w) and "l2.rg2" not in w and "l0.mlp.e6.gate" not in w
    assert w["l0.mlp.router"].shape == (8, 64) and w["l0.mix.g"].shape == (3, 64) and w["l1.mix.w1"].shape == (12, 64)
    assert w["l0.mix.dkv"].shape == (48, 64) and w["l0.mix.uq"].shape == (72, 24) and w["l1.mix.u"].shape == (2, 20)
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
