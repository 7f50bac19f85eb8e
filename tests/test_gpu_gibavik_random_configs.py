"""Gibavik configurations drawn at random (sizes, head counts, layer order, layers that read an earlier layer's keys,
windows, every optional key present or absent), each run through the engine against the plain implementation: a
whole prompt, portions beside single tokens of other requests, and decoding, on a cache and state slots that are
given back and taken again, in float32 and in bfloat16. A second set draws the sizes of a larger model (heads of 64
to 128, windows of hundreds, dozens of experts)."""
import json
import os
import random

import pytest
import torch

import plain_gibavik as plain
from gibavik_helpers import draw_weights, read_folder, write_folder
from helpers import random_tokens, rel_err, run_plan
from test_gibavik_engine import assert_close
from reinfer_amd.engine import ModelRunner

pytestmark = pytest.mark.gpu


def draw_config(rng: random.Random, wide: bool = False) -> dict:
    width = rng.choice([24, 36, 40, 64, 72] if not wide else [128, 160, 256])

    def heads():
        kv = rng.choice([1, 2, 3, 4] if not wide else [1, 2, 4])
        return kv * rng.choice([1, 2, 3, 4, 8] if not wide else [1, 2, 4, 7]), kv

    def full(kv_from=None, like=None):
        if like is not None:
            m = {k: like[k] for k in ("dim", "heads", "kv_heads", "vdim")}
            m["scale"] = rng.choice([0.1, 0.25, 0.5])
            m["kv_from"] = kv_from
            return m
        H, G = heads()
        m = {"dim": rng.choice([4, 8, 12, 16, 24, 40, 48] if not wide else [64, 80, 96, 128]), "heads": H, "kv_heads": G,
             "vdim": rng.choice([4, 8, 16, 20, 32, 56] if not wide else [32, 64, 96, 128])}
        if rng.random() < 0.8:
            m["scale"] = rng.choice([0.1, 0.25, 0.5])
        return m

    def left():
        H, G = heads()
        dim = rng.choice([4, 8, 12, 16, 24, 40, 48] if not wide else [64, 80, 96, 128])
        m = {"dim": dim, "heads": H, "kv_heads": G,
             "vdim": rng.choice([4, 8, 16, 20, 32, 56] if not wide else [32, 64, 96, 128])}
        if rng.random() < 0.85:
            m["mask"] = {"size": rng.choice([1, 2, 5, 16, 17, 33, 64] if not wide else [16, 100, 150, 257])}
        if rng.random() < 0.85:
            m["rot"] = {"base": rng.choice([100.0, 10000.0, 500000.0]), "dims": rng.choice([d for d in (2, 4, 8, 16, 32, 64, dim) if d <= dim and d % 2 == 0])}
        if rng.random() < 0.8:
            m["softcap"] = rng.choice([2.0, 25.0, 50.0])
        if rng.random() < 0.8:
            m["scale"] = rng.choice([0.1, 0.25, 0.5])
        return m

    def right():
        H = rng.choice([1, 2, 3, 5] if not wide else [2, 4, 8])
        return {"decay": [rng.choice([0.3, 0.6, 0.9, 0.97, 0.999]) for _ in range(H)],
                "dim": rng.choice([4, 9, 16, 32, 40, 64, 72] if not wide else [64, 128, 136]), "heads": H,
                "vdim": rng.choice([4, 8, 12, 32, 40] if not wide else [32, 64, 128])}

    def mlp():
        kind = rng.choice(["dense", "moe", "moe", None])
        if kind is None:
            return None
        if kind == "dense":
            return {"ff": rng.choice([16, 40, 100] if not wide else [256, 384]), "kind": "dense",
                    "limit": rng.choice([0.5, 1.0, 3.0, 7.0])}
        experts = rng.choice([1, 2, 3, 5, 8] if not wide else [8, 16, 32])
        return {"expert": {"ff": rng.choice([8, 20, 48] if not wide else [64, 96])}, "kind": "moe",
                "router": {"experts": experts, "top": rng.randint(1, min(experts, 4))}}

    layers = []
    for i in range(rng.randint(2, 5)):
        own = [j for j, L in enumerate(layers) if L["type"] == "attention" and "kv_from" not in L["mixer"]]
        if own and rng.random() < 0.3:
            j = rng.choice(own)
            layers.append({"type": "attention", "mixer": full(j, layers[j]["mixer"]), "mlp": mlp()})
        elif rng.random() < 0.5:
            pair = {"left": left(), "right": right()}
            if rng.random() < 0.8:
                pair["left_scale"], pair["right_scale"] = rng.choice([0.3, 0.7, 1.0]), rng.choice([0.5, 0.8, 1.4])
            layers.append({"type": "parallel", "mixer": pair, "mlp": mlp()})
        else:
            layers.append({"type": "attention", "mixer": full(), "mlp": mlp()})
    raw = {"architecture": "Gibavik", "vocab": rng.choice([50, 131, 400]), "width": width,
           "norm": {"eps": rng.choice([1e-6, 1e-5])}, "layers": layers}
    if rng.random() < 0.8:
        raw["embedding"] = {"scale": rng.choice([1.0, 3.0, 9.0])}
    if rng.random() < 0.8:
        raw["logit_softcap"] = rng.choice([5.0, 18.0, 30.0])
    return raw


@pytest.mark.parametrize("seed,dtype", [(s, "float32") for s in range(16)] + [(s, "bfloat16") for s in range(16, 28)]
                         + [(s, "float32") for s in range(100, 106)] + [(s, "bfloat16") for s in range(106, 112)])
def test_random_configuration(tmp_path, seed, dtype):
    rng = random.Random(3000 + seed)
    raw = draw_config(rng, wide=seed >= 100)
    print("configuration:", json.dumps(raw), flush=True)
    folder = write_folder(str(tmp_path / "m"), raw,
                          draw_weights(raw, seed, torch.bfloat16 if dtype == "bfloat16" else torch.float32))
    raw, w = read_folder(folder)
    V = raw["vocab"]
    lens = {"a": rng.randint(60, 140), "b": rng.randint(20, 70), "c": rng.randint(5, 40), "d": rng.randint(2, 30),
            "e": rng.randint(30, 90)}
    if seed >= 100:
        lens["a"] = rng.randint(280, 330)                           # past the widest window
    seqs = {r: random_tokens(n, V, seed * 10 + i) for i, (r, n) in enumerate(lens.items())}
    refs = {r: plain.forward(raw, w, t).float() for r, t in seqs.items()}
    # a plan of random portions: up to four live requests, the fifth comes when one has ended; the last tokens one by one
    left = dict(lens)
    waiting, live, plan = list(lens), [], []
    while waiting or live:
        while waiting and len(live) < 4:
            live.append(waiting.pop(0))
        items = []
        for r in list(live):
            if rng.random() < 0.25 and len(live) > 1:
                continue                                            # left out of this step
            c = 1 if left[r] <= 6 else min(left[r] - 6, rng.choice([1, 2, 3, 7, 16, 17, 33, 64, 130]))
            items.append((r, c))
            left[r] -= c
            if left[r] == 0:
                live.remove(r)
        if items:
            plan.append(items)
    runner = ModelRunner.from_folder(folder, dtype=dtype, device="cuda:0", max_tokens=384 + 3 * 192, max_seqs=4)
    runner.poison_freed_blocks()
    got = run_plan(runner, seqs, plan)
    whole = run_plan(runner, {"a": seqs["a"]}, [[("a", lens["a"])]])["a"]
    if dtype == "float32":
        bound = 1e-4 if seed >= 100 else 3e-5
        for r in seqs:
            assert rel_err(got[r], refs[r]) < bound, (r, json.dumps(raw))
        assert rel_err(whole, refs["a"]) < bound, json.dumps(raw)
        # and the schedule itself changes nothing beyond the last bits
        assert rel_err(whole, got["a"]) < 3e-5, json.dumps(raw)
    else:
        for r in seqs:
            assert_close(got[r], refs[r], dtype, (r, json.dumps(raw)))
        assert_close(whole, refs["a"], dtype, json.dumps(raw))
