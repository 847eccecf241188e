"""Kobolix configurations drawn at random (sizes, head counts, layer order, every optional section present or
absent), each run through the engine against the plain implementation: a whole prompt, portions beside single
tokens of other requests, and decoding, on a cache and state slots that are given back and taken again. In float32
as drawn; in bfloat16 with every router choosing all its experts (which of two nearly equal scores is the larger
after rounding is decided differently by any two implementations) and the bound position by position."""
import json
import os
import random

import pytest
import torch

import plain_kobolix as plain
from helpers import random_tokens, rel_err, run_plan
from kobolix_helpers import draw_weights, read_folder
from test_kobolix_engine import assert_close
from reinfer_amd.engine import ModelRunner
from reinfer_amd.weights.safetensors_io import write_safetensors

pytestmark = pytest.mark.gpu


def draw_config(rng: random.Random) -> dict:
    width = rng.choice([24, 40, 64, 72, 128])

    def memory():
        m = {"dim": rng.choice([4, 12, 33, 64, 150, 260]), "heads": rng.choice([1, 2, 3, 5]), "vdim": rng.choice([3, 8, 20, 70])}
        if rng.random() < 0.8:
            m["gate_cap"] = rng.choice([5.0, 10.0, 30.0])
        return m

    def pair():
        kv = rng.choice([1, 2, 3])
        dim = rng.choice([8, 24, 32, 80])
        left = {"dim": dim, "heads": kv * rng.choice([1, 2, 4]), "kv_heads": kv, "vdim": rng.choice([8, 16, 40, 96])}
        if rng.random() < 0.8:
            left["rot"] = {"base": rng.choice([100.0, 10000.0, 1e6]), "dims": rng.choice([2, dim // 2 // 2 * 2, dim])}
        if rng.random() < 0.7:
            left["scale"] = rng.choice([0.1, 0.25, 0.5])
        kh = rng.choice([1, 2, 3])
        right = {"conv": rng.choice([1, 2, 3, 4, 6]), "dim": rng.choice([6, 16, 40, 136]), "heads": kh * rng.choice([1, 2, 3]),
                 "kv_heads": kh, "vdim": rng.choice([4, 12, 32, 50])}
        return {"left": left, "right": right}

    def mlp():
        kind = rng.choice(["dense", "moe", "moe", None])
        if kind is None:
            return None
        if kind == "dense":
            return {"ff": rng.choice([16, 40, 100]), "kind": "dense"}
        groups = rng.choice([1, 2, 3, 5])
        per = rng.choice([1, 2, 4])
        keep = rng.randint(1, groups)
        router = {"experts": groups * per, "top": rng.randint(1, keep * per)}
        if groups > 1 or rng.random() < 0.5:
            router["groups"] = {"count": groups, "keep": keep}
        if rng.random() < 0.7:
            router["scale"] = rng.choice([0.5, 1.0, 2.5])
        out = {"expert": {"ff": rng.choice([8, 20, 48])}, "kind": "moe", "router": router}
        if rng.random() < 0.6:
            out["shared"] = {"ff": rng.choice([8, 36])}
        return out

    layers = []
    for _ in range(rng.randint(2, 4)):
        if rng.random() < 0.5:
            layers.append({"type": "mlstm", "mixer": memory(), "mlp": mlp()})
        else:
            layers.append({"type": "parallel", "mixer": pair(), "mlp": mlp()})
    raw = {"architecture": "Kobolix", "vocab": rng.choice([50, 131, 400]), "width": width,
           "norm": {"eps": rng.choice([1e-6, 1e-5])}, "layers": layers}
    if rng.random() < 0.8:
        raw["residual_mult"] = rng.choice([0.2, 0.5, 1.0, 1.5])
    if rng.random() < 0.8:
        raw["embedding"] = {"scale": rng.choice([1.0, 3.0, 10.0])}
    return raw


@pytest.mark.parametrize("seed,dtype", [(s, "float32") for s in range(20)] + [(s, "bfloat16") for s in range(20, 30)])
def test_random_configuration(tmp_path, seed, dtype):
    rng = random.Random(1000 + seed)
    raw = draw_config(rng)
    if dtype == "bfloat16":
        for L in raw["layers"]:
            if L["mlp"] is not None and L["mlp"]["kind"] == "moe":
                router = L["mlp"]["router"]
                router["top"] = router["experts"]
                if "groups" in router:
                    router["groups"]["keep"] = router["groups"]["count"]
    folder = str(tmp_path / "m")
    os.makedirs(folder)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(raw, f)
    write_safetensors(os.path.join(folder, "model.safetensors"), draw_weights(raw, seed, torch.bfloat16 if dtype == "bfloat16" else torch.float32), metadata={"format": "pt"})
    raw, w = read_folder(folder)
    V = raw["vocab"]
    lens = {"a": rng.randint(60, 140), "b": rng.randint(20, 70), "c": rng.randint(5, 40), "d": rng.randint(2, 30),
            "e": rng.randint(30, 90)}
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
            c = 1 if left[r] <= 6 else min(left[r] - 6, rng.choice([1, 2, 3, 7, 16, 17, 33, 64]))
            items.append((r, c))
            left[r] -= c
            if left[r] == 0:
                live.remove(r)
        if items:
            plan.append(items)
    runner = ModelRunner.from_folder(folder, dtype=dtype, device="cuda:0", max_tokens=4 * 192, max_seqs=4)
    runner.poison_freed_blocks()
    got = run_plan(runner, seqs, plan)
    whole = run_plan(runner, {"a": seqs["a"]}, [[("a", lens["a"])]])["a"]
    if dtype == "float32":
        for r in seqs:
            assert rel_err(got[r], refs[r]) < 3e-5, (r, json.dumps(raw))
        assert rel_err(whole, refs["a"]) < 3e-5, json.dumps(raw)
    else:
        for r in seqs:
            assert_close(got[r], refs[r], dtype, (r, json.dumps(raw)))
        assert_close(whole, refs["a"], dtype, json.dumps(raw))
