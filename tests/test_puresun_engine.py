"""Puresun through the engine against the plain implementation: configuration, whole prompts, prompts
against token-by-token decoding, portions down to two tokens, unequal requests in one batch with blocks and
state slots that are given back and used again, keys at the edges of windows and blocks, the first tokens,
long decoding, sharp attention that makes one key stand out, and greedy generation through the entry point
and the scheduler. Without a GPU the engine's bookkeeping runs on the CPU stand-in for the kernels (float32);
the ``gpu`` tests run the same checks on the real kernels in float32 and bfloat16.

bfloat16 runs use the configuration whose feed-forwards choose all their experts: which of two nearly equal
router logits is the larger after rounding is decided differently by any two implementations, and the choice
itself is checked in float32 and in the kernel tests."""
import json
import os

import pytest
import torch

import plain_puresun as plain
from helpers import random_tokens, rel_err, run_plan
from kernel_double import KernelDouble
from puresun_helpers import CONFIGS, PS_A, make_folder, read_folder
from reinfer_amd import LLMEngine, SamplingParams, kernels
from reinfer_amd.config import ConfigError, PuresunConfig, config_from_dict
from reinfer_amd.engine import ModelRunner, StepEntry

# float32: both sides add a few hundred float or double terms in another order, over at most seven layer
# runs: 2e-5 of the largest logit leaves a margin of ten. bfloat16: one rounding is 2^-9; about ten storage
# roundings a layer run, in quadrature over seven runs: 1.6e-2 of the stream; 5e-2 is three deviations.
TOL = {"float32": 2e-5, "bfloat16": 5e-2}


# ------------------------------------------------------------------ configuration
def test_configuration_round_trip_and_spec():
    for which, (raw, _) in CONFIGS.items():
        cfg = config_from_dict(raw)
        assert isinstance(cfg, PuresunConfig)
        assert config_from_dict(cfg.to_dict()) == cfg, which
    spec = config_from_dict(PS_A).to_spec()
    assert [e.block for e in spec.run_order] == [0, 1, 2, 1, 2, 1, 2]
    before = [(e.before.embedding, e.before.row) if e.before else None for e in spec.run_order]
    assert before == [None, (False, 0), None, (True, 1), None, (True, 2), None]
    assert spec.blocks[1].ffn is None and spec.blocks[0].ffn.params.top == 2
    assert spec.blocks[1].mixer.position.rotary_dim == 8 and spec.blocks[1].mixer.params.rot_width == 16
    assert spec.logit_softcap == 20.0 and spec.inputs[0].params.buckets == 97


def test_configuration_errors_name_the_key():
    def broken(path, value):
        raw = json.loads(json.dumps(PS_A))
        node = raw
        for k in path[:-1]:
            node = node[k]
        if value is None:
            del node[path[-1]]
        else:
            node[path[-1]] = value
        return raw
    for path, value, key in ((["width"], None, "width"), (["norm", "eps"], None, "norm.eps"),
                             (["layers", 0, "mixer", "kv_rank"], None, "layers[0].mixer.kv_rank"),
                             (["layers", 1, "type"], "conv", "layers[1].type"),
                             (["layers", 0, "mlp", "router", "top"], 9, "layers[0].mlp.router.top"),
                             (["loop", "stop"], 7, "loop"),
                             (["embedding", "bigram", "buckets"], 0, "embedding.bigram.buckets")):
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
        assert rel_err(whole, ref) < TOL[dtype], (n, "whole")
        ones = run_plan(runner, {"r": toks}, [[("r", 1)]] * n)["r"]
        assert rel_err(ones, ref) < TOL[dtype], (n, "one by one")
    assert all(p.num_free == p.num_blocks for p in runner.manager.pools)


def check_portions(folder, which, device, dtype):
    runner = runner_for(folder, device, dtype, max_tokens=256)
    n = 131
    toks = random_tokens(n, vocab(which), 22)
    ref = reference(folder, toks)
    for cuts in ([7, 2, 16, 3, 2, 17, 2, 31, 2, 15, 1, 16, 2, 2, 13], [64, 2, 62, 1, 1, 1], [2] * 20 + [91],
                 [100] + [1] * 31):
        assert sum(cuts) == n
        got = run_plan(runner, {"r": toks}, [[("r", c)] for c in cuts])["r"]
        assert rel_err(got, ref) < TOL[dtype], cuts[:4]


def check_mixed_with_reuse(folder, which, device, dtype):
    """Six requests in a pool of 128 tokens and four state slots: blocks and slots go back and are taken
    again; freed blocks are filled with NaN so that a read outside a request's own shows."""
    runner = runner_for(folder, device, dtype, max_tokens=128, max_seqs=4)
    lens = {"a": 30, "b": 20, "c": 30, "d": 20, "e": 40, "f": 25}
    plan = [[("a", 9), ("b", 2)],
            [("a", 1), ("b", 17), ("c", 5)],
            [("a", 20), ("b", 1), ("c", 12), ("d", 17)],
            [("c", 13), ("d", 3), ("e", 3)],
            [("e", 36), ("f", 2)],
            [("e", 1), ("f", 23)]]
    seqs = {r: random_tokens(n, vocab(which), 300 + i) for i, (r, n) in enumerate(lens.items())}
    for c in runner.caches:
        if c is not None and c.k is not None:
            c.k.fill_(float("nan"))
            c.v.fill_(float("nan"))
    runner.poison_freed_blocks()
    got = run_plan(runner, seqs, plan)
    for r, toks in seqs.items():
        assert rel_err(got[r], reference(folder, toks)) < TOL[dtype], r
    for c in (c for c in runner.caches if c is not None):
        assert runner.manager.pools[c.group].num_free == runner.manager.pools[c.group].num_blocks
    # each request alone gives the same logits as in the batch, beyond rounding
    alone = run_plan(runner, {"c": seqs["c"]}, [[("c", 30)]])["c"]
    assert rel_err(alone, got["c"]) < TOL[dtype]


def check_long_decoding(folder, which, device, dtype):
    runner = runner_for(folder, device, dtype, max_tokens=256)
    n = 150
    toks = random_tokens(n, vocab(which), 23)
    got = run_plan(runner, {"r": toks}, [[("r", 3)]] + [[("r", 1)]] * (n - 3))["r"]
    assert rel_err(got, reference(folder, toks)) < TOL[dtype]


def check_greedy_generation(folder, which, device, dtype):
    raw, w = read_folder(folder)
    prompts = [random_tokens(n, vocab(which), 40 + n) for n in (5, 17, 33)]
    want = [plain.greedy_generate(raw, w, p, 12) for p in prompts]
    eng = LLMEngine(folder, dtype=dtype, device=device, num_blocks=32)
    outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12))
    assert [o.token_ids for o in outs] == want
    # portions of eight beside decoding requests, and so few blocks that requests wait or are recomputed
    small = LLMEngine(folder, dtype=dtype, device=device, num_blocks=8, max_num_batched_tokens=8,
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


def test_greedy_generation_cpu(tmp_path_factory):
    folder = make_folder(tmp_path_factory.getbasetemp(), "A", "float32")
    with kernels.use(KernelDouble()):
        check_greedy_generation(folder, "A", "cpu", "float32")


def test_previous_token_is_request_state_cpu(tmp_path_factory):
    """Two requests whose portions alternate: each portion's first token pairs with its own request's last
    token, not with the row before it in the batch, and a state slot that is taken again starts afresh."""
    folder = make_folder(tmp_path_factory.getbasetemp(), "C", "float32")
    with kernels.use(KernelDouble()):
        runner = runner_for(folder, "cpu", "float32", max_tokens=128, max_seqs=2)
        a, b, c = (random_tokens(n, vocab("C"), s) for n, s in ((12, 1), (9, 2), (6, 3)))
        plan = [[("a", 3), ("b", 1)], [("b", 4), ("a", 1)], [("a", 8), ("b", 4)], [("c", 6)]]
        got = run_plan(runner, {"a": a, "b": b, "c": c}, plan)
        for r, toks in (("a", a), ("b", b), ("c", c)):
            assert rel_err(got[r], reference(folder, toks)) < TOL["float32"], r


# ------------------------------------------------------------------ GPU: the real kernels
GPU_CASES = [("A", "float32"), ("B", "float32"), ("C", "float32"), ("A16", "bfloat16"), ("B", "bfloat16"),
             ("D", "float32"), ("D", "bfloat16")]


@pytest.mark.gpu
@pytest.mark.parametrize("check", CHECKS, ids=lambda f: f.__name__)
@pytest.mark.parametrize("which,dtype", GPU_CASES)
def test_engine_gpu(tmp_path_factory, check, which, dtype):
    assert kernels.current().name == "hip-gfx950"
    folder = make_folder(tmp_path_factory.getbasetemp(), which, dtype)
    check(folder, which, "cuda:0", dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("which,dtype", [("A", "float32"), ("C", "float32"), ("A16", "bfloat16")])
def test_sharp_attention_gpu(tmp_path_factory, which, dtype):
    """Query weights of every layer times six: the softmax of most queries rests on one or two keys, and for
    many of them those are the oldest the window still holds, or a key far back where there is no window. A
    window that is one key off, or a block-table walk that loses a far key, changes the logits by more than
    the bound. Whole, in portions that end inside windows and blocks, and one by one."""
    n_layers = len(CONFIGS[which][0]["layers"])
    folder = make_folder(tmp_path_factory.getbasetemp(), which, dtype,
                         scales={f"l{i}.mix.q": 6.0 for i in range(n_layers)}, tag="_sharp")
    runner = runner_for(folder, "cuda:0", dtype, max_tokens=512)
    n = 300
    toks = random_tokens(n, vocab(which), 77)
    ref = reference(folder, toks)
    for cuts in ([n], [150, 20, 1, 1, 13, 8, 9, 21, 15, 17, 45], [250] + [1] * 50):
        assert sum(cuts) == n
        got = run_plan(runner, {"r": toks}, [[("r", c)] for c in cuts])["r"]
        assert rel_err(got, ref) < TOL[dtype], cuts[:3]


def test_window_edge_moves_the_logits(tmp_path_factory):
    """That the sharp test can see a window that is one key off: the plain implementation with every window
    one key longer differs from itself by several times the wider of the two bounds."""
    n_layers = len(PS_A["layers"])
    folder = make_folder(tmp_path_factory.getbasetemp(), "A", "float32",
                         scales={f"l{i}.mix.q": 6.0 for i in range(n_layers)}, tag="_sharp")
    raw, w = read_folder(folder)
    toks = random_tokens(120, vocab("A"), 77)
    off = json.loads(json.dumps(raw))
    for L in off["layers"]:
        L["mixer"]["mask"]["size"] += 1
    assert rel_err(plain.forward(off, w, toks).float(), plain.forward(raw, w, toks).float()) > 4 * TOL["bfloat16"]


@pytest.mark.gpu
@pytest.mark.parametrize("which,dtype", [("A", "float32"), ("B", "bfloat16")])
def test_greedy_generation_gpu(tmp_path_factory, which, dtype):
    folder = make_folder(tmp_path_factory.getbasetemp(), which, "float32" if dtype == "float32" else "bfloat16")
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
    src.write_text(json.dumps(PS_A))
    out = tmp_path / "model"
    assert cli.main(["init", str(src), "--seed", "3", "--out", str(out), "--dtype", "float32"]) == 0
    raw, w = read_folder(str(out))
    assert raw["architecture"] == "Puresun" and raw["layers"][1]["mlp"] is None
    assert {"embed", "bigram", "loop.step", "l0.norm1", "l0.mix.dkv.norm", "l2.mlp.e2.down", "l0.mlp.router",
            "final.norm", "head"} <= set(w) and "l1.mlp.router" not in w
    assert w["loop.step"].shape == (3, 48) and w["bigram"].shape == (98, 48) and w["l1.mix.uk"].shape == (16, 24)
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
