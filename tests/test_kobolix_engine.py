"""Kobolix through the engine against the plain implementation: configuration, whole prompts, prompts against
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

import plain_kobolix as plain
from helpers import random_tokens, rel_err, run_plan
from kernel_double import KernelDouble
from kobolix_helpers import CONFIGS, KB_A, make_folder, read_folder
from reinfer_amd import LLMEngine, SamplingParams, kernels
from reinfer_amd.config import ConfigError, KobolixConfig, config_from_dict
from reinfer_amd.engine import ModelRunner

# float32: both sides add a few hundred float or double terms in another order over four layers, and a recurrent
# state carries its rounding on for as long as its gates keep it: 2e-5 of the largest logit leaves a margin of
# five over what was seen. bfloat16: one rounding is 2^-9; about a dozen storage roundings a layer, in quadrature
# over three layers: 1.3e-2 of the stream; 5e-2 is more than three deviations.
TOL = {"float32": 2e-5, "bfloat16": 5e-2}


def assert_close(got, ref, dtype, what):
    """float32: no logit further from the reference than the bound (of the largest logit). bfloat16: the same bound
    position by position, but one position in fifty (at least one) may exceed it, by up to five times: the matrix
    memory divides by |n . q|, a sum with cancellation, and where that sum of bfloat16-rounded q and k comes out
    near zero the rounding is amplified at that one position, in every way of cutting and batching alike (the
    engine's own results for whole prompts and token by token agree to 1e-7 there). A lost key or state moves
    many positions, or one by far more."""
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
        assert isinstance(cfg, KobolixConfig)
        assert config_from_dict(cfg.to_dict()) == cfg, which
        assert cfg.to_dict()["layers"] == config_from_dict(json.loads(json.dumps(cfg.to_dict()))).to_dict()["layers"]
    spec = config_from_dict(KB_A).to_spec()
    assert [b.mixer.kind for b in spec.blocks] == ["side_by_side", "matrix_memory", "matrix_memory", "side_by_side"]
    assert spec.blocks[2].ffn is None and spec.blocks[2].ffn_norm is None
    assert spec.tie_embeddings and spec.embed_scale == 4.0 and spec.final_norm.offset == 1.0
    assert all(b.residual_scale == 0.5 for b in spec.blocks)
    left, right = (m for _, m in spec.blocks[0].mixer.params.members)
    assert (left.head_dim, left.value_dim, left.position.rotary_dim, left.position.kind) == (24, 16, 12, "rope_interleaved")
    assert (right.params.key_heads, right.params.conv_taps) == (1, 3)
    moe = spec.blocks[0].ffn.params
    assert (moe.groups, moe.groups_kept, moe.top, moe.shared, moe.weight_scale) == (4, 2, 2, 40, 1.5)
    assert spec.blocks[3].ffn.params.groups == 1 and spec.blocks[3].ffn.params.shared == 0


def test_configuration_errors_name_the_key():
    def broken(path, value):
        raw = json.loads(json.dumps(KB_A))
        node = raw
        for k in path[:-1]:
            node = node[k]
        if value is None:
            del node[path[-1]]
        else:
            node[path[-1]] = value
        return raw
    for path, value, key in ((["width"], None, "width"), (["norm", "eps"], None, "norm.eps"),
                             (["layers", 1, "mixer", "gate_cap"], -2.0, "layers[1].mixer.gate_cap"),
                             (["layers", 1, "mixer", "vdim"], None, "layers[1].mixer.vdim"),
                             (["layers", 1, "type"], "conv", "layers[1].type"),
                             (["layers", 0, "mixer", "left", "kv_heads"], 3, "layers[0].mixer.left.kv_heads"),
                             (["layers", 0, "mixer", "left", "rot", "dims"], 26, "layers[0].mixer.left.rot.dims"),
                             (["layers", 0, "mixer", "right", "conv"], 0, "layers[0].mixer.right.conv"),
                             (["layers", 0, "mlp", "router", "top"], 5, "layers[0].mlp.router.top"),
                             (["layers", 0, "mlp", "router", "groups", "count"], 3, "layers[0].mlp.router.groups.count"),
                             (["layers", 1, "mlp", "kind"], "glu", "layers[1].mlp.kind")):
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
    again; freed blocks are filled with NaN and every state slot starts out as NaN, so that a read outside a
    request's own, or a state that is not cleared at a request's start, shows."""
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
    for top in runner.caches:
        for c in (top.flat() if top is not None else ()):
            if c.state is not None:
                c.state.fill_(float("nan"))
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
SHARP = {"left.q": 8.0}                                   # softmax rests on one or two keys, many of them far back
LONG_MEMORY = {"f.b": 5.0}                                # forget gates near 1: the state lasts
LONG_BOTH = {"f.b": 5.0, "A_log": -4.0}                   # the delta rule's decay near 1 as well


def test_a_far_key_and_a_lost_state_move_the_logits(tmp_path_factory):
    """That the sharp and the long-memory tests can see what they are for, in the plain implementation alone:
    with sharp queries, other tokens in the first 40 places change the logits of the last 200 by several times
    the wider bound; with long memories, a state that starts afresh 50 tokens before the end (what a lost or
    cleared state slot would do at a cut) changes the last 20."""
    tmp = tmp_path_factory.getbasetemp()
    raw, w = read_folder(make_folder(tmp, "A", "float32", scales=SHARP, tag="_sharp"))
    toks = random_tokens(300, vocab("A"), 77)
    full = plain.forward(raw, w, toks)
    other = plain.forward(raw, w, random_tokens(40, vocab("A"), 5) + toks[40:])
    assert rel_err(other[-200:].float(), full[-200:].float()) > 3 * TOL["bfloat16"]
    raw, w = read_folder(make_folder(tmp, "B", "float32", shifts=LONG_MEMORY, tag="_long"))
    toks = random_tokens(300, vocab("B"), 78)
    a, b = plain.forward(raw, w, toks), plain.forward(raw, w, toks[-50:])         # no layer of B knows positions
    assert rel_err(a[-20:].float(), b[-20:].float()) > 4 * TOL["bfloat16"]


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


# ------------------------------------------------------------------ GPU: the real kernels
GPU_CASES = [("A", "float32"), ("B", "float32"), ("C", "float32"), ("D", "float32"), ("C", "bfloat16"), ("B", "bfloat16"),
             ("D", "bfloat16")]


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
    ("B", "float32", None, LONG_MEMORY, "_long"), ("C", "float32", SHARP, LONG_BOTH, "_both")])
def test_sharp_attention_and_long_memory_gpu(tmp_path_factory, which, dtype, scales, shifts, tag):
    check_sharp_and_long(tmp_path_factory.getbasetemp(), which, "cuda:0", dtype, scales, shifts, tag)


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
    src.write_text(json.dumps(KB_A))
    out = tmp_path / "model"
    assert cli.main(["init", str(src), "--seed", "3", "--out", str(out), "--dtype", "float32"]) == 0
    raw, w = read_folder(str(out))
    assert raw["architecture"] == "Kobolix" and raw["layers"][2]["mlp"] is None
    assert {"embed", "l0.norm1", "l0.mix.left.q", "l0.mix.right.q.conv", "l0.mix.right.A_log", "l0.mix.left.out",
            "l0.mlp.e7.gate", "l0.mlp.shared.down", "l0.mlp.router", "l1.mix.i.b", "l1.mlp.down", "l3.mlp.e5.up",
            "final.norm"} <= set(w)
    assert "l2.norm2" not in w and "head" not in w and "l3.mlp.shared.up" not in w
    assert w["l0.mix.left.v"].shape == (32, 64) and w["l0.mix.right.q.conv"].shape == (20, 3)
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
