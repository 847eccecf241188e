"""The plain implementation of Kobolix, pinned mechanism by mechanism: by numbers worked out by hand, by closed
forms of one or two tokens written out here from the equations, and by cases that reduce to something simpler.
Each is chosen so that a plausible misreading fails it (the running maximum starting at minus infinity, the
read-out before the write, pairs (i, i + d/2) instead of (2i, 2i + 1), a filter applied back to front, a group
scored by its best expert alone, weights renormalised)."""
import math

import torch

import plain_kobolix as plain

D = torch.float64


def rnd(*shape, seed=0, std=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=D) * std


def test_norm_with_a_weight_around_zero():
    x = torch.tensor([[3.0, 4.0]], dtype=D)
    out = plain.norm_offset(x, torch.tensor([0.0, 1.0], dtype=D), 0.0)
    r = math.sqrt(12.5)
    assert torch.allclose(out, torch.tensor([[3 / r, 2 * 4 / r]], dtype=D))
    # eps inside the root
    assert torch.allclose(plain.rms(torch.zeros(1, 2, dtype=D) + 1e-3, 1.0), torch.full((1, 2), 1e-3 / math.sqrt(1e-6 + 1.0), dtype=D))


def test_pairs_of_neighbours_are_turned():
    x = torch.tensor([[[1.0, 2.0, 3.0, 4.0, 5.0, 6.0]]], dtype=D).repeat(2, 1, 1)       # two positions, one head
    out = plain.rotate_pairs(x, torch.tensor([0, 3]), 4, 100.0)
    assert torch.equal(out[0], x[0])                                                    # position 0: unchanged
    a0, a1 = 3 * 1.0, 3 * 100.0 ** -0.5                                                 # f_i = base^(-2i/dims)
    want = [1 * math.cos(a0) - 2 * math.sin(a0), 2 * math.cos(a0) + 1 * math.sin(a0),
            3 * math.cos(a1) - 4 * math.sin(a1), 4 * math.cos(a1) + 3 * math.sin(a1), 5.0, 6.0]
    assert torch.allclose(out[1, 0], torch.tensor(want, dtype=D))


def test_attention_groups_value_size_and_scale():
    H, G, dk, dv, width, T = 4, 2, 6, 3, 5, 7
    cfg = {"heads": H, "kv_heads": G, "dim": dk, "vdim": dv, "scale": 0.37, "rot": {"dims": 4, "base": 50.0}}
    w = {"q": rnd(H * dk, width, seed=1), "k": rnd(G * dk, width, seed=2), "v": rnd(G * dv, width, seed=3),
         "o": torch.eye(H * dv, dtype=D)}
    h = rnd(T, width, seed=4)
    out = plain.attention(h, w, "", cfg).view(T, H, dv)
    # the first token sees itself alone: its output is its own value, of the KV head floor(head / (H / G))
    v = (h @ w["v"].T).view(T, G, dv)
    for a in range(H):
        assert torch.allclose(out[0, a], v[0, a // 2])
    # token 2, head 3, by hand from the definition
    pos = torch.arange(T)
    q = plain.rotate_pairs((h @ w["q"].T).view(T, H, dk), pos, 4, 50.0)
    k = plain.rotate_pairs((h @ w["k"].T).view(T, G, dk), pos, 4, 50.0)
    s = torch.tensor([float(q[2, 3] @ k[j, 1]) * 0.37 for j in range(3)], dtype=D)
    p = torch.exp(s - s.max()) / torch.exp(s - s.max()).sum()
    assert torch.allclose(out[2, 3], p @ v[:3, 1])


def _memory_weights(H, dk, dv, width, seed):
    return {"q": rnd(H * dk, width, seed=seed), "k": rnd(H * dk, width, seed=seed + 1), "v": rnd(H * dv, width, seed=seed + 2),
            "g": rnd(H * dv, width, seed=seed + 3), "o": torch.eye(H * dv, dtype=D), "norm": torch.ones(H * dv, dtype=D),
            "i": rnd(H, width, seed=seed + 4), "i.b": rnd(H, seed=seed + 5), "f": rnd(H, width, seed=seed + 6),
            "f.b": rnd(H, seed=seed + 7)}


def test_matrix_memory_first_two_tokens_in_closed_form():
    H, dk, dv, width, cap, eps = 2, 3, 4, 5, 2.5, 1e-5
    cfg = {"heads": H, "dim": dk, "vdim": dv, "gate_cap": cap}
    w = _memory_weights(H, dk, dv, width, 10)
    h = rnd(2, width, seed=20)
    got = plain.mlstm(h, w, "", cfg, eps).view(2, H, dv)
    gate = torch.sigmoid(h @ w["g"].T).view(2, H, dv)
    for a in range(H):
        q = [(w["q"][a * dk:(a + 1) * dk] @ h[t]) / math.sqrt(dk) for t in range(2)]
        k = [w["k"][a * dk:(a + 1) * dk] @ h[t] for t in range(2)]
        v = [w["v"][a * dv:(a + 1) * dv] @ h[t] for t in range(2)]
        gi = [cap * math.tanh(float(w["i"][a] @ h[t] + w["i.b"][a]) / cap) for t in range(2)]
        zf = [cap * math.tanh(float(w["f"][a] @ h[t] + w["f.b"][a]) / cap) for t in range(2)]
        gf = [-math.log1p(math.exp(-z)) for z in zf]
        # token 0: the maximum before it is 0, not minus infinity
        m0 = max(gf[0] + 0.0, gi[0])
        c0 = math.exp(gi[0] - m0)
        o0 = c0 * float(k[0] @ q[0]) * v[0] / (max(abs(c0 * float(k[0] @ q[0])), math.exp(-m0)) + 1e-6)
        # token 1
        m1 = max(gf[1] + m0, gi[1])
        d1, c1 = math.exp(gf[1] + m0 - m1), math.exp(gi[1] - m1)
        num = d1 * c0 * float(k[0] @ q[1]) * v[0] + c1 * float(k[1] @ q[1]) * v[1]
        nq = d1 * c0 * float(k[0] @ q[1]) + c1 * float(k[1] @ q[1])
        o1 = num / (max(abs(nq), math.exp(-m1)) + 1e-6)
        for t, o in ((0, o0), (1, o1)):
            want = o / torch.sqrt((o * o).mean() + eps) * gate[t, a]
            assert torch.allclose(got[t, a], want, rtol=1e-10, atol=1e-12), (a, t)


def test_matrix_memory_gates_are_capped():
    # pre-activations far beyond the cap give the same result as at +-infinity of tanh: cap and -cap
    H, dk, dv, width = 1, 2, 2, 3
    cfg = {"heads": H, "dim": dk, "vdim": dv, "gate_cap": 1.5}
    w = _memory_weights(H, dk, dv, width, 30)
    h = rnd(4, width, seed=31)
    w["i.b"], w["f.b"] = torch.tensor([400.0], dtype=D), torch.tensor([-300.0], dtype=D)
    a = plain.mlstm(h, w, "", cfg, 1e-6)
    w["i.b"], w["f.b"] = torch.tensor([4000.0], dtype=D), torch.tensor([-3000.0], dtype=D)
    assert torch.allclose(a, plain.mlstm(h, w, "", cfg, 1e-6))
    assert torch.isfinite(a).all()


def test_filter_runs_forward_in_time_with_zeros_before_the_start():
    x = torch.tensor([[1.0, 10.0], [2.0, 20.0], [3.0, 30.0]], dtype=D)
    f = torch.tensor([[0.5, 0.0, 2.0], [1.0, 1.0, 1.0]], dtype=D)          # last column: the current token's
    y = plain.short_conv(x, f)
    assert torch.allclose(y, torch.tensor([[2.0, 10.0], [4.0, 30.0], [6.5, 60.0]], dtype=D))


def test_delta_rule_reads_after_it_writes():
    H, G, dk, dv, width, eps = 2, 1, 3, 2, 4, 1e-5
    cfg = {"heads": H, "kv_heads": G, "dim": dk, "vdim": dv, "conv": 2}
    w = {"q": rnd(G * dk, width, seed=40), "k": rnd(G * dk, width, seed=41), "v": rnd(H * dv, width, seed=42),
         "q.conv": rnd(G * dk, 2, seed=43), "k.conv": rnd(G * dk, 2, seed=44), "v.conv": rnd(H * dv, 2, seed=45),
         "b": rnd(H, width, seed=46), "a": rnd(H, width, seed=47), "A_log": rnd(H, seed=48), "dt_bias": rnd(H, seed=49),
         "norm": torch.tensor([1.0, 2.0], dtype=D), "g": rnd(H * dv, width, seed=50), "o": torch.eye(H * dv, dtype=D)}
    h = rnd(2, width, seed=51)
    got = plain.delta_rule(h, w, "", cfg, eps).view(2, H, dv)
    silu = lambda z: z / (1 + torch.exp(-z))
    unit = lambda z: z / torch.sqrt((z * z).sum() + 1e-6)
    x = {n: h @ w[n].T for n in ("q", "k", "v")}
    y = {n: [silu(w[n + ".conv"][:, 1] * x[n][0]), silu(w[n + ".conv"][:, 0] * x[n][0] + w[n + ".conv"][:, 1] * x[n][1])]
         for n in ("q", "k", "v")}
    for a in range(H):
        q = [unit(y["q"][t]) / math.sqrt(dk) for t in range(2)]
        k = [unit(y["k"][t]) for t in range(2)]
        v = [y["v"][t][a * dv:(a + 1) * dv] for t in range(2)]
        beta = [float(torch.sigmoid(w["b"][a] @ h[t])) for t in range(2)]
        g = [math.exp(-math.exp(float(w["A_log"][a])) * math.log1p(math.exp(float(w["a"][a] @ h[t] + w["dt_bias"][a]))))
             for t in range(2)]
        # token 0: S = k0 u0^T with u0 = beta0 v0 (the state was zero); the read-out sees it
        u0 = beta[0] * v[0]
        o0 = float(k[0] @ q[0]) * u0
        # token 1: the old state decays, is corrected along k1, and is read
        S = g[1] * torch.outer(k[0], u0)
        u1 = beta[1] * (v[1] - S.T @ k[1])
        o1 = (S + torch.outer(k[1], u1)).T @ q[1]
        gate = [silu(w["g"][a * dv:(a + 1) * dv] @ h[t]) for t in range(2)]
        for t, o in ((0, o0), (1, o1)):
            want = o / torch.sqrt((o * o).mean() + eps) * w["norm"] * gate[t]
            assert torch.allclose(got[t, a], want, rtol=1e-10, atol=1e-12), (a, t)


def test_side_by_side_is_half_the_sum_of_two_normed_outputs(monkeypatch):
    left, right = rnd(3, 4, seed=60), rnd(3, 4, seed=61) * 5
    monkeypatch.setattr(plain, "attention", lambda *a: left)
    monkeypatch.setattr(plain, "delta_rule", lambda *a: right)
    w = {"left.out": torch.tensor([1.0, 2.0, 3.0, 4.0], dtype=D), "right.out": torch.tensor([0.5, 0.5, 0.5, 0.5], dtype=D)}
    got = plain.side_by_side(None, w, "", {"left": {}, "right": {}}, 0.0)
    unit = lambda z: z / torch.sqrt((z * z).mean(-1, keepdim=True))
    assert torch.allclose(got, 0.5 * (unit(left) * w["left.out"] + unit(right) * w["right.out"]))


def test_router_groups_by_hand():
    #            group 0          group 1          group 2
    s = torch.tensor([[0.98, 0.01, 0.02, 0.60, 0.55, 0.50, 0.58, 0.57, 0.10]], dtype=D)
    # sums of the two largest: 0.99 (or 1.00), 1.15, 1.15 -> with one group kept the tie goes to the lower group
    assert plain.route(s, 2, 3, 1) == [[3, 4]]
    assert plain.route(s, 3, 3, 2) == [[3, 6, 7]]                 # groups 1 and 2: the best expert of all is out
    assert plain.route(s, 2, 3, 3) == [[0, 3]]
    assert plain.route(s, 2, 1, 1) == [[0, 3]]


def test_expert_weights_are_scores_times_a_constant_and_the_shared_expert_is_added():
    width, ff, E = 4, 3, 4
    w = {"router": rnd(E, width, seed=70)}
    for i, e in enumerate(list(range(E)) + ["s"]):
        p = "shared." if e == "s" else f"e{e}."
        w[p + "gate"], w[p + "up"], w[p + "down"] = rnd(ff, width, seed=100 + i), rnd(ff, width, seed=200 + i), \
            rnd(width, ff, seed=300 + i)
    cfg = {"router": {"experts": E, "top": 2, "scale": 2.5, "groups": {"count": 2, "keep": 1}}, "shared": {"ff": ff}}
    h = rnd(1, width, seed=72)
    s = torch.sigmoid(h @ w["router"].T)[0]
    groups = [float(s[0] + s[1]), float(s[2] + s[3])]
    pick = [0, 1] if groups[0] >= groups[1] else [2, 3]
    want = sum(2.5 * float(s[e]) * plain.dense_ff(h, w, f"e{e}.") for e in pick) + plain.dense_ff(h, w, "shared.")
    assert torch.allclose(plain.moe_ff(h, w, "", cfg), want)
    assert abs(sum(2.5 * float(s[e]) for e in pick) - 1.0) > 1e-3          # not renormalised


def test_layer_and_model_factors():
    """x <- x + m mixer(norm1 x), then x + m ff(norm2 x); the embedding is scaled on its way in only."""
    raw = {"vocab": 7, "width": 4, "norm": {"eps": 1e-6}, "residual_mult": 0.25, "embedding": {"scale": 3.0},
           "layers": [{"type": "mlstm", "mixer": {"heads": 1, "dim": 2, "vdim": 2, "gate_cap": 5.0},
                       "mlp": {"kind": "dense", "ff": 3}}]}
    w = {"embed": rnd(7, 4, seed=80), "l0.norm1": rnd(4, seed=81, std=0.1), "l0.norm2": rnd(4, seed=82, std=0.1),
         "final.norm": rnd(4, seed=83, std=0.1), "l0.mlp.gate": rnd(3, 4, seed=84), "l0.mlp.up": rnd(3, 4, seed=85),
         "l0.mlp.down": rnd(4, 3, seed=86)}
    for n, t in _memory_weights(1, 2, 2, 4, 87).items():
        w["l0.mix." + n] = t
    w["l0.mix.o"] = rnd(4, 2, seed=99)
    toks = [3, 1, 6]
    x = w["embed"][torch.tensor(toks)] * 3.0
    x = x + 0.25 * plain.mlstm(plain.norm_offset(x, w["l0.norm1"], 1e-6), w, "l0.mix.", raw["layers"][0]["mixer"], 1e-6)
    x = x + 0.25 * plain.dense_ff(plain.norm_offset(x, w["l0.norm2"], 1e-6), w, "l0.mlp.")
    want = plain.norm_offset(x, w["final.norm"], 1e-6) @ w["embed"].T
    assert torch.allclose(plain.forward(raw, w, toks), want)
