"""The plain Puresun implementation pinned by numbers worked out by hand, by special cases and by
identities, each chosen so that a plausible misreading fails it."""
import math

import pytest
import torch

import plain_puresun as plain
from puresun_helpers import CONFIGS, PS_A, PS_B, PS_C, draw_weights

torch.manual_seed(0)


def test_pair_rows_by_hand():
    # (prev * 13 + cur * 5) mod 97, the first token takes row 97
    assert plain.bigram_rows([4, 9, 0, 96, 96], 97, 13, 5) == [97, (4 * 13 + 9 * 5) % 97, (9 * 13) % 97,
                                                               (96 * 5) % 97, (96 * 18) % 97]
    assert plain.bigram_rows([7], 3, 1, 1) == [3]
    # the previous token is multiplied by mul_prev, not the current one
    assert plain.bigram_rows([1, 0], 1000, 10, 3) == [1000, 10]


def test_run_order_by_hand():
    assert [(l, p) for l, p, f in plain.run_order(PS_A)] == [(0, None), (1, 0), (2, 0), (1, 1), (2, 1), (1, 2), (2, 2)]
    assert [f for _, _, f in plain.run_order(PS_A)] == [False, True, False, True, False, True, False]
    assert [(l, p) for l, p, f in plain.run_order(PS_C)] == [(0, 0), (0, 1), (1, None)]
    assert [l for l, _, _ in plain.run_order(PS_B)] == [0, 1]


def test_rms_norm_by_hand():
    x = torch.tensor([[3.0, 4.0]], dtype=torch.float64)
    # mean of squares 12.5; eps inside the root
    want = x / math.sqrt(12.5 + 0.5) * torch.tensor([2.0, 1.0], dtype=torch.float64)
    assert torch.allclose(plain.rms_norm(x, torch.tensor([2.0, 1.0], dtype=torch.float64), 0.5), want)


def test_rotation_by_hand():
    # dims 4 of 6: pairs (0, 2) and (1, 3); entries 4, 5 pass; frequencies 1 and base^(-1/2)
    x = torch.tensor([[[1.0, 2.0, 3.0, 4.0, 5.0, 6.0]]], dtype=torch.float64).repeat(3, 1, 1)
    y = plain.rotate_half_split(x, torch.tensor([0, 1, 7]), 100.0, 4)
    assert torch.equal(y[0], x[0])                                      # position 0 turns nothing
    for p, row in ((1, y[1, 0]), (7, y[2, 0])):
        a0, a1 = p * 1.0, p * 0.1
        want = [1 * math.cos(a0) - 3 * math.sin(a0), 2 * math.cos(a1) - 4 * math.sin(a1),
                3 * math.cos(a0) + 1 * math.sin(a0), 4 * math.cos(a1) + 2 * math.sin(a1), 5.0, 6.0]
        assert torch.allclose(row, torch.tensor(want, dtype=torch.float64), atol=1e-12)
    # a turn keeps the length, and q.k depends on the distance of the positions only
    q, k = torch.randn(1, 1, 8, dtype=torch.float64), torch.randn(1, 1, 8, dtype=torch.float64)
    def dot(pq, pk):
        return float((plain.rotate_half_split(q, torch.tensor([pq]), 50.0, 8) *
                      plain.rotate_half_split(k, torch.tensor([pk]), 50.0, 8)).sum())
    assert abs(dot(9, 4) - dot(105, 100)) < 1e-9 and abs(dot(9, 4) - dot(9, 5)) > 1e-6


def test_window_by_hand():
    """Values are one-hot in the position, equal scores: the output is the uniform average over the keys
    seen, which shows exactly which they are: i - window < j <= i."""
    n, W = 7, 3
    q = torch.zeros(n, 1, 2, dtype=torch.float64)
    k = torch.zeros(n, 1, 2, dtype=torch.float64)
    v = torch.eye(n, dtype=torch.float64)[:, None, :]
    o = plain.windowed_softmax_attention(q, k, v, 1.0, W)[:, 0]
    for i in range(n):
        seen = [j for j in range(n) if 0 <= i - j < W]
        want = torch.zeros(n, dtype=torch.float64)
        want[seen] = 1.0 / len(seen)
        assert torch.allclose(o[i], want), i
    full = plain.windowed_softmax_attention(q, k, v, 1.0, 0)[:, 0]
    assert torch.allclose(full[5], torch.tensor([1 / 6] * 6 + [0.0], dtype=torch.float64))


def test_routing_by_hand():
    h = torch.eye(4, dtype=torch.float64)[:2]                        # token 0 reads column 0 of the router, ...
    router = torch.tensor([[1.0, 0.0], [3.0, 5.0], [2.0, 5.5], [-1.0, 9.0]], dtype=torch.float64)
    router = torch.cat([router, torch.zeros(4, 2, dtype=torch.float64)], dim=1)
    idx, p = plain.route(h, router, 2)
    assert idx.tolist() == [[1, 2], [3, 2]]
    e = math.exp(-1.0)
    assert torch.allclose(p[0], torch.tensor([1 / (1 + e), e / (1 + e)], dtype=torch.float64))   # over the chosen only
    e = math.exp(-3.5)
    assert torch.allclose(p[1], torch.tensor([1 / (1 + e), e / (1 + e)], dtype=torch.float64))


def test_expert_by_hand():
    h = torch.tensor([[1.0, -2.0]], dtype=torch.float64)
    up = torch.tensor([[1.0, 0.0], [0.0, 1.0], [2.0, 0.5]], dtype=torch.float64)       # pre-activations 1, -2, 1
    down = torch.tensor([[1.0, 10.0, 100.0]], dtype=torch.float64)
    assert plain.expert(h, up, down).tolist() == [[1.0 + 0.0 + 100.0]]                # relu squared


def test_moe_is_the_weighted_sum_of_the_chosen():
    raw, seed = CONFIGS["A"]
    w = draw_weights(raw, seed, torch.float64)
    f = raw["layers"][0]["mlp"]
    h = torch.randn(6, raw["width"], dtype=torch.float64)
    got = plain.moe_feed_forward(h, w, "l0.mlp.", f)
    idx, p = plain.route(h, w["l0.mlp.router"], f["router"]["top"])
    for t in range(6):
        want = sum(p[t, j] * plain.expert(h[t:t + 1], w[f"l0.mlp.e{int(idx[t, j])}.up"], w[f"l0.mlp.e{int(idx[t, j])}.down"])
                   for j in range(idx.shape[1]))
        assert torch.allclose(got[t], want[0], atol=1e-12)
    assert abs(float(p.sum(-1)[0]) - 1.0) < 1e-12


def test_latent_attention_through_the_cached_rows():
    """The same mixer computed the way an engine can that caches only the latent and the rotated key part:
    queries taken through the key matrices, one shared row a token for keys and values, results through the
    value matrices."""
    raw, seed = CONFIGS["A"]
    w = draw_weights(raw, seed, torch.float64)
    m = raw["layers"][0]["mixer"]
    n = 40
    h = torch.randn(n, raw["width"], dtype=torch.float64)
    want = plain.latent_attention(h, w, "l0.mix.", m, raw["norm"]["eps"])
    H, D, R, Dv, rank, W = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["mask"]["size"]
    pos = torch.arange(n)
    q = (h @ w["l0.mix.q"].T).view(n, H, D + R)
    down = h @ w["l0.mix.dkv"].T
    c = plain.rms_norm(down[:, :rank], w["l0.mix.dkv.norm"], raw["norm"]["eps"])
    kr = plain.rotate_half_split(down[:, None, rank:], pos, m["rot"]["base"], m["rot"]["dims"])[:, 0]
    qr = plain.rotate_half_split(q[:, :, D:], pos, m["rot"]["base"], m["rot"]["dims"])
    uk = w["l0.mix.uk"].view(H, D, rank)
    uv = w["l0.mix.uv"].view(H, Dv, rank)
    out = torch.zeros(n, H, Dv, dtype=torch.float64)
    for i in range(n):
        lo = max(0, i - W + 1)
        for a in range(H):
            qa = uk[a].T @ q[i, a, :D]
            s = (c[lo:i + 1] @ qa + kr[lo:i + 1] @ qr[i, a]) * m["scale"]
            p = torch.softmax(s, dim=0)
            out[i, a] = uv[a] @ (p @ c[lo:i + 1])
    got = (out.reshape(n, H * Dv) * torch.sigmoid(h @ w["l0.mix.g"].T)) @ w["l0.mix.o"].T
    assert torch.allclose(got, want, atol=1e-10)


def test_a_layer_in_closed_form():
    """Output projection and expert down projections zero: the model is embedding (+ pair rows, + the
    vectors and the embedding again before the passes), norm, head, cap."""
    raw, seed = CONFIGS["C"]
    w = draw_weights(raw, seed, torch.float64)
    for name in list(w):
        if name.endswith(".mix.o") or name.endswith(".down"):
            w[name] = torch.zeros_like(w[name])
    toks = [5, 9, 9, 130]
    got = plain.forward(raw, w, toks)
    rows = plain.bigram_rows(toks, 31, 3, 11)
    e = w["embed"][toks] + w["bigram"][rows]
    x = e + w["loop.step"][0] + e + w["loop.step"][1]
    y = plain.rms_norm(x, w["final.norm"], raw["norm"]["eps"]) @ w["head"].T
    assert torch.allclose(got, 7.5 * torch.tanh(y / 7.5), atol=1e-12)


def test_layers_out_has_one_entry_per_layer_run():
    raw, seed = CONFIGS["A"]
    w = draw_weights(raw, seed, torch.float64)
    seen = []
    plain.forward(raw, w, [1, 2, 3], seen)
    assert len(seen) == 7 and all(s.shape == (3, raw["width"]) for s in seen)
