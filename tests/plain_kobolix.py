"""Kobolix, slowly and plainly: one function per mechanism, a loop over tokens wherever the design has a
recurrence, double precision on the CPU. It shares no code with the package; the engine is compared with it.

Notation. h: a layer's normed input row; x: the residual stream. Weights are [out, in]. A model is
(raw config dict, name -> tensor).

  norm_offset(x, w)   x / sqrt(mean x^2 + eps) * (1 + w)
  mlstm               matrix memory with exponential gates and a running maximum, token by token
  rotate_pairs        (x[2i], x[2i+1]) turned by p * base^(-2i/dims), first `dims` entries of a head
  attention           causal softmax attention, grouped heads, value size of its own
  short_conv          causal per-channel filter over time, zeros before the start
  delta_rule          S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q
  side_by_side        half the sum of two mixers, each RMS-normed over the width with a plain weight
  dense_ff, moe_ff    gated feed-forwards; sigmoid router restricted to the best groups of experts
"""
from __future__ import annotations

import math
from typing import Dict, List, Sequence

import torch

D = torch.float64


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def norm_offset(x, w, eps):
    return rms(x, eps) * (1.0 + w)


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def logsigmoid(z):
    return -softplus(-z)


# ------------------------------------------------------------------ matrix memory (mLSTM)
def mlstm(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, cfg: dict, eps: float) -> torch.Tensor:
    """h [T, width] -> [T, width]. State per head: S [dim, vdim], n [dim], m (scalar, starts at 0)."""
    H, dk, dv, cap = cfg["heads"], cfg["dim"], cfg["vdim"], cfg.get("gate_cap")
    T = h.shape[0]
    q = (h @ w[p + "q"].T).view(T, H, dk) * dk ** -0.5
    k = (h @ w[p + "k"].T).view(T, H, dk)
    v = (h @ w[p + "v"].T).view(T, H, dv)
    soft = (lambda z: float(cap) * torch.tanh(z / float(cap))) if cap else (lambda z: z)      # no cap given: none
    gi = soft(h @ w[p + "i"].T + w[p + "i.b"])                                         # [T, H] log input gate
    gf = logsigmoid(soft(h @ w[p + "f"].T + w[p + "f.b"]))                             # [T, H] log forget gate
    out = torch.zeros(T, H, dv, dtype=D)
    for a in range(H):
        S = torch.zeros(dk, dv, dtype=D)
        n = torch.zeros(dk, dtype=D)
        m = 0.0
        for t in range(T):
            m_new = max(float(gf[t, a]) + m, float(gi[t, a]))
            keep = math.exp(float(gf[t, a]) + m - m_new)
            take = math.exp(float(gi[t, a]) - m_new)
            S = keep * S + take * torch.outer(k[t, a], v[t, a])
            n = keep * n + take * k[t, a]
            m = m_new
            den = max(abs(float(n @ q[t, a])), math.exp(-m)) + 1e-6
            out[t, a] = (S.T @ q[t, a]) / den
    o = rms(out, eps).reshape(T, H * dv) * w[p + "norm"]
    o = o * torch.sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


# ------------------------------------------------------------------ attention
def rotate_pairs(x: torch.Tensor, pos: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """x [T, heads, d]; entries 2i and 2i+1 (i < dims/2) are a pair turned by pos * base^(-2i/dims)."""
    if dims == 0:
        return x
    out = x.clone()
    i = torch.arange(dims // 2, dtype=D)
    ang = pos.to(D)[:, None] * base ** (-2.0 * i / dims)[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    a, b = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = a * c - b * s
    out[..., 1:dims:2] = b * c + a * s
    return out


def attention(h, w, p, cfg) -> torch.Tensor:
    H, G, dk, dv = cfg["heads"], cfg["kv_heads"], cfg["dim"], cfg["vdim"]
    T = h.shape[0]
    pos = torch.arange(T)
    rot = cfg.get("rot") or {"dims": 0, "base": 1.0}
    q = rotate_pairs((h @ w[p + "q"].T).view(T, H, dk), pos, rot["dims"], rot["base"])
    k = rotate_pairs((h @ w[p + "k"].T).view(T, G, dk), pos, rot["dims"], rot["base"])
    v = (h @ w[p + "v"].T).view(T, G, dv)
    out = torch.zeros(T, H, dv, dtype=D)
    for a in range(H):
        g = a // (H // G)
        s = (q[:, a] @ k[:, g].T) * cfg.get("scale", dk ** -0.5)
        s = s.masked_fill(torch.triu(torch.ones(T, T, dtype=torch.bool), 1), float("-inf"))
        out[:, a] = torch.softmax(s, dim=-1) @ v[:, g]
    return out.reshape(T, H * dv) @ w[p + "o"].T


# ------------------------------------------------------------------ gated delta rule
def short_conv(x: torch.Tensor, f: torch.Tensor) -> torch.Tensor:
    """x [T, C], f [C, taps]; y[t] = sum_j f[:, j] * x[t - (taps - 1) + j], zeros before the start."""
    T, C = x.shape
    taps = f.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, C, dtype=x.dtype), x], dim=0)
    y = torch.zeros_like(x)
    for j in range(taps):
        y = y + pad[j:j + T] * f[:, j][None, :]
    return y


def delta_rule(h, w, p, cfg, eps) -> torch.Tensor:
    H, G, dk, dv = cfg["heads"], cfg["kv_heads"], cfg["dim"], cfg["vdim"]
    T = h.shape[0]
    q = silu(short_conv(h @ w[p + "q"].T, w[p + "q.conv"])).view(T, G, dk)
    k = silu(short_conv(h @ w[p + "k"].T, w[p + "k.conv"])).view(T, G, dk)
    v = silu(short_conv(h @ w[p + "v"].T, w[p + "v.conv"])).view(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dk ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w[p + "b"].T)                                                   # [T, H]
    decay = torch.exp(-torch.exp(w[p + "A_log"]) * softplus(h @ w[p + "a"].T + w[p + "dt_bias"]))   # [T, H]
    out = torch.zeros(T, H, dv, dtype=D)
    for a in range(H):
        g = a // (H // G)
        S = torch.zeros(dk, dv, dtype=D)
        for t in range(T):
            S = decay[t, a] * S
            u = beta[t, a] * (v[t, a] - S.T @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            out[t, a] = S.T @ q[t, g]
    o = rms(out, eps) * w[p + "norm"]
    o = o.reshape(T, H * dv) * silu(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


def side_by_side(h, w, p, cfg, eps) -> torch.Tensor:
    left = attention(h, w, p + "left.", cfg["left"])
    right = delta_rule(h, w, p + "right.", cfg["right"], eps)
    return 0.5 * (rms(left, eps) * w[p + "left.out"] + rms(right, eps) * w[p + "right.out"])


# ------------------------------------------------------------------ feed-forwards
def dense_ff(h, w, p) -> torch.Tensor:
    return (silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def route(scores: torch.Tensor, top: int, groups: int, keep: int) -> List[List[int]]:
    """The chosen experts of every row of ``scores`` [T, E]: the ``top`` largest among the experts of the
    ``keep`` groups (of ``groups`` equal runs of neighbours) whose two largest scores sum highest."""
    T, E = scores.shape
    size = E // groups
    out = []
    for t in range(T):
        s = scores[t].tolist()
        gs = []
        for g in range(groups):
            part = sorted(s[g * size:(g + 1) * size], reverse=True)
            gs.append(sum(part[:2]))
        best = sorted(range(groups), key=lambda g: (-gs[g], g))[:keep]
        allowed = [e for e in range(E) if e // size in best]
        out.append(sorted(allowed, key=lambda e: (-s[e], e))[:top])
    return out


def moe_ff(h, w, p, cfg) -> torch.Tensor:
    r = cfg["router"]
    groups = r.get("groups") or {"count": 1, "keep": 1}
    s = torch.sigmoid(h @ w[p + "router"].T)
    chosen = route(s, r["top"], groups["count"], groups["keep"])
    y = torch.zeros(h.shape[0], w[p + "e0.down"].shape[0], dtype=D)
    for t, es in enumerate(chosen):
        for e in es:
            y[t] += float(s[t, e]) * float(r.get("scale", 1.0)) * dense_ff(h[t:t + 1], w, f"{p}e{e}.")[0]
    if cfg.get("shared") is not None:
        y = y + dense_ff(h, w, p + "shared.")
    return y


# ------------------------------------------------------------------ the model
def layer(x, w, i: int, L: dict, eps: float, mult: float) -> torch.Tensor:
    p = f"l{i}."
    h = norm_offset(x, w[p + "norm1"], eps)
    if L["type"] == "mlstm":
        y = mlstm(h, w, p + "mix.", L["mixer"], eps)
    elif L["type"] == "parallel":
        y = side_by_side(h, w, p + "mix.", L["mixer"], eps)
    else:
        raise ValueError(L["type"])
    x = x + mult * y
    if L.get("mlp") is not None:
        h = norm_offset(x, w[p + "norm2"], eps)
        y = dense_ff(h, w, p + "mlp.") if L["mlp"]["kind"] == "dense" else moe_ff(h, w, p + "mlp.", L["mlp"])
        x = x + mult * y
    return x


def forward(raw: dict, w: Dict[str, torch.Tensor], tokens: Sequence[int], layers_out: list = None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence from its start; ``layers_out`` collects the stream behind every layer."""
    w = {k: v.to(D) for k, v in w.items()}
    eps = float(raw["norm"]["eps"])
    mult = float(raw.get("residual_mult", 1.0))
    x = w["embed"][torch.tensor(list(tokens))] * float((raw.get("embedding") or {}).get("scale", 1.0))
    for i, L in enumerate(raw["layers"]):
        x = layer(x, w, i, L, eps, mult)
        if layers_out is not None:
            layers_out.append(x.clone())
    return norm_offset(x, w["final.norm"], eps) @ w["embed"].T


def greedy_generate(raw, w, prompt: Sequence[int], n: int) -> List[int]:
    toks, out = list(prompt), []
    for _ in range(n):
        row = forward(raw, w, toks)[-1]
        t = int(torch.nonzero(row == row.max())[0])
        out.append(t)
        toks.append(t)
    return out
