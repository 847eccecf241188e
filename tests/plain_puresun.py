"""A plain, slow Puresun decoder on the CPU: one function per mechanism, float64 or float32,
whole sequences only, no cache. It shares no code with ``reinfer_amd`` and is what the engine is
compared with.

Notation: x is the residual stream [n, width]; W matrices are [out, in] and act as ``x @ W.T``.

* embedding: x_i = E[t_i] + B[r_i], r_0 = buckets (the table's last row),
  r_i = (t_{i-1} * mul_prev + t_i * mul_cur) mod buckets
* run order: layers start..stop-1 run ``times`` times with the same weights, then the rest; before
  pass number p > 0 the embedding output is added again, and before every pass S[p] is added
* layer: h = rms(x) * w_norm;  x <- x + (mixer(h) + ff(h))
* latent attention: q = W_q h, per head [dim | rot_dim]; (c_raw | kr) = W_dkv h; c = rms(c_raw) * w_c;
  per head k = W_uk c, v = W_uv c; rotation of the rot_dim parts (half-split pairs, angle p * base^(-2i/R));
  s_ij = scale * (q_i . k_j + qr_i . kr_j) for 0 <= i - j < window; softmax; heads concatenated,
  times sigmoid(W_g h), then W_o
* mixture of experts: z = W_r h; the ``top`` largest z; softmax over those; sum_e p_e W_down,e relu(W_up,e h)^2
* output: rms(x) * w_final, logits = W_head x, then cap * tanh(logits / cap)
"""
from __future__ import annotations

import math
from typing import Dict, List, Mapping, Optional, Sequence

import torch


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return rms_unit(x, eps) * w


def bigram_rows(tokens: Sequence[int], buckets: int, mul_prev: int, mul_cur: int) -> List[int]:
    rows = []
    for i, t in enumerate(tokens):
        rows.append(buckets if i == 0 else (tokens[i - 1] * mul_prev + t * mul_cur) % buckets)
    return rows


def embed(tokens: Sequence[int], table: torch.Tensor, bigram: Optional[torch.Tensor],
          bigram_cfg: Optional[Mapping]) -> torch.Tensor:
    x = table[torch.tensor(list(tokens), dtype=torch.long)]
    if bigram is not None:
        rows = bigram_rows(tokens, int(bigram_cfg["buckets"]), int(bigram_cfg["mul_prev"]), int(bigram_cfg["mul_cur"]))
        x = x + bigram[torch.tensor(rows, dtype=torch.long)]
    return x


def rotate_half_split(x: torch.Tensor, positions: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """x [n, ..., D]: the first ``dims`` entries of the last axis are turned, pair (i, i + dims/2)."""
    half = dims // 2
    i = torch.arange(half, dtype=torch.float64)
    freq = torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / dims).to(x.dtype)
    ang = positions.to(x.dtype)[:, None] * freq[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    c, s = torch.cos(ang).view(shape), torch.sin(ang).view(shape)
    u, v = x[..., :half], x[..., half:dims]
    out = x.clone()
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


def windowed_softmax_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                               window: int) -> torch.Tensor:
    """q, k [n, H, Dk], v [n, H, Dv] -> [n, H, Dv]; query i sees keys j with 0 <= i - j < window
    (window 0: every j <= i)."""
    n = q.shape[0]
    s = torch.einsum("ihd,jhd->hij", q, k) * scale
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    seen = (j <= i) if window <= 0 else ((j <= i) & (i - j < window))
    s = s.masked_fill(~seen[None], float("-inf"))
    p = torch.softmax(s, dim=-1)
    return torch.einsum("hij,jhd->ihd", p, v)


def latent_attention(h: torch.Tensor, w: Mapping[str, torch.Tensor], pre: str, m: Mapping, eps: float) -> torch.Tensor:
    n = h.shape[0]
    H, D, R, Dv, rank = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
    pos = torch.arange(n)
    q = (h @ w[pre + "q"].T).view(n, H, D + R)
    down = h @ w[pre + "dkv"].T
    c = rms_norm(down[:, :rank], w[pre + "dkv.norm"], eps)
    kr = down[:, rank:rank + R]
    k = (c @ w[pre + "uk"].T).view(n, H, D)
    v = (c @ w[pre + "uv"].T).view(n, H, Dv)
    base, dims = float(m["rot"]["base"]), int(m["rot"]["dims"])
    qr = rotate_half_split(q[:, :, D:], pos, base, dims)
    kr = rotate_half_split(kr[:, None, :], pos, base, dims).expand(n, H, R)
    qq = torch.cat([q[:, :, :D], qr], dim=-1)
    kk = torch.cat([k, kr], dim=-1)
    window = int((m.get("mask") or {}).get("size", 0))
    o = windowed_softmax_attention(qq, kk, v, float(m["scale"]), window).reshape(n, H * Dv)
    o = o * torch.sigmoid(h @ w[pre + "g"].T)
    return o @ w[pre + "o"].T


def route(h: torch.Tensor, router: torch.Tensor, top: int):
    """(chosen experts [n, top] in falling order of their logits, their weights [n, top])."""
    z = h @ router.T
    val, idx = torch.topk(z, top, dim=-1)
    return idx, torch.softmax(val, dim=-1)


def expert(h: torch.Tensor, up: torch.Tensor, down: torch.Tensor) -> torch.Tensor:
    return (torch.relu(h @ up.T) ** 2) @ down.T


def moe_feed_forward(h: torch.Tensor, w: Mapping[str, torch.Tensor], pre: str, f: Mapping) -> torch.Tensor:
    E, top = int(f["router"]["experts"]), int(f["router"]["top"])
    idx, p = route(h, w[pre + "router"], top)
    out = torch.zeros_like(h)
    for e in range(E):
        share = (p * (idx == e)).sum(dim=-1, keepdim=True)          # 0 where the token did not choose e
        rows = share[:, 0] > 0
        if rows.any():
            out[rows] += share[rows] * expert(h[rows], w[f"{pre}e{e}.up"], w[f"{pre}e{e}.down"])
    return out


def run_order(cfg: Mapping) -> List[tuple]:
    """[(layer, pass number or None, first of its pass)]"""
    n = len(cfg["layers"])
    loop = cfg.get("loop") or None
    if not loop:
        return [(i, 0 if i == 0 else None, i == 0) for i in range(n)]
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    out = [(i, None, False) for i in range(a)]
    for p in range(times):
        out += [(i, p, i == a) for i in range(a, b)]
    out += [(i, None, False) for i in range(b, n)]
    return out


def forward(cfg: Mapping, w: Mapping[str, torch.Tensor], tokens: Sequence[int], layers_out: Optional[list] = None,
            softcap: bool = True) -> torch.Tensor:
    """Logits [n, vocab] of a whole sequence; ``layers_out`` collects x behind every layer run."""
    eps = float(cfg["norm"]["eps"])
    big = (cfg.get("embedding") or {}).get("bigram")
    x = embed(tokens, w["embed"], w.get("bigram") if big else None, big)
    x0 = x.clone()
    loop = cfg.get("loop") or None
    for layer, p, first in run_order(cfg):
        if loop and first and p is not None:
            if p > 0:
                x = x + x0
            x = x + w["loop.step"][p]
        L = cfg["layers"][layer]
        pre = f"l{layer}."
        h = rms_norm(x, w[pre + "norm1"], eps)
        if L["type"] != "latent_attention":
            raise ValueError(L["type"])
        d = latent_attention(h, w, pre + "mix.", L["mixer"], eps)
        if L.get("mlp"):
            d = d + moe_feed_forward(h, w, pre + "mlp.", L["mlp"])
        x = x + d
        if layers_out is not None:
            layers_out.append(x.clone())
    y = rms_norm(x, w["final.norm"], eps) @ w["head"].T
    cap = cfg.get("logit_softcap")
    if softcap and cap:
        y = float(cap) * torch.tanh(y / float(cap))
    return y


def greedy_generate(cfg: Mapping, w: Mapping[str, torch.Tensor], prompt: Sequence[int], n_new: int) -> List[int]:
    """The first maximum of the last position's logits, n_new times, the whole sequence recomputed each time."""
    toks, out = list(prompt), []
    for _ in range(n_new):
        t = int(torch.argmax(forward(cfg, w, toks)[-1]))
        out.append(t)
        toks.append(t)
    return out
