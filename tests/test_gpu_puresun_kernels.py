"""The kernels behind Puresun's mechanisms, each against a plain float32 PyTorch computation of the same
operation: the hashed token-pair rows with their per-request state word, the stream add, the logit cap, the
latent norm / rotation / cache write, the products head by head, the router and the routed activation."""
import math
from types import SimpleNamespace

import pytest
import torch

from kernel_double import k_index, v_index
from reinfer_amd import kernels

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def ops():
    k = kernels.current()
    assert k.name == "hip-gfx950"
    return k


def i32(x):
    return torch.tensor(x, dtype=torch.int32, device=DEV)


def close(got, want, dtype):
    tol = 1e-5 if dtype == torch.float32 else 1.2e-2
    got, want = got.float().cpu(), want.float().cpu()
    assert torch.isfinite(got).all()
    assert float((got - want).abs().max()) <= tol * max(1.0, float(want.abs().max())), float((got - want).abs().max())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_pair_hash_add_and_its_state(dtype):
    g = torch.Generator().manual_seed(1)
    buckets, mp, mc, h = 53, 40009, 70001, 40          # products beyond 32 bits with ids near 60000
    table = torch.randn(buckets + 1, h, generator=g).to(dtype).to(DEV)
    state = i32([111, 222, 333, 444])
    # three requests: slot 2 continues (position 5, previous token from its state word), slot 0 starts, a padding row
    ids = [59999, 3, 58000, 7, 9]
    batch = SimpleNamespace(num_tokens=5, num_seqs=3, token_ids=i32(ids), positions=i32([5, 6, 0, 1, 0]),
                            seq_of_token=i32([0, 0, 1, 1, 2]), cu_tokens=i32([0, 2, 4, 5]),
                            state_slots=i32([2, 0, -1]))
    resid = torch.randn(5, h, generator=g).to(DEV)
    want = resid.clone().cpu()
    rows = [(333 * mp + 59999 * mc) % buckets, (59999 * mp + 3 * mc) % buckets, buckets, (58000 * mp + 7 * mc) % buckets,
            buckets]
    want += table.float().cpu()[rows]
    ops().pair_hash_add(resid, table, batch, state, buckets, mp, mc)
    close(resid, want, torch.float32)
    assert state.tolist() == [7, 222, 3, 444]           # each portion's last token; the padding row wrote nothing


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_stream_add_and_cap(dtype):
    g = torch.Generator().manual_seed(2)
    T, h = 7, 100
    resid = torch.randn(T, h, generator=g).to(DEV)
    delta = torch.randn(T, h, generator=g).to(dtype).to(DEV)
    other = torch.randn(T, h, generator=g).to(DEV)
    vec = torch.randn(h, generator=g).to(dtype).to(DEV)
    for d, o, v in ((delta, other, vec), (None, other, vec), (delta, None, None), (None, None, vec)):
        x = resid.clone()
        want = x.clone()
        for t in (d, o, v):
            if t is not None:
                want = want + t.float()
        ops().stream_add(x, d, o, v)
        close(x, want, torch.float32)
    logits = (torch.randn(3, 301, generator=g) * 40).to(DEV)
    want = 25.0 * torch.tanh(logits / 25.0)
    ops().tanh_cap(logits, 25.0)
    close(logits, want, torch.float32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,D,R,rot,rank", [(3, 16, 8, 8, 40), (2, 8, 16, 8, 24), (5, 24, 6, 6, 100), (1, 64, 32, 32, 96)])
def test_latent_prep(dtype, H, D, R, rot, rank):
    g = torch.Generator().manual_seed(3)
    T, bs, blocks, eps = 9, 16, 4, 1e-5
    Dp = -(-(rank + R) // 16) * 16
    q_off, dkv_off = 0, H * (D + R)
    width = dkv_off + rank + R + 5
    proj = torch.randn(T, width, generator=g).to(dtype).to(DEV)
    cw = (torch.rand(rank, generator=g) + 0.5).to(dtype).to(DEV)
    pos = i32([0, 1, 2, 17, 100, 3000, 5, 6, 7])
    slots = i32([0, 1, 15, 16, 33, -1, 63, 47, 20])
    inv = torch.pow(torch.tensor(10000.0, dtype=torch.float64), -2.0 * torch.arange(rot // 2, dtype=torch.float64) / rot) \
        .float().to(DEV)
    kc = torch.full((blocks, 1, bs // 16, 16 * Dp), float("nan"), dtype=dtype, device=DEV)
    vc = kc.clone()
    q_lat = torch.full((T, H, Dp), float("nan"), dtype=dtype, device=DEV)
    ops().latent_prep(proj, q_off, dkv_off, cw, eps, pos, inv, rot, R, rank, H, D, q_lat, slots, kc, vc)

    p = proj.float().cpu()
    ang = pos.cpu().float()[:, None] * inv.cpu()[None, :]
    c, s = torch.cos(ang), torch.sin(ang)

    def turn(x):                        # [T, R]
        y = x.clone()
        half = rot // 2
        y[:, :half] = x[:, :half] * c - x[:, half:rot] * s
        y[:, half:rot] = x[:, half:rot] * c + x[:, :half] * s
        return y
    craw = p[:, dkv_off:dkv_off + rank]
    row = torch.zeros(T, Dp)
    row[:, :rank] = craw / torch.sqrt((craw * craw).mean(-1, keepdim=True) + eps) * cw.float().cpu()
    row[:, rank:rank + R] = turn(p[:, dkv_off + rank:dkv_off + rank + R])
    e = torch.arange(Dp)
    kflat, vflat = kc.float().cpu().view(blocks, -1), vc.float().cpu().view(blocks, -1)
    for t in range(T):
        sl = int(slots[t])
        if sl < 0:
            continue
        close(kflat[sl // bs][k_index(sl % bs, e, Dp)], row[t], dtype)
        close(vflat[sl // bs][v_index(sl % bs, e, Dp)], row[t], dtype)
    written = sorted(int(x) for x in slots.tolist() if x >= 0)
    untouched = [x for x in range(blocks * bs) if x not in written]
    assert all(torch.isnan(kflat[x // bs][k_index(x % bs, e, Dp)]).all() for x in untouched)
    ql = q_lat.float().cpu()
    assert torch.isnan(ql[:, :, :rank]).all()                    # the head products' columns are not touched
    for a in range(H):
        want = torch.zeros(T, Dp - rank)
        want[:, :R] = turn(p[:, q_off + a * (D + R) + D:q_off + (a + 1) * (D + R)])
        close(ql[:, a, rank:], want, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,H,K,N,pad", [(1, 3, 16, 40, 7), (17, 2, 24, 8, 8), (70, 5, 100, 4, 7), (33, 1, 96, 300, 0),
                                         (16, 3, 40, 24, 8), (130, 2, 64, 50, 16), (5, 18, 128, 192, 64)])
def test_head_linear(dtype, T, H, K, N, pad):
    """Odd sizes and strides (the plain kernel) and sizes in steps of 8 (matrix cores in bfloat16): token
    counts on both sides of the tiles of 16 and 64, column counts that end inside a tile."""
    g = torch.Generator().manual_seed(4)
    x_head, o_head = K + pad, N + 3
    lead = 5 if pad == 7 else 8
    x = torch.randn(T, lead + H * x_head, generator=g).to(dtype).to(DEV)
    w = (torch.randn(H, N, K, generator=g) / math.sqrt(K)).to(dtype).to(DEV)
    gate = torch.randn(T, H * N + 2, generator=g).to(dtype).to(DEV)
    for use_gate in (False, True):
        out = torch.full((T, H * o_head), float("nan"), dtype=dtype, device=DEV)
        ops().head_linear(x[:, lead:], x_head, w, out, o_head, gate=gate if use_gate else None)
        got = out.float().cpu().view(T, H, o_head)
        assert torch.isnan(got[:, :, N:]).all()
        xs = x.float().cpu()[:, lead:].view(T, H, x_head)[:, :, :K]
        want = torch.einsum("thk,hnk->thn", xs, w.float().cpu())
        if use_gate:
            want = want * torch.sigmoid(gate.float().cpu()[:, :H * N].view(T, H, N))
        close(got[:, :, :N], want, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("E,top,width", [(8, 2, 48), (5, 5, 36), (1, 1, 64), (70, 6, 200)])
def test_moe_route(dtype, E, top, width):
    g = torch.Generator().manual_seed(5)
    T = 19
    x = torch.randn(T, width + 8, generator=g).to(dtype).to(DEV)[:, :width]
    router = torch.randn(E, width, generator=g).to(dtype).to(DEV)
    ids = torch.full((T, top), -1, dtype=torch.int32, device=DEV)
    wts = torch.full((T, top), float("nan"), dtype=torch.float32, device=DEV)
    ops().moe_route(x, router, top, ids, wts)
    z = x.float().cpu().double() @ router.float().cpu().double().T
    val, idx = torch.topk(z, top, dim=-1)
    assert ids.cpu().tolist() == idx.tolist()
    close(wts, torch.softmax(val, dim=-1), torch.float32)
    # equal logits: the lower expert first, equal weights
    same = router[:1].repeat(E, 1).contiguous()
    ops().moe_route(x, same, top, ids, wts)
    assert ids.cpu().tolist() == [list(range(top))] * T
    close(wts, torch.full((T, top), 1.0 / top), torch.float32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("ff", [20, 24])
def test_moe_relu2_scale(dtype, ff):
    g = torch.Generator().manual_seed(6)
    T, E, top = 11, 6, 3
    up = torch.randn(T, E * ff, generator=g).to(dtype).to(DEV)
    ids = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(T)]).to(torch.int32).to(DEV)
    wts = torch.rand(T, top, generator=g).to(DEV)
    act = torch.full((T, E * ff), float("nan"), dtype=dtype, device=DEV)
    ops().moe_relu2_scale(up, act, ids, wts, E, ff)
    gate = torch.zeros(T, E)
    gate.scatter_(1, ids.cpu().long(), wts.cpu())
    u = torch.relu(up.float().cpu()).view(T, E, ff)
    close(act, (gate[:, :, None] * u * u).view(T, E * ff), dtype)
    assert (act.float().cpu().view(T, E, ff)[gate == 0] == 0).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,E,top,ff,width", [(1, 6, 2, 24, 48), (2, 9, 3, 20, 36), (3, 16, 1, 64, 128), (1, 5, 5, 8, 200)])
def test_moe_chosen_experts(dtype, T, E, top, ff, width):
    """Only the chosen experts' rows: against all experts computed plainly and weighted, into the stream and
    into a result of its own; sizes in steps of 8 (16-byte reads) and not."""
    g = torch.Generator().manual_seed(7)
    x = torch.randn(T, width, generator=g).to(dtype).to(DEV)
    w_up = (torch.randn(E * ff, width, generator=g) / math.sqrt(width)).to(dtype).to(DEV)
    w_down = (torch.randn(width, E * ff, generator=g) / math.sqrt(ff)).to(dtype).to(DEV)
    ids = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(T)]).to(torch.int32).to(DEV)
    wts = torch.rand(T, top, generator=g).to(DEV)
    act = torch.full((T * top, ff), float("nan"), dtype=dtype, device=DEV)
    ops().moe_up_chosen(x, w_up, ids, wts, act, ff)
    xf, uf, df = x.float().cpu(), w_up.float().cpu().view(E, ff, width), w_down.float().cpu().view(width, E, ff)
    want_act = torch.stack([float(wts[t, j]) * torch.relu(uf[int(ids[t, j])] @ xf[t]) ** 2
                            for t in range(T) for j in range(top)])
    close(act, want_act, dtype)
    a = act.float().cpu().view(T, top, ff)
    want = torch.stack([sum(df[:, int(ids[t, j])] @ a[t, j] for j in range(top)) for t in range(T)])
    out = torch.full((T, width), float("nan"), dtype=dtype, device=DEV)
    ops().moe_down_chosen(act, w_down, ids, ff, out=out)
    close(out, want, dtype)
    resid = torch.randn(T, width, generator=g).to(DEV)
    base = resid.clone().cpu()
    ops().moe_down_chosen(act, w_down, ids, ff, resid=resid)
    close(resid, base + want, torch.float32 if dtype == torch.float32 else dtype)
