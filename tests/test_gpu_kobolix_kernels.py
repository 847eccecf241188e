"""The kernels of the recurrent mixers, the grouped router and the scaled row kernels, each against a plain
PyTorch float32 form of the same operation (the CPU stand-in's, which has the same signature and shares no code
with the product): sizes on either side of every switch in the kernels (8 or 32 lanes a column, 2 to 16 elements a
lane, heads that do not fill a wave, columns that do not fill the last wave), several requests of unequal length
in one call, a second and third call that go on from the state the calls before left, a request that starts afresh
in a slot that was used, and padding rows (state slot -1) that must leave every state alone."""
from types import SimpleNamespace

import pytest
import torch

from kernel_double import KernelDouble
from reinfer_amd import kernels

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def make_batch(q_lens, slots, fresh, device):
    cu = [0]
    for q in q_lens:
        cu.append(cu[-1] + q)
    seq_of = [i for i, q in enumerate(q_lens) for _ in range(q)]
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=device)
    return SimpleNamespace(num_seqs=len(q_lens), num_tokens=cu[-1], cu_tokens=i32(cu), state_slots=i32(slots),
                           fresh=i32(fresh), seq_of_token=i32(seq_of), q_lens=list(q_lens))


# four calls: slots 2 and 0 start; they go on beside a padding row; slot 2 starts afresh beside slot 0 going on; both go
# on with portions of several staged chunks, the last of them part full
CALLS = [([5, 3], [2, 0], [1, 1]), ([1, 1, 4], [2, -1, 0], [0, 0, 0]), ([7, 2], [2, 0], [1, 0]), ([53, 1, 40], [0, 3, 2], [0, 1, 0])]


def close(got, ref, tol, what):
    got, ref = got.float().cpu(), ref.float().cpu()
    assert torch.isfinite(got).all(), what
    err = float((got - ref).abs().max() / ref.abs().max().clamp_min(1e-20))
    assert err < tol, (what, err)


@pytest.mark.parametrize("H,dk,dv", [(2, 40, 72), (3, 20, 28), (1, 136, 8), (2, 128, 40), (1, 8, 3), (2, 300, 17), (5, 12, 70), (2, 4, 20)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_matrix_memory_scan(H, dk, dv, dtype):
    ops, ref = kernels.current(), KernelDouble()
    g = torch.Generator().manual_seed(H * 1000 + dk)
    width = 2 * H * dk + H * dv + 5
    q_off, k_off, v_off = 3, 3 + H * dk, 3 + 2 * H * dk
    bias = torch.randn(2 * H, generator=g)
    st_gpu = torch.full((4, ops.scan_state_floats("matrix_memory", H, dk, dv)), float("nan"), device=DEV)
    st_ref = torch.full((4, ref.scan_state_floats("matrix_memory", H, dk, dv)), float("nan"))
    for n, (q_lens, slots, fresh) in enumerate(CALLS):
        T = sum(q_lens)
        proj = (torch.randn(T, width, generator=g) * 0.7).to(dtype)
        gates = torch.randn(T, 2 * H, generator=g) * 3.0
        out_ref = torch.empty(T, H * dv)
        ref.matrix_memory_scan(proj, q_off, k_off, v_off, gates.clone(), bias, st_ref, make_batch(q_lens, slots, fresh, "cpu"),
                               H, dk, dv, 6.0, dk ** -0.5, 1e-6, out_ref)
        out = torch.empty(T, H * dv, device=DEV)
        before = st_gpu.clone()
        ops.matrix_memory_scan(proj.to(DEV), q_off, k_off, v_off, gates.to(DEV), bias.to(DEV), st_gpu,
                               make_batch(q_lens, slots, fresh, DEV), H, dk, dv, 6.0, dk ** -0.5, 1e-6, out)
        close(out, out_ref, 2e-5, f"call {n}")
        untouched = [s for s in range(4) if s not in slots]
        assert torch.equal(torch.nan_to_num(st_gpu[untouched], nan=7.0), torch.nan_to_num(before[untouched], nan=7.0))


@pytest.mark.parametrize("H,G,dk,dv,taps", [(4, 2, 32, 48, 4), (4, 1, 20, 12, 3), (2, 2, 136, 8, 1), (1, 1, 16, 70, 2), (4, 2, 16, 50, 4),
                                            (6, 3, 130, 9, 5)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_delta_rule_prepare_and_scan(H, G, dk, dv, taps, dtype):
    ops, ref = kernels.current(), KernelDouble()
    g = torch.Generator().manual_seed(H * 1000 + dk + taps)
    C = 2 * G * dk + H * dv
    filt = torch.randn(C, taps, generator=g) * 0.6
    a_log, dt_bias = torch.randn(H, generator=g) * 0.5 - 1.0, torch.randn(H, generator=g) * 0.5
    off_gpu, off_ref = ops.scan_state_floats("delta_rule", H, dk, dv), ref.scan_state_floats("delta_rule", H, dk, dv)
    st_gpu = torch.full((4, off_gpu + (taps - 1) * C), float("nan"), device=DEV)
    st_ref = torch.full((4, off_ref + (taps - 1) * C), float("nan"))
    for n, (q_lens, slots, fresh) in enumerate(CALLS):
        T = sum(q_lens)
        proj = torch.randn(T, C + 7, generator=g).to(dtype)
        ba = torch.randn(T, 2 * H, generator=g) * 2.0
        qkv_ref, out_ref = torch.empty(T, C), torch.empty(T, H * dv)
        b_ref = make_batch(q_lens, slots, fresh, "cpu")
        ref.delta_rule_prepare(proj, filt, st_ref, off_ref, b_ref, G, dk, H, dv, taps, 1e-6, dk ** -0.5, qkv_ref)
        ref.delta_rule_scan(qkv_ref, ba.clone(), a_log, dt_bias, st_ref, b_ref, H, G, dk, dv, out_ref)
        qkv, out = torch.empty(T, C, device=DEV), torch.empty(T, H * dv, device=DEV)
        b_gpu = make_batch(q_lens, slots, fresh, DEV)
        ops.delta_rule_prepare(proj.to(DEV), filt.to(DEV), st_gpu, off_gpu, b_gpu, G, dk, H, dv, taps, 1e-6, dk ** -0.5, qkv)
        close(qkv, qkv_ref, 1e-5, f"prepare, call {n}")
        ops.delta_rule_scan(qkv, ba.to(DEV), a_log.to(DEV), dt_bias.to(DEV), st_gpu, b_gpu, H, G, dk, dv, out)
        close(out, out_ref, 3e-5, f"scan, call {n}")
        # the filter's tail is stored plainly: rows of the portion, oldest first
        live = [s for s in slots if s >= 0]
        close(st_gpu[live, off_gpu:], st_ref[live, off_ref:], 1e-6, f"tail, call {n}") if taps > 1 else None


@pytest.mark.parametrize("H,dv,per_head,kind", [(2, 64, True, "sigmoid"), (4, 12, False, "silu"), (1, 200, True, "silu")])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_head_norm_gate(H, dv, per_head, kind, dtype):
    ops, ref = kernels.current(), KernelDouble()
    g = torch.Generator().manual_seed(dv)
    T = 9
    read = torch.randn(T, H * dv, generator=g) * 3
    weight = torch.rand(H * dv if per_head else dv, generator=g) + 0.5
    wide = torch.randn(T, H * dv + 11, generator=g).to(dtype)
    out_ref = torch.empty(T, H * dv, dtype=dtype)
    ref.head_norm_gate(read, weight, per_head, wide[:, 11:], kind, 1e-5, H, dv, out_ref)
    out = torch.empty(T, H * dv, dtype=dtype, device=DEV)
    ops.head_norm_gate(read.to(DEV), weight.to(DEV), per_head, wide.to(DEV)[:, 11:], kind, 1e-5, H, dv, out)
    close(out, out_ref, 1e-5 if dtype == torch.float32 else 1e-2, "head_norm_gate")


@pytest.mark.parametrize("n,h", [(2, 256), (1, 36), (3, 1000)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_normed_mean(n, h, dtype):
    ops, ref = kernels.current(), KernelDouble()
    g = torch.Generator().manual_seed(h)
    T = 7
    xs = [(torch.randn(T, h, generator=g) * (i + 1)).to(dtype) for i in range(n)]
    ws = [torch.rand(h, generator=g) + 0.5 for _ in range(n)]
    out_ref = torch.empty(T, h, dtype=dtype)
    ref.normed_mean(xs, ws, 1e-6, out=out_ref)
    out = torch.empty(T, h, dtype=dtype, device=DEV)
    ops.normed_mean([x.to(DEV) for x in xs], [w.to(DEV) for w in ws], 1e-6, out=out)
    close(out, out_ref, 1e-5 if dtype == torch.float32 else 1e-2, "out")
    resid = torch.randn(T, h, generator=g)
    resid_ref = resid.clone()
    ref.normed_mean(xs, ws, 1e-6, resid=resid_ref, scale=0.6)
    resid_gpu = resid.to(DEV)
    ops.normed_mean([x.to(DEV) for x in xs], [w.to(DEV) for w in ws], 1e-6, resid=resid_gpu, scale=0.6)
    close(resid_gpu, resid_ref, 1e-5, "into the stream")


@pytest.mark.parametrize("E,top,groups,kept,group_top", [(15, 4, 5, 3, 2), (8, 2, 4, 2, 2), (6, 6, 1, 1, 2), (64, 8, 8, 4, 2),
                                                         (9, 2, 9, 3, 2), (130, 5, 2, 1, 3)])
def test_moe_route_sigmoid_groups(E, top, groups, kept, group_top):
    ops, ref = kernels.current(), KernelDouble()
    g = torch.Generator().manual_seed(E)
    T, width = 37, 24
    x, router = torch.randn(T, width, generator=g), torch.randn(E, width, generator=g) * 0.4
    ids_ref, w_ref = torch.empty(T, top, dtype=torch.int32), torch.empty(T, top)
    ref.moe_route(x, router, top, ids_ref, w_ref, scoring="sigmoid", scale=2.5, groups=groups, groups_kept=kept,
                  group_top=group_top)
    ids, w = torch.empty(T, top, dtype=torch.int32, device=DEV), torch.empty(T, top, device=DEV)
    ops.moe_route(x.to(DEV), router.to(DEV), top, ids, w, scoring="sigmoid", scale=2.5, groups=groups, groups_kept=kept,
                  group_top=group_top)
    assert torch.equal(ids.cpu(), ids_ref)
    close(w, w_ref, 1e-5, "weights")


def test_moe_route_restricts_to_the_best_groups():
    """Scores made by hand: the two largest scores lie in a group whose other members are small beside two groups
    of evenly high scores; with one group kept the choice must come from an evenly high group."""
    ops = kernels.current()
    z = torch.tensor([[4.0, -6.0, -6.0, 2.0, 2.1, 2.2, 1.9, 2.0, 1.8]], device=DEV)        # 3 groups of 3
    x, router = torch.eye(9, device=DEV)[:1] * 0 + 1.0, None
    # logits come from a product: make the router so that x . router^T = z
    x = torch.zeros(1, 9, device=DEV)
    x[0, 0] = 1.0
    router = torch.zeros(9, 9, device=DEV)
    router[:, 0] = z[0]
    ids, w = torch.empty(1, 2, dtype=torch.int32, device=DEV), torch.empty(1, 2, device=DEV)
    ops.moe_route(x, router, 2, ids, w, scoring="sigmoid", scale=1.0, groups=3, groups_kept=1, group_top=2)
    # group sums of the two largest sigmoids: g0 = s(4) + s(-6) = 0.98 + 0.002; g1 = s(2.2) + s(2.1) = 1.79; g2 = 1.76
    assert ids.cpu().tolist() == [[5, 4]]
    assert torch.allclose(w.cpu(), torch.sigmoid(torch.tensor([[2.2, 2.1]])), atol=1e-6)
    ops.moe_route(x, router, 2, ids, w, scoring="sigmoid", scale=1.0, groups=3, groups_kept=2, group_top=2)
    assert ids.cpu().tolist() == [[5, 4]]                 # groups 1 and 2 stay; expert 0 cannot be chosen
    ops.moe_route(x, router, 2, ids, w, scoring="sigmoid", scale=1.0, groups=3, groups_kept=3, group_top=2)
    assert ids.cpu().tolist() == [[0, 5]]


@pytest.mark.parametrize("E,ff,shared,top", [(10, 48, 72, 4), (5, 7, 0, 5), (3, 10, 3, 1)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_moe_silu_gate_scale(E, ff, shared, top, dtype):
    ops, ref = kernels.current(), KernelDouble()
    g = torch.Generator().manual_seed(ff)
    T = 11
    n = E * ff + shared
    gu = torch.randn(T, 2 * n, generator=g).to(dtype)
    ids = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(T)]).to(torch.int32)
    w = torch.rand(T, top, generator=g) + 0.1
    act_ref = torch.empty(T, n, dtype=dtype)
    ref.moe_silu_gate_scale(gu, act_ref, ids, w, E, ff, shared)
    act = torch.empty(T, n, dtype=dtype, device=DEV)
    ops.moe_silu_gate_scale(gu.to(DEV), act, ids.to(DEV), w.to(DEV), E, ff, shared)
    close(act, act_ref, 1e-5 if dtype == torch.float32 else 1e-2, "act")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_scaled_adds_and_embedding(dtype):
    ops, ref = kernels.current(), KernelDouble()
    g = torch.Generator().manual_seed(3)
    T, h = 13, 200
    resid, delta = torch.randn(T, h, generator=g), torch.randn(T, h, generator=g).to(dtype)
    weight = torch.rand(h, generator=g) + 0.5
    rows = torch.tensor([12, 0, 5], dtype=torch.int32)
    for r in (None, rows):
        a, b = resid.clone(), resid.clone().to(DEV)
        n = T if r is None else 3
        out_ref, out = torch.empty(n, h, dtype=dtype), torch.empty(n, h, dtype=dtype, device=DEV)
        ref.add_rmsnorm(a, delta, weight, 1e-6, out_ref, r, delta_scale=0.45)
        ops.add_rmsnorm(b, delta.to(DEV), weight.to(DEV), 1e-6, out, None if r is None else r.to(DEV), delta_scale=0.45)
        close(out, out_ref, 1e-5 if dtype == torch.float32 else 1e-2, "norm")
        close(b, a, 1e-6, "stream")
    a, b = resid.clone(), resid.clone().to(DEV)
    ref.stream_add(a, delta, delta_scale=-1.7)
    ops.stream_add(b, delta.to(DEV), delta_scale=-1.7)
    close(b, a, 1e-6, "stream_add")
    table = torch.randn(50, h, generator=g).to(dtype)
    ids = torch.randint(0, 50, (T,), generator=g).to(torch.int32)
    a, b = torch.empty(T, h), torch.empty(T, h, device=DEV)
    ref.embed(table, ids, a, scale=5.0)
    ops.embed(table.to(DEV), ids.to(DEV), b, scale=5.0)
    close(b, a, 1e-7, "embed")


@pytest.mark.parametrize("M", [1, 8, 16, 17, 33, 64, 65, 100, 128, 200, 2048])
@pytest.mark.parametrize("N,K", [(256, 128), (2048, 2048), (4096, 1024), (96, 144)])
def test_accumulating_product_with_a_factor(M, N, K):
    """out += alpha * (x . W^T) through whichever product takes the row count: both weight-streaming kernels, the
    one that cuts K into ranges, and the library's."""
    ops = kernels.current()
    g = torch.Generator().manual_seed(M + N)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16).to(DEV)
    w = (torch.randn(N, K, generator=g) * 0.05).to(torch.bfloat16).to(DEV)
    out = torch.randn(M, N, generator=g).to(DEV)
    if not ops.can_accumulate(x, w):
        pytest.skip("no accumulating product at this row count")
    ref = out.double() + 0.6 * (x.double() @ w.double().T)
    ops.linear_skinny(x, w, out, accumulate=True, alpha=0.6)
    close(out, ref, 2e-5, "scaled accumulate")
