"""Backward passes of the router, SwiGLU, MLP and expert ops and of the whole block, against autograd of the oracle
(float64 on the CPU) evaluated on the same inputs and, where a selection is involved, on the HIP path's own indices."""
import pytest
import torch

from helpers import rel_fro
from oracle import flashmoe_oracle as orc

pytestmark = pytest.mark.gpu

GRAD_FRO = {torch.float32: 2e-5, torch.bfloat16: 1.5e-2, torch.float16: 3e-3}


def gen(seed):
    return torch.Generator().manual_seed(seed)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,nk,K", [(64, 32, 16), (300, 128, 64), (17, 512, 128), (5, 8, 1),
                                    (6, 9000, 48)])    # more keys than one LDS row pair holds: rows built 4096 keys at a time
def test_router_backward(dtype, T, nk, K):
    from flash_moe.ops import flash_router_func
    from flash_moe.ops.hip.flash_router import router_topk_backward

    lp = orc.make_router_inputs(T, nk, seed=1).to(dtype)
    lp_dev = lp.cuda().requires_grad_(True)
    scores, indices = flash_router_func(lp_dev, nk, K)
    ds = torch.randn(T, K, generator=gen(2)).to(dtype)
    scores.backward(ds.cuda())
    idx = indices.cpu()
    # scatter-add restated with index_add_ in float64
    ref = torch.zeros(2, T, nk, dtype=torch.float64)
    rows = torch.arange(T).repeat_interleave(K)
    ref[0].index_put_((rows, (idx // nk).flatten()), ds.double().flatten(), accumulate=True)
    ref[1].index_put_((rows, (idx % nk).flatten()), ds.double().flatten(), accumulate=True)
    got = lp_dev.grad
    assert got.shape == (2, T, nk) and got.dtype == dtype
    tol = {torch.float32: 1e-6, torch.bfloat16: 8e-3, torch.float16: 1e-3}[dtype]
    torch.testing.assert_close(got.double().cpu(), ref, rtol=tol, atol=tol * max(1.0, float(ref.abs().max())))
    # the op-level function gives the same tensor, twice
    again = router_topk_backward(ds.cuda(), indices, nk)
    assert torch.equal(again, got) and torch.equal(router_topk_backward(ds.cuda(), indices, nk), got)
    # the gradient of an unselected key is exactly zero and the total is conserved per token and half
    torch.testing.assert_close(got.double().sum(-1).cpu(), ref.sum(-1), rtol=5 * tol, atol=5 * tol * max(1.0, float(ref.abs().max())))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("norm", [False, True])
@pytest.mark.parametrize("T,nk,K", [(64, 32, 16), (130, 128, 64), (9, 512, 128), (5, 8, 1),
                                    (5, 8192, 64), (6, 20000, 96)])   # the last: rows built 4096 keys at a time
def test_route_backward(dtype, norm, T, nk, K):
    """Gate gradients -> gradient of the fp32 gate logits, against float64 autograd of log-softmax, pair sums, exp and
    renormalisation on the same ids; ids out of range carry nothing; the gradient of the returned logits is added."""
    from flash_moe.ops.hip.flash_router import route_backward

    logits = torch.randn(T, 2 * nk, generator=gen(1)) * 2.0
    if nk <= 512:
        idx = torch.stack([torch.randperm(nk * nk, generator=gen(10 + t))[:K] for t in range(T)])
    else:   # pairs that share keys (several gradients per key) and lie on both sides of every 4096-key boundary
        idx = torch.randint(0, nk, (T, K), generator=gen(10)) * nk + torch.randint(0, nk, (T, K), generator=gen(11))
        idx[:, : K // 2] = idx[:, K // 2 : 2 * (K // 2)] // nk * nk + (idx[:, : K // 2] % nk)
    if K > 2:
        idx[::3, 1] = nk * nk + 7
        idx[1::4, 2] = -1
    dg = torch.randn(T, K, generator=gen(2)).to(dtype)
    extra = (torch.randn(T, 2 * nk, generator=gen(3)) * 0.1).to(dtype)
    valid = (idx >= 0) & (idx < nk * nk)
    safe = idx.clamp(0, nk * nk - 1)
    lg = logits.double().requires_grad_(True)
    lp = torch.log_softmax(lg.view(T, 2, nk), -1)
    e = (lp[:, 0].gather(1, safe // nk) + lp[:, 1].gather(1, safe % nk)).exp() * valid
    gates = e / e.sum(-1, keepdim=True) if norm else e
    ((gates * dg.double()).sum() + (lg * extra.double()).sum()).backward()
    got = route_backward(dg.cuda(), idx.cuda(), logits.cuda(), nk, norm, extra.cuda())
    assert got.dtype == torch.float32 and got.shape == (T, 2 * nk)
    assert rel_fro(got, lg.grad) < 2e-5, rel_fro(got, lg.grad)
    without = route_backward(dg.cuda(), idx.cuda(), logits.cuda(), nk, norm)
    torch.testing.assert_close(without.cpu().double() + extra.double(), lg.grad, rtol=1e-4, atol=1e-5)
    assert torch.equal(route_backward(dg.cuda(), idx.cuda(), logits.cuda(), nk, norm, extra.cuda()), got)


@pytest.mark.parametrize("dtype,norm", [(torch.float32, False), (torch.float32, True), (torch.bfloat16, True)])
def test_block_autograd_node_equals_the_composition_of_ops(dtype, norm):
    """forward_autograd (one node, library calls only) and forward_autograd_ops (the reference's composition on the
    differentiable per-op functions) give the same outputs and gradients."""
    from test_block_gpu import build

    m, _ = build(128, 256, 1024, 8, norm, dtype, seed=4, std=0.05)
    x = torch.randn(2, 96, 128, generator=gen(5)).to(dtype).cuda()
    wy = torch.randn(2, 96, 128, generator=gen(6)).cuda()
    wl = (torch.randn(2, 192, 32, generator=gen(7)) * 0.1).cuda()
    results = []
    for fwd in (m.forward_autograd, m.forward_autograd_ops):
        m.router_norm.reset_running_stats()
        for p in m.parameters():
            p.grad = None
        xg = x.clone().requires_grad_(True)
        y, logits = fwd(xg)
        ((y.float() * wy).sum() + (logits.float() * wl).sum()).backward()
        results.append((y.detach(), logits.detach(), xg.grad, {k: v.grad.clone() for k, v in m.named_parameters()}))
    (y0, l0, gx0, gp0), (y1, l1, gx1, gp1) = results
    tol = 2e-5 if dtype == torch.float32 else 1.5e-2
    # same kernels for the logits; the gates come from the fused router here and from torch's exp there
    assert torch.equal(l0, l1) and rel_fro(y0, y1) < tol
    assert rel_fro(gx0, gx1) < tol, rel_fro(gx0, gx1)
    for k in gp0:
        assert rel_fro(gp0[k], gp1[k]) < tol, (k, rel_fro(gp0[k], gp1[k]))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(7, 64), (3, 5, 256), (128, 1024)])
def test_swiglu_backward(dtype, shape):
    from flash_moe.ops.hip.flash_mlp import swiglu_backward

    a, b, dc = (torch.randn(shape, generator=gen(s)).to(dtype) for s in (1, 2, 3))
    a64, b64 = a.double().requires_grad_(True), b.double().requires_grad_(True)
    (torch.nn.functional.silu(a64) * b64).backward(dc.double())
    da, db = swiglu_backward(a.cuda(), b.cuda(), dc.cuda())
    assert da.shape == a.shape and db.dtype == dtype
    tol = {torch.float32: 2e-6, torch.bfloat16: 8e-3, torch.float16: 1e-3}[dtype]
    torch.testing.assert_close(da.double().cpu(), a64.grad, rtol=tol, atol=tol)
    torch.testing.assert_close(db.double().cpu(), b64.grad, rtol=tol, atol=tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,H,I", [(128, 256, 512), (96, 64, 192), (512, 1024, 1024)])
def test_mlp_backward(dtype, T, H, I):
    from flash_moe.ops import flash_mlp_func

    x = torch.randn(T, H, generator=gen(1)).to(dtype)
    wg, wu, wd = ((torch.randn(s, generator=gen(k)) * 0.05).to(dtype) for k, s in ((2, (I, H)), (3, (I, H)), (4, (H, I))))
    dy = torch.randn(T, H, generator=gen(5)).to(dtype)
    leaves = [t.cuda().requires_grad_(True) for t in (x, wg, wu, wd)]
    flash_mlp_func(*leaves).backward(dy.cuda())
    ref_leaves = [t.double().requires_grad_(True) for t in (x, wg, wu, wd)]
    orc.mlp_forward(*ref_leaves).backward(dy.double())
    for name, got, ref in zip(("dx", "dgate", "dup", "ddown"), leaves, ref_leaves):
        assert got.grad.dtype == dtype and got.grad.shape == ref.shape
        fro = rel_fro(got.grad, ref.grad)
        assert fro < GRAD_FRO[dtype], f"{name}: relative Frobenius error {fro:.3e}"


def expert_case(T, H, E, K, dtype, seed, duplicates=False):
    x, wd, wu, idx, g = orc.make_expert_inputs(T, H, E, K, seed=seed)
    if duplicates:
        idx[:, K // 2:] = idx[:, : K - K // 2]        # every id twice per token: contributions add
    return x.to(dtype), wd.to(dtype), wu.to(dtype), idx, g.to(dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,H,E,K,dup", [(64, 128, 256, 8, False), (200, 256, 64, 16, True), (33, 1024, 4096, 5, False),
                                         (16, 2048, 512, 4, False),
                                         (12, 8192, 48, 4, False), (20, 5120, 40, 3, True)])   # rows beyond one wave's registers
def test_expert_backward(dtype, T, H, E, K, dup):
    from flash_moe.ops import flash_expert_func
    from flash_moe.ops.hip.flash_expert import expert_backward

    x, wd, wu, idx, g = expert_case(T, H, E, K, dtype, seed=3, duplicates=dup)
    do = torch.randn(T, H, generator=gen(9)).to(dtype)
    leaves = [t.cuda().requires_grad_(True) for t in (x, wd, wu, g)]
    out = flash_expert_func(leaves[0], leaves[1], leaves[2], idx.cuda(), leaves[3])
    out.backward(do.cuda())
    ref_leaves = [t.double().requires_grad_(True) for t in (x, wd, wu, g)]
    orc.expert_forward(ref_leaves[0], ref_leaves[1], ref_leaves[2], idx, ref_leaves[3]).backward(do.double())
    for name, got, ref in zip(("dx", "ddown", "dup", "dgates"), leaves, ref_leaves):
        assert got.grad.dtype == dtype and got.grad.shape == ref.shape
        fro = rel_fro(got.grad, ref.grad)
        assert fro < GRAD_FRO[dtype], f"{name}: relative Frobenius error {fro:.3e}"
    # rows of experts nobody selected are exactly zero; the run is reproducible bit for bit
    unused = torch.ones(E, dtype=torch.bool)
    unused[idx.flatten()] = False
    assert (leaves[1].grad[unused.cuda()] == 0).all() and (leaves[2].grad[unused.cuda()] == 0).all()
    again = expert_backward(do.cuda(), x.cuda(), wd.cuda(), wu.cuda(), idx.cuda(), g.cuda())
    for a, b in zip(again, (leaves[0].grad, leaves[1].grad, leaves[2].grad, leaves[3].grad)):
        assert torch.equal(a, b)


def test_expert_backward_ignores_ids_out_of_range_and_handles_one_hot_expert():
    from flash_moe.ops.hip.flash_expert import expert_backward

    T, H, E, K, dtype = 96, 128, 32, 4, torch.float32
    x, wd, wu, idx, g = expert_case(T, H, E, K, dtype, seed=5)
    idx[:, 0] = 7                       # one expert takes a pair of every token: a long segment
    idx[::3, 1] = E + 5                 # invalid ids contribute nothing
    idx[1::3, 2] = -1
    do = torch.randn(T, H, generator=gen(4))
    dx, dwd, dwu, dg = expert_backward(*(t.cuda() for t in (do, x, wd, wu, idx, g)))
    valid = (idx >= 0) & (idx < E)
    ref_leaves = [t.double().requires_grad_(True) for t in (x, wd, wu, g)]
    safe = idx.clamp(0, E - 1)
    gates_masked = ref_leaves[3] * valid.double()
    orc.expert_forward(ref_leaves[0], ref_leaves[1], ref_leaves[2], safe, gates_masked).backward(do.double())
    for name, got, ref in zip(("dx", "ddown", "dup"), (dx, dwd, dwu), ref_leaves):
        assert rel_fro(got, ref.grad) < GRAD_FRO[dtype], name
    assert rel_fro(dg, ref_leaves[3].grad * valid.double()) < GRAD_FRO[dtype] and (dg.cpu()[~valid] == 0).all()


@pytest.mark.parametrize("norm", [False, True])
def test_block_backward_fp32(norm):
    """All parameter and input gradients of the block, against float64 autograd of the oracle's formulas evaluated on
    the HIP path's own selection (the selection itself carries no gradient)."""
    from test_block_gpu import build

    H, I, E, K, T = 128, 256, 1024, 8, 192
    nk = 32
    m, w = build(H, I, E, K, norm, torch.float32, seed=2, std=0.05)
    x = torch.randn(2, T // 2, H, generator=gen(3))
    xd = x.cuda().requires_grad_(True)
    y, logits = m(xd)
    wy, wl = torch.randn(y.shape, generator=gen(4)), torch.randn(logits.shape, generator=gen(5)) * 0.1
    ((y * wy.cuda()).sum() + (logits * wl.cuda()).sum()).backward()
    assert int(m.router_norm.num_batches_tracked) == 1

    with torch.no_grad():
        m.router_norm.reset_running_stats()
        _, _, indices, _ = m.route(xd.detach().view(-1, H))
    idx = indices.cpu()
    p = {k: v.detach().double().cpu().requires_grad_(True) for k, v in m.named_parameters()}
    x64 = x.double().requires_grad_(True)
    tok = x64.view(-1, H)
    q = torch.nn.functional.batch_norm(tok, None, None, training=True, eps=1e-5)
    lg = q @ p["router_gate.weight"].t()
    lp = torch.log_softmax(lg.view(T, 2, nk), -1)
    scores = lp[:, 0].gather(1, idx // nk) + lp[:, 1].gather(1, idx % nk)
    gates = scores.exp()
    if norm:
        gates = gates / gates.sum(-1, keepdim=True)
    y64 = orc.mlp_forward(tok, p["gate_proj.weight"], p["up_proj.weight"], p["down_proj.weight"]) + orc.expert_forward(
        tok, p["down_embed.weight"], p["up_embed.weight"], idx, gates)
    ((y64.view(y.shape) * wy.double()).sum() + (lg.view(T, 2, nk).transpose(0, 1) * wl.double()).sum()).backward()
    assert rel_fro(y, y64.view(y.shape)) < 2e-5
    assert rel_fro(xd.grad, x64.grad) < 2e-4, f"dx {rel_fro(xd.grad, x64.grad):.3e}"
    for k, v in m.named_parameters():
        fro = rel_fro(v.grad, p[k].grad)
        assert fro < 2e-4, f"{k}: relative Frobenius error {fro:.3e}"


def test_block_backward_bf16_runs_and_matches_the_fused_forward():
    from test_block_gpu import build

    m, _ = build(256, 512, 4096, 16, True, torch.bfloat16, seed=1)
    x = torch.randn(1, 256, 256, generator=gen(2)).to(torch.bfloat16).cuda()
    with torch.no_grad():
        y0, l0 = m(x)
    m.router_norm.reset_running_stats()
    y1, l1 = m(x.clone().requires_grad_(True))
    y1.float().square().mean().backward()
    assert rel_fro(y1, y0) < 1e-2 and rel_fro(l1, l0) < 1e-2
    for k, v in m.named_parameters():
        assert v.grad is not None and torch.isfinite(v.grad).all(), k


def test_expert_backward_c4_tables_fewer_tokens():
    """C4's tables (16384 experts of width 1024, top-64, bf16) on 256 tokens: float64 autograd of the oracle in chunks."""
    from flash_moe.ops.hip.flash_expert import expert_backward

    T, H, E, K, dtype = 256, 1024, 16384, 64, torch.bfloat16
    x, wd, wu, idx, g = expert_case(T, H, E, K, dtype, seed=11)
    do = torch.randn(T, H, generator=gen(12)).to(dtype)
    dx, dwd, dwu, dg = expert_backward(*(t.cuda() for t in (do, x, wd, wu, idx, g)))
    ref = [t.double().requires_grad_(True) for t in (x, wd, wu, g)]
    orc.expert_forward(ref[0], ref[1], ref[2], idx, ref[3], token_chunk=64).backward(do.double())
    for name, got, r in zip(("dx", "ddown", "dup", "dgates"), (dx, dwd, dwu, dg), ref):
        fro = rel_fro(got, r.grad)
        assert fro < GRAD_FRO[dtype], f"{name}: relative Frobenius error {fro:.3e}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_expert_backward_column_slices(dtype):
    """Enough pairs (65536) for the column-slice schedule of the per-token part; some ids invalid, some doubled."""
    from flash_moe import _C
    from flash_moe.ops.hip.flash_expert import expert_backward

    T, H, E, K = 1024, 264, 4096, 64                    # 264 columns: the last slice is partial
    code = _C.dtype_code(dtype)
    lib = _C.lib()
    assert lib.fmoe_expert_backward_workspace_bytes(T, H, E, K, code) > lib.fmoe_expert_backward_workspace_bytes(T // 2, H, E, K, code) * 3
    x, wd, wu, idx, g = expert_case(T, H, E, K, dtype, seed=21)
    idx[:, 5] = idx[:, 4]
    idx[::7, 9] = E + 3
    idx[3::11, 17] = -2
    do = torch.randn(T, H, generator=gen(22)).to(dtype)
    dx, dwd, dwu, dg = expert_backward(*(t.cuda() for t in (do, x, wd, wu, idx, g)))
    valid = (idx >= 0) & (idx < E)
    ref = [t.double().requires_grad_(True) for t in (x, wd, wu, g)]
    orc.expert_forward(ref[0], ref[1], ref[2], idx.clamp(0, E - 1), ref[3] * valid.double(), token_chunk=128).backward(do.double())
    for name, got, r in zip(("dx", "ddown", "dup"), (dx, dwd, dwu), ref):
        fro = rel_fro(got, r.grad)
        assert fro < GRAD_FRO[dtype], f"{name}: relative Frobenius error {fro:.3e}"
    assert rel_fro(dg, ref[3].grad * valid.double()) < GRAD_FRO[dtype] and (dg.cpu()[~valid] == 0).all()
    again = expert_backward(*(t.cuda() for t in (do, x, wd, wu, idx, g)))
    assert all(torch.equal(a, b) for a, b in zip(again, (dx, dwd, dwu, dg)))


def test_block_backward_c4_full_size_properties():
    """Forward + backward of the README block at full size: finite, reproducible gradients for every parameter, and the
    gradient of the input agrees with a finite difference of the loss along a random direction (fp32 accumulation of
    a bf16 forward, so the bar is loose)."""
    from test_block_gpu import build

    dtype = torch.bfloat16
    m, _ = build(1024, 4096, 16384, 64, False, dtype)
    m.eval()                                     # running statistics: the loss is a fixed function of x
    x = torch.randn(1, 4096, 1024, generator=gen(0)).to(dtype).cuda()
    wy = torch.randn(1, 4096, 1024, generator=gen(1)).to(dtype).cuda()

    def run():
        for p in m.parameters():
            p.grad = None
        xg = x.clone().requires_grad_(True)
        y, _ = m(xg)
        (y.float() * wy.float()).sum().backward()
        return xg.grad, {k: v.grad.clone() for k, v in m.named_parameters()}

    gx, gp = run()
    gx2, gp2 = run()
    assert torch.equal(gx, gx2) and all(torch.equal(gp[k], gp2[k]) for k in gp)
    assert torch.isfinite(gx).all() and all(torch.isfinite(v).all() and v.abs().sum() > 0 for k, v in gp.items()
                                            if k != "router_gate.weight")
    # expert rows without a selected pair have zero gradient, the others (almost surely) not
    with torch.no_grad():
        _, _, indices, _ = m.route(x.view(-1, 1024))
    used = torch.zeros(16384, dtype=torch.bool, device="cuda")
    used[indices.flatten()] = True
    assert (gp["down_embed.weight"][~used] == 0).all() and (gp["up_embed.weight"][~used] == 0).all()
    assert (gp["up_embed.weight"][used].abs().sum(-1) > 0).all()


def test_backward_of_empty_batches():
    from flash_moe.ops.hip.flash_expert import expert_backward
    from flash_moe.ops.hip.flash_mlp import mlp_backward
    from flash_moe.ops.hip.flash_router import router_topk_backward

    H, E, K, I, nk = 64, 32, 4, 128, 8
    z = lambda *s: torch.zeros(*s, device="cuda")
    assert router_topk_backward(z(0, K), torch.zeros(0, K, dtype=torch.int64, device="cuda"), nk).shape == (2, 0, nk)
    wd, wu = torch.randn(E, H, device="cuda"), torch.randn(E, H, device="cuda")
    dx, dwd, dwu, dg = expert_backward(z(0, H), z(0, H), wd, wu, torch.zeros(0, K, dtype=torch.int64, device="cuda"), z(0, K))
    assert dx.shape == (0, H) and dg.shape == (0, K) and (dwd == 0).all() and (dwu == 0).all()
    dx, dwg, dwu2, dwd2 = mlp_backward(z(0, H), z(0, H), torch.randn(I, H, device="cuda"), torch.randn(I, H, device="cuda"),
                                       torch.randn(H, I, device="cuda"))
    assert dx.shape == (0, H) and (dwg == 0).all() and (dwu2 == 0).all() and (dwd2 == 0).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_autograd_of_an_empty_batch_gives_zero_gradients(dtype):
    """An empty batch with trainable parameters: the autograd functions return zero gradients of the right shapes."""
    from flash_moe.modules.flash_moe import FlashMoE, FlashMoEConfig
    from flash_moe.ops.hip.flash_mlp import flash_mlp_func

    H, I = 64, 128
    wg, wu, wd = (torch.randn(s, device="cuda").to(dtype).requires_grad_(True) for s in ((I, H), (I, H), (H, I)))
    x = torch.zeros(0, H, device="cuda", dtype=dtype, requires_grad=True)
    y = flash_mlp_func(x, wg, wu, wd)
    assert y.shape == (0, H)
    y.sum().backward()
    assert x.grad.shape == (0, H) and all(w.grad is not None and (w.grad == 0).all() for w in (wg, wu, wd))

    m = FlashMoE(FlashMoEConfig(H, I, "silu", 64, 4, False)).to(device="cuda", dtype=dtype).eval()
    out, logits = m(torch.zeros(1, 0, H, device="cuda", dtype=dtype))
    assert out.shape == (1, 0, H) and logits.shape == (2, 0, 8)
    (out.float().sum() + logits.float().sum()).backward()
    for name, p in m.named_parameters():
        assert p.grad is None or (p.grad == 0).all(), name


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_block_backward_with_a_key_count_that_is_not_a_multiple_of_four(dtype):
    """num_experts = 100 -> 10 keys per half: rows of the gate gradient are not whole 16-byte packets."""
    from flash_moe.modules.flash_moe import FlashMoE, FlashMoEConfig

    H, I, E, K, T = 64, 128, 100, 4, 96
    m = FlashMoE(FlashMoEConfig(H, I, "silu", E, K, True)).to(device="cuda", dtype=dtype)
    x = torch.randn(2, T // 2, H, generator=gen(3)).to(dtype).cuda()

    def grads(forward):
        for p in m.parameters():
            p.grad = None
        m.router_norm.reset_running_stats()
        xg = x.clone().requires_grad_(True)
        y, logits = forward(xg)
        (y.float().square().sum() + logits.float().sum() * 0.01).backward()
        return xg.grad, {k: v.grad.clone() for k, v in m.named_parameters()}

    gx, gp = grads(m.forward_autograd)
    gx2, gp2 = grads(m.forward_autograd_ops)
    tol = 1e-4 if dtype == torch.float32 else 3e-2
    assert torch.isfinite(gx).all() and rel_fro(gx, gx2) < tol
    for k in gp:
        assert torch.isfinite(gp[k]).all() and rel_fro(gp[k], gp2[k]) < tol, k
    assert gp["router_gate.weight"].shape == (20, H) and gp["router_gate.weight"].abs().sum() > 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_mlp_backward_with_saved_products_equals_recomputation(dtype):
    from flash_moe.ops.hip.flash_mlp import mlp_backward, mlp_forward, mlp_forward_saving

    T, H, I = 256, 256, 512
    x = torch.randn(T, H, generator=gen(1)).to(dtype).cuda()
    wg, wu, wd = ((torch.randn(s, generator=gen(k)) * 0.05).to(dtype).cuda() for k, s in ((2, (I, H)), (3, (I, H)), (4, (H, I))))
    dy = torch.randn(T, H, generator=gen(5)).to(dtype).cuda()
    out, saved = mlp_forward_saving(x, wg, wu, wd)
    assert torch.equal(out, mlp_forward(x, wg, wu, wd)) and saved.shape == (2, T, I)
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    torch.testing.assert_close(saved[0].float(), x.float() @ wg.float().t(), rtol=tol, atol=tol)
    torch.testing.assert_close(saved[1].float(), x.float() @ wu.float().t(), rtol=tol, atol=tol)
    for a, b in zip(mlp_backward(dy, x, wg, wu, wd, saved), mlp_backward(dy, x, wg, wu, wd)):
        assert rel_fro(a, b) < (1e-6 if dtype == torch.float32 else 2e-3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("stacked_weights", [False, True])
@pytest.mark.parametrize("stacked_grads", [False, True])
def test_mlp_backward_with_adjacent_and_separate_buffers(dtype, stacked_weights, stacked_grads):
    # fmoe_mlp_backward forms dWg and dWu as one product when dup_w starts where dgate_w ends, two otherwise; weights that
    # happen to follow each other in memory must make no difference.  Every combination against float64.
    from flash_moe import _C

    T, H, I = 320, 256, 384
    x = torch.randn(T, H, generator=gen(1)).to(dtype)
    wg, wu, wd = ((torch.randn(s, generator=gen(k)) * 0.05).to(dtype) for k, s in ((2, (I, H)), (3, (I, H)), (4, (H, I))))
    dy = torch.randn(T, H, generator=gen(5)).to(dtype)
    ref_leaves = [t.double().requires_grad_(True) for t in (x, wg, wu, wd)]
    orc.mlp_forward(*ref_leaves).backward(dy.double())

    xg, dyg, wdg = x.cuda(), dy.cuda(), wd.cuda()
    if stacked_weights:
        w2 = torch.cat([wg, wu]).cuda()
        wgg, wug = w2[:I], w2[I:]
        assert wug.data_ptr() == wgg.data_ptr() + I * H * wgg.element_size()
    else:
        w2 = torch.empty(2 * I * H + 64, device="cuda", dtype=dtype)          # a gap of 64 elements between the two
        wgg, wug = w2[:I * H].view(I, H).copy_(wg), w2[I * H + 64:].view(I, H).copy_(wu)
    if stacked_grads:
        g2 = torch.empty(2 * I, H, device="cuda", dtype=dtype)
        dwg, dwu = g2[:I], g2[I:]
    else:
        g2 = torch.empty(2 * I * H + 64, device="cuda", dtype=dtype)
        dwg, dwu = g2[:I * H].view(I, H), g2[I * H + 64:].view(I, H)
    dx, dwd = torch.empty_like(xg), torch.empty_like(wdg)
    L, code = _C.lib(), _C.dtype_code(dtype)
    ws_bytes = L.fmoe_mlp_backward_workspace_bytes(T, H, I, code)
    ws = torch.empty(ws_bytes, device="cuda", dtype=torch.uint8)
    status = L.fmoe_mlp_backward(_C.ptr(dyg), _C.ptr(xg), _C.ptr(wgg), _C.ptr(wug), _C.ptr(wdg), None, T, H, I, code, _C.ptr(dx),
                                 _C.ptr(dwg), _C.ptr(dwu), _C.ptr(dwd), _C.ptr(ws), ws_bytes, _C.current_stream(xg.device))
    _C.check(status, "fmoe_mlp_backward")
    torch.cuda.synchronize()
    for name, got, ref in zip(("dx", "dgate", "dup", "ddown"), (dx, dwg, dwu, dwd), ref_leaves):
        fro = rel_fro(got.cpu(), ref.grad)
        assert fro < GRAD_FRO[dtype], f"{name}: relative Frobenius error {fro:.3e}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("training", [True, False])
@pytest.mark.parametrize("T,H,nk", [(256, 128, 16), (1000, 1024, 128), (65, 64, 8), (256, 128, 32), (1024, 1024, 128),
                                    (128, 64, 10), (70, 64, 6), (64, 128, 30), (40, 32, 81)])
def test_router_prologue_backward(dtype, training, T, H, nk):
    """Batch norm + gate product: gradients of the input and of the gate weights against float64 autograd."""
    from flash_moe.ops.hip.flash_router import router_prologue

    x = (torch.randn(T, H, generator=gen(1)) * 1.5 + 0.3).to(dtype)
    w = (torch.randn(2 * nk, H, generator=gen(2)) * 0.05).to(dtype)
    g32 = torch.randn(T, 2 * nk, generator=gen(3))
    g16 = (torch.randn(T, 2 * nk, generator=gen(4)) * 0.5).to(dtype)
    norm = torch.nn.BatchNorm1d(H, affine=False).cuda().to(dtype)
    with torch.no_grad():
        norm.running_mean.normal_(0.0, 0.2, generator=torch.Generator(device="cuda").manual_seed(5))
        norm.running_var.uniform_(0.5, 2.0, generator=torch.Generator(device="cuda").manual_seed(6))
    rm0, rv0 = norm.running_mean.clone(), norm.running_var.clone()
    norm.train(training)
    xd, wd = x.cuda().requires_grad_(True), w.cuda().requires_grad_(True)
    logits32, logits = router_prologue(xd, wd, norm)
    assert logits32.dtype == torch.float32 and logits.dtype == dtype
    ((logits32 * g32.cuda()).sum() + (logits.float() * g16.cuda().float()).sum()).backward()

    x64, w64 = x.double().requires_grad_(True), w.double().requires_grad_(True)
    q = torch.nn.functional.batch_norm(x64, rm0.double().cpu(), rv0.double().cpu(), training=training, eps=1e-5)
    ref = q @ w64.t()
    (ref * (g32.double() + g16.double())).sum().backward()
    tol = {torch.float32: 2e-5, torch.bfloat16: 1.2e-2, torch.float16: 3e-3}[dtype]
    assert rel_fro(logits32, ref) < tol
    assert rel_fro(xd.grad, x64.grad) < tol, f"dx {rel_fro(xd.grad, x64.grad):.3e}"
    assert rel_fro(wd.grad, w64.grad) < tol, f"dgate {rel_fro(wd.grad, w64.grad):.3e}"
    if training:   # a constant shift of the loss gradient along tokens cannot change dx: columns of dx sum to ~0
        assert float(xd.grad.float().sum(0).abs().max()) < 50 * tol * float(xd.grad.float().abs().max()) * T ** 0.5


def test_expert_backward_with_skewed_routing_is_exact_and_quick():
    """One expert selected by every one of 8192 tokens (a segment of 8192 pairs, as early in training or after a router
    collapse) next to ordinary experts: gradients against float64, bit-reproducible, and the call stays in the range of
    an ordinary backward (the long segment is walked once, in order)."""
    import time

    from flash_moe.ops.hip.flash_expert import expert_backward

    T, H, E, K = 8192, 1024, 4096, 8
    g = gen(31)
    x = torch.randn(T, H, generator=g).bfloat16()
    wd = (torch.randn(E, H, generator=g) * 0.05).bfloat16()
    wu = (torch.randn(E, H, generator=g) * 0.05).bfloat16()
    idx = torch.stack([torch.randperm(E - 1, generator=g)[:K] + 1 for _ in range(T)])
    idx[:, 3] = 0                                                # every token also selects expert 0
    gates = torch.softmax(torch.randn(T, K, generator=g), -1).bfloat16()
    dout = (torch.randn(T, H, generator=g) * 0.1).bfloat16()
    args = tuple(t.cuda() for t in (dout, x, wd, wu, idx, gates))
    got = expert_backward(*args)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    again = expert_backward(*args)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    assert all(torch.equal(a, b) for a, b in zip(got, again))
    assert elapsed < 0.05, f"{elapsed * 1e3:.1f} ms for a backward with one 8192-pair segment"
    # the hot expert's rows against float64: ddown[0] = sum_t ds_t x_t, dup[0] = sum_t silu(s_t) g_t dout_t
    x64, wd64, wu64, g64, do64 = (t.double() for t in (x, wd, wu, gates, dout))
    s = x64 @ wd64[0]
    sig = torch.sigmoid(s)
    act = s * sig
    u = do64 @ wu64[0]
    ds = u * g64[:, 3] * (sig * (1 + s * (1 - sig)))
    assert rel_fro(got[1][0], ds @ x64) < 1.5e-2
    assert rel_fro(got[2][0], (act * g64[:, 3]) @ do64) < 1.5e-2
    # an ordinary expert's rows too
    e = int(idx[5, 0])
    sel = (idx == e)
    tok, slot = sel.nonzero(as_tuple=True)
    s_e = x64[tok] @ wd64[e]
    sig_e = torch.sigmoid(s_e)
    u_e = do64[tok] @ wu64[e]
    assert rel_fro(got[2][e], (s_e * sig_e * g64[tok, slot]) @ do64[tok]) < 1.5e-2
    assert rel_fro(got[1][e], (u_e * g64[tok, slot] * (sig_e * (1 + s_e * (1 - sig_e)))) @ x64[tok]) < 1.5e-2
