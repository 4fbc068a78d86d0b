"""Reference-style throughput tests (the case lists of the reference's tests/test_router.py:75-88, test_expert.py:277-290,
test_mlp.py:167-176), HIP ops against a torch-eager baseline on the same device, with validation that asserts.
Run with `pytest -s` to see the tables.  By default one small and one large case per op run; FMOE_FULL_BENCH=1 runs them all."""
import os

import pytest
import torch

import harness
from oracle import flashmoe_oracle as orc

pytestmark = pytest.mark.gpu
FULL = os.environ.get("FMOE_FULL_BENCH") == "1"


def pick(cases):
    return cases if FULL else [cases[0], cases[-1]]


ROUTER_CASES = [(4096, 64, 8), (4096, 128, 16), (8192, 64, 8), (8192, 128, 16), (16384, 64, 8), (16384, 128, 16),
                (32768, 64, 8), (32768, 128, 16)]
EXPERT_CASES = [(1024, 1024, 102400, 512), (1024, 1024, 102400, 1024), (1024, 1024, 102400, 2048), (1024, 1024, 102400, 4096),
                (2048, 1024, 102400, 512), (4096, 1024, 102400, 512), (8192, 1024, 102400, 512), (16384, 1024, 102400, 512)]
MLP_CASES = [(1024, 4096, 16384), (2048, 4096, 16384), (4096, 4096, 16384), (8192, 4096, 16384)]


def gen(seed=0):
    return torch.Generator(device="cuda").manual_seed(seed)


def torch_router(lp, nk, k):
    """Exhaustive baseline in chunks of tokens: all nk*nk sums, torch.topk (tests/test_router.py:8-16)."""
    scores, indices = [], []
    for lo in range(0, lp.shape[1], 4096):
        s = (lp[0, lo:lo + 4096, :, None] + lp[1, lo:lo + 4096, None, :]).flatten(1)
        v, i = s.topk(k, dim=-1)
        scores.append(v); indices.append(i)
    return torch.cat(scores), torch.cat(indices)


@pytest.mark.parametrize("case", pick(ROUTER_CASES))
def test_router_forward_throughput(case):
    from flash_moe.ops import flash_router_func

    T, nk, K = case
    lp = torch.log_softmax(torch.randn(2, T, nk, device="cuda", generator=gen()), -1)

    def validate(out, ref):
        torch.testing.assert_close(out[0], ref[0], rtol=0, atol=1e-6)
        tied = (ref[0][:, 1:] - ref[0][:, :-1]).abs().min(-1).values < 1e-6      # exact ties may pick another index
        same = (out[1].sort(-1).values == ref[1].sort(-1).values).all(-1)
        assert (same | tied).all()

    with torch.no_grad():
        harness.run([harness.Impl(harness.BASELINE, lambda x: torch_router(x, nk, K)),
                     harness.Impl(harness.HIP, lambda x: flash_router_func(x, nk, K))], lambda: (lp,),
                    flops=4.0 * 2 * T * nk * nk, what=f"router forward T={T} E={nk * nk} K={K}", validate=validate)


@pytest.mark.parametrize("case", pick(ROUTER_CASES))
def test_router_backward_throughput(case):
    from flash_moe.ops import flash_router_func

    T, nk, K = case
    lp = torch.log_softmax(torch.randn(2, T, nk, device="cuda", generator=gen()), -1)
    ds = torch.randn(T, K, device="cuda", generator=gen(1))

    def step(fn):
        def run(x):
            x = x.detach().requires_grad_(True)
            fn(x)[0].backward(ds)
            return x.grad
        return run

    # where sums tie exactly inside the top K+1 the two implementations may order or pick the tied pairs differently,
    # which moves a gradient from one key to another: those few tokens are compared by their per-half totals only
    with torch.no_grad():
        top = torch_router(lp, nk, K + 1)[0]
    clean = ((top[:, 1:] - top[:, :-1]).abs() > 1e-6).all(-1)
    assert clean.float().mean() > 0.99

    def validate(out, ref):
        torch.testing.assert_close(out[:, clean], ref[:, clean], rtol=1e-5, atol=1e-5)
        torch.testing.assert_close(out.sum(-1), ref.sum(-1), rtol=1e-4, atol=1e-4)

    harness.run([harness.Impl(harness.BASELINE, step(lambda x: torch_router(x, nk, K))),
                 harness.Impl(harness.HIP, step(lambda x: flash_router_func(x, nk, K)))], lambda: (lp,),
                flops=2 * 4.0 * 2 * T * nk * nk, what=f"router forward+backward T={T} E={nk * nk} K={K}", validate=validate)


def expert_inputs(T, H, E, K, dtype):
    g = gen()
    x = torch.randn(T, H, device="cuda", generator=g).to(dtype)
    wd = (torch.randn(E, H, device="cuda", generator=g) * 0.02).to(dtype)
    wu = (torch.randn(E, H, device="cuda", generator=g) * 0.02).to(dtype)
    idx = torch.randint(0, E, (T, K), device="cuda", generator=g)
    gates = torch.softmax(torch.randn(T, K, device="cuda", generator=g), -1).to(dtype)
    return x, wd, wu, idx, gates


@pytest.mark.parametrize("case", pick(EXPERT_CASES))
def test_expert_forward_throughput(case):
    from flash_moe.ops import flash_expert_func

    T, H, E, K = case
    x, wd, wu, idx, g = expert_inputs(T, H, E, K, torch.bfloat16)
    chunk = max(1, (1 << 28) // (K * H))         # the baseline's two [chunk, K, H] gathers stay around 1 GiB
    with torch.no_grad():
        harness.run([harness.Impl(harness.BASELINE, lambda *a: orc.expert_forward(*a, token_chunk=chunk)),
                     harness.Impl(harness.HIP, flash_expert_func)], lambda: (x, wd, wu, idx, g),
                    flops=4.0 * T * K * H, what=f"expert forward T={T} H={H} E={E} K={K}")


@pytest.mark.parametrize("case", pick(EXPERT_CASES[:1] + EXPERT_CASES[4:6]))
def test_expert_backward_throughput(case):
    from flash_moe.ops import flash_expert_func

    T, H, E, K = case
    x, wd, wu, idx, g = expert_inputs(T, H, E, K, torch.bfloat16)
    do = torch.randn(T, H, device="cuda", generator=gen(2)).to(torch.bfloat16)
    chunk = max(1, (1 << 27) // (K * H))

    def step(fn):
        def run(*a):
            leaves = [t.detach().requires_grad_(True) for t in (a[0], a[1], a[2], a[4])]
            fn(leaves[0], leaves[1], leaves[2], a[3], leaves[3]).backward(do)
            return tuple(t.grad for t in leaves)
        return run

    def validate(out, ref):
        # the eager baseline accumulates its gradients in bf16; compare at the scale of each tensor
        for o, r, name in zip(out, ref, ("dx", "ddown", "dup", "dgates")):
            err = (o.float() - r.float()).norm() / r.float().norm().clamp_min(1e-30)
            assert err < 5e-2, f"{name}: relative Frobenius error {float(err):.3e}"

    harness.run([harness.Impl(harness.BASELINE, step(lambda *a: orc.expert_forward(*a, token_chunk=chunk))),
                 harness.Impl(harness.HIP, step(flash_expert_func))], lambda: (x, wd, wu, idx, g),
                flops=3 * 4.0 * T * K * H, what=f"expert forward+backward T={T} H={H} E={E} K={K}", repeat=5, validate=validate)


def mlp_inputs(T, H, I, dtype):
    g = gen()
    x = torch.randn(T, H, device="cuda", generator=g).to(dtype)
    ws = [(torch.randn(s, device="cuda", generator=g) * 0.02).to(dtype) for s in ((I, H), (I, H), (H, I))]
    return (x, *ws)


@pytest.mark.parametrize("case", pick(MLP_CASES))
def test_mlp_forward_throughput(case):
    from flash_moe.ops import flash_mlp_func

    T, H, I = case
    args = mlp_inputs(T, H, I, torch.bfloat16)
    with torch.no_grad():
        harness.run([harness.Impl(harness.BASELINE, orc.mlp_forward), harness.Impl(harness.HIP, flash_mlp_func)], lambda: args,
                    flops=6.0 * T * H * I, what=f"mlp forward T={T} H={H} I={I}")


@pytest.mark.parametrize("case", pick(MLP_CASES))
def test_mlp_backward_throughput(case):
    from flash_moe.ops import flash_mlp_func

    T, H, I = case
    args = mlp_inputs(T, H, I, torch.bfloat16)
    dy = torch.randn(T, H, device="cuda", generator=gen(3)).to(torch.bfloat16)

    def step(fn):
        def run(*a):
            leaves = [t.detach().requires_grad_(True) for t in a]
            fn(*leaves).backward(dy)
            return tuple(t.grad for t in leaves)
        return run

    def validate(out, ref):
        for o, r, name in zip(out, ref, ("dx", "dgate", "dup", "ddown")):
            err = (o.float() - r.float()).norm() / r.float().norm().clamp_min(1e-30)
            assert err < 3e-2, f"{name}: relative Frobenius error {float(err):.3e}"

    harness.run([harness.Impl(harness.BASELINE, step(orc.mlp_forward)), harness.Impl(harness.HIP, step(flash_mlp_func))],
                lambda: args, flops=3 * 6.0 * T * H * I, what=f"mlp forward+backward T={T} H={H} I={I}", repeat=10, validate=validate)


PEER_CASES = [(1024, 1024, 102400, 1250), (1024, 1024, 102400, 2500), (1024, 1024, 102400, 6250), (1024, 1024, 102400, 12500),
              (2048, 1024, 102400, 1250), (4096, 1024, 102400, 1250), (8192, 1024, 102400, 1250), (16384, 1024, 102400, 1250)]
PKM_CASES = [(1024, 1024, 197136, 2500), (1024, 1024, 197136, 5000), (1024, 1024, 197136, 12500), (1024, 1024, 197136, 25000),
             (2048, 1024, 197136, 2500), (4096, 1024, 197136, 2500), (8192, 1024, 197136, 2500), (16384, 1024, 197136, 2500)]


def chunked(fn, chunk, token_args):
    """Eager baseline over token chunks (its [chunk, K, H] gathers would not fit otherwise); `token_args` are the
    positions of the per-token arguments."""
    def run(*a):
        T = a[token_args[0]].shape[0]
        return torch.cat([fn(*[t[lo:lo + chunk] if i in token_args else t for i, t in enumerate(a)]) for lo in range(0, T, chunk)])
    return run


@pytest.mark.parametrize("case", pick(PEER_CASES))
def test_peer_forward_throughput(case):
    """Case list of the reference's tests/test_peer.py:226-237."""
    from flash_moe.ops.triton.peer import triton_peer_func
    from test_peer_pkm_gpu import peer_reference

    T, H, E, K = case
    x, wd, wu, idx, w = expert_inputs(T, H, E, K, torch.bfloat16)
    chunk = max(1, (1 << 28) // (K * H))
    with torch.no_grad():
        harness.run([harness.Impl(harness.BASELINE, chunked(peer_reference, chunk, (0, 3, 4))),
                     harness.Impl(harness.HIP, triton_peer_func)], lambda: (x, wd, wu, w, idx),
                    flops=4.0 * T * H * K, what=f"peer forward T={T} H={H} E={E} K={K}", repeat=5)


@pytest.mark.parametrize("case", pick(PKM_CASES))
def test_pkm_forward_throughput(case):
    """Case list of the reference's tests/test_pkm.py:170-181."""
    from flash_moe.ops.triton.pkm import triton_pkm_func
    from test_peer_pkm_gpu import pkm_reference

    T, H, E, K = case
    _, values, _, idx, w = expert_inputs(T, H, E, K, torch.bfloat16)
    chunk = max(1, (1 << 28) // (K * H))
    with torch.no_grad():
        harness.run([harness.Impl(harness.BASELINE, chunked(pkm_reference, chunk, (1, 2))),
                     harness.Impl(harness.HIP, triton_pkm_func)], lambda: (values, w, idx),
                    flops=2.0 * T * H * K, what=f"pkm forward T={T} H={H} E={E} K={K}", repeat=5)
