"""Parity of the HIP product-key router with the CPU oracle, through the op (and so the C ABI)."""
import numpy as np
import pytest
import torch

from helpers import cuda
from oracle import bruteforce as bf
from oracle import flashmoe_oracle as orc

pytestmark = pytest.mark.gpu


def oracle_topk_chunked(lp, nk, K, chunk=512):
    s, i = [], []
    for lo in range(0, lp.shape[1], chunk):
        a, b = orc.router_topk(lp[:, lo:lo + chunk].contiguous(), nk, K)
        s.append(a); i.append(b)
    return torch.cat(s), torch.cat(i)


def check_fp32_case(lp, nk, K):
    from flash_moe.ops import flash_router_func

    T = lp.shape[1]
    scores, idx = flash_router_func(cuda(lp), nk, K)
    assert scores.shape == (T, K) and idx.shape == (T, K)
    assert scores.dtype == torch.float32 and idx.dtype == torch.int64
    scores, idx = scores.cpu(), idx.cpu()
    # one extra rank from the oracle tells where the cut is a tie
    Kx = min(K + 1, nk * nk)
    o_scores, o_idx = oracle_topk_chunked(lp, nk, Kx)
    # the K largest sums, bit for bit, in descending order
    assert torch.equal(scores, o_scores[:, :K])
    # every index reproduces its score exactly, is in range and distinct within the token
    again = lp[0].gather(-1, idx // nk) + lp[1].gather(-1, idx % nk)
    assert torch.equal(again, scores)
    assert idx.min() >= 0 and idx.max() < nk * nk
    assert (idx.sort(-1).values.diff(dim=-1) != 0).all()
    # index sets equal the oracle's except where the K-th and (K+1)-th sums are closer than 1e-6
    same = (idx.sort(-1).values == o_idx[:, :K].sort(-1).values).all(-1)
    if Kx > K:
        tie_at_cut = (o_scores[:, K - 1] - o_scores[:, K]).abs() < 1e-6
        assert (same | tie_at_cut).all(), f"{(~(same | tie_at_cut)).sum().item()} tokens differ without a tie"
    else:
        assert same.all()
    # where no two of the K+1 best sums tie, the order is the oracle's too
    strict = (o_scores[:, :-1] - o_scores[:, 1:] > 0).all(-1) if Kx > 1 else torch.ones(T, dtype=torch.bool)
    assert torch.equal(idx[strict], o_idx[:, :K][strict])
    return scores, idx


@pytest.mark.parametrize("T,nk,K", [
    (4096, 64, 8), (4096, 128, 16),            # shapes of the reference's router test (tests/test_router.py:78-79)
    (512, 32, 16),                             # C1
    (8192, 128, 64),                           # C2
    (300, 512, 128),                           # C5 keys, few tokens
    (77, 100, 37), (5, 13, 13), (64, 8, 1), (33, 256, 200), (1, 128, 64), (1030, 64, 64),
    # every top-k kernel variant: lists in registers (nk <= 128 or <= 512, K <= 64 or <= 128) and the group scan beyond
    (200, 128, 128), (150, 512, 64), (40, 300, 100), (64, 600, 64), (48, 520, 128),
    # more than four tokens per SIMD: the instances compiled for eight waves per SIMD (C2 above is one; C5 in the block tests)
    (4200, 128, 100), (4200, 320, 48), (4200, 512, 128),
    # top_k beyond 256, up to num_keys as the reference allows (flash_router.py:261-263): the workgroup-per-token kernel
    (24, 512, 512), (20, 300, 257), (12, 1024, 1000), (600, 400, 320),
    # beyond what sorts in LDS (top_k > 1024, or > 256 with more than 8192 keys): radix selection, up to top_k 4096
    (5, 2048, 1500), (3, 9000, 300), (2, 4096, 4096), (40, 1100, 1100),
])
def test_router_fp32_log_probs(T, nk, K):
    check_fp32_case(orc.make_router_inputs(T, nk, seed=T + nk), nk, K)


def test_router_fp32_raw_normals():
    # the reference's own router benchmark feeds raw normals, not log-probabilities (tests/test_router.py:43-46)
    check_fp32_case(orc.make_router_inputs(2048, 128, seed=0, log_probs=False), 128, 16)


def test_router_matches_exhaustive_scan_with_lowest_index_ties():
    # quantised scores force many exact ties; the exhaustive C scan breaks them to the lowest flat index,
    # the rule of the reference kernel (tl.argmax).  Scores must agree exactly; indices may differ only
    # inside a group of equal sums that straddles the cut.
    from flash_moe.ops import flash_router_func

    T, nk, K = 200, 32, 16
    lp = (orc.make_router_inputs(T, nk, seed=3) * 2).round() / 2
    s, i = flash_router_func(cuda(lp), nk, K)
    b_s, b_i = bf.router_topk(lp.numpy(), nk, K)
    assert np.array_equal(s.cpu().numpy(), b_s)
    i = i.cpu()
    again = lp[0].gather(-1, i // nk) + lp[1].gather(-1, i % nk)
    assert torch.equal(again, s.cpu())
    above_cut = torch.from_numpy(b_s) > torch.from_numpy(b_s[:, -1:])
    for t in range(T):
        want = set(b_i[t][above_cut[t].numpy()].tolist())      # strictly better than the K-th sum: forced
        assert want <= set(i[t].tolist())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_router_16bit_scores(dtype):
    # sums are rounded to the input dtype as the reference adds in the input dtype (flash_router.py:51-53)
    from flash_moe.ops import flash_router_func

    T, nk, K = 1024, 128, 64
    lp = orc.make_router_inputs(T, nk, seed=1).to(dtype)
    s, i = flash_router_func(cuda(lp), nk, K)
    assert s.dtype == dtype
    s, i = s.cpu(), i.cpu()
    o_s, _ = oracle_topk_chunked(lp, nk, K)
    assert torch.equal(s, o_s)                                   # same multiset of rounded sums, same order
    again = lp[0].gather(-1, i // nk) + lp[1].gather(-1, i % nk)
    assert torch.equal(again, s)
    assert (i.sort(-1).values.diff(dim=-1) != 0).all()


@pytest.mark.parametrize("norm", [False, True])
def test_router_gates(norm):
    from flash_moe.ops.hip.flash_router import router_topk_gates

    T, nk, K = 777, 128, 64
    lp = orc.make_router_inputs(T, nk, seed=2)
    s, i, g = router_topk_gates(cuda(lp), nk, K, with_gates=True, norm_topk_prob=norm)
    ref = orc.routing_weights(s.cpu(), norm)
    torch.testing.assert_close(g.cpu(), ref, rtol=1e-5, atol=1e-9)
    if norm:
        torch.testing.assert_close(g.sum(-1).cpu(), torch.ones(T), rtol=1e-5, atol=1e-5)


def test_router_limits_of_the_large_top_k_kernel():
    from flash_moe.ops import flash_router_func

    with pytest.raises(ValueError, match="top_k"):
        flash_router_func(torch.zeros(2, 2, 8192, device="cuda"), 8192, 4097)          # beyond 4096


def test_router_noncontiguous_input_and_empty():
    from flash_moe.ops import flash_router_func

    T, nk, K = 64, 32, 8
    lp = orc.make_router_inputs(T, nk, seed=4)
    view = cuda(lp.transpose(0, 1).contiguous()).transpose(0, 1)   # [2,T,nk] view of [T,2,nk], as in the module
    assert not view.is_contiguous()
    s, i = flash_router_func(view, nk, K)
    s2, i2 = flash_router_func(cuda(lp), nk, K)
    assert torch.equal(s, s2) and torch.equal(i, i2)
    s0, i0 = flash_router_func(cuda(lp), nk, 0)
    assert s0.shape == (T, 0) and i0.shape == (T, 0)
    se, ie = flash_router_func(torch.empty(2, 0, nk, device="cuda"), nk, K)
    assert se.shape == (0, K)


# ------------------------------------------------------------------------------------------------
# the block's fused routing stage (batch-norm -> gate -> log-softmax -> top-k -> gates)
# ------------------------------------------------------------------------------------------------
def _fused(x, wr, nk, K, norm_flag, dtype, training=True, rm=None, rv=None):
    from flash_moe.ops.hip.flash_router import router_forward

    H = x.shape[1]
    bn = torch.nn.BatchNorm1d(H, affine=False)
    if rm is not None:
        bn.running_mean.copy_(rm); bn.running_var.copy_(rv)
    bn = bn.to(device="cuda", dtype=dtype)
    bn.train(training)
    out = router_forward(x.to(dtype).cuda(), wr.to(dtype).cuda(), bn, nk, K, norm_flag, return_logits32=True)
    return out, bn


@pytest.mark.parametrize("T,H,nk,K", [(512, 256, 32, 16), (1000, 1024, 128, 64), (130, 72, 100, 37), (64, 2048, 512, 128),
                                      (40, 256, 320, 300),
                                      (24, 128, 1200, 1100)])     # top_k beyond 1024: the radix-selection kernel, from logits
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_fused_router_matches_oracle_prologue(T, H, nk, K, dtype):
    g = torch.Generator().manual_seed(T + nk)
    x = (torch.randn(T, H, generator=g) * 1.7 + 0.3).to(dtype)
    wr = (torch.randn(2 * nk, H, generator=g) * 0.02).to(dtype)
    (logits, scores, indices, gates, logits32), bn = _fused(x.float(), wr.float(), nk, K, False, dtype)
    assert logits.shape == (T, 2 * nk) and logits.dtype == dtype and logits32.dtype == torch.float32
    # oracle: batch-norm as torch runs it in this dtype, the rest in fp32 on those values
    rm, rv = torch.zeros(H, dtype=dtype), torch.ones(H, dtype=dtype)
    q = torch.nn.functional.batch_norm(x, rm, rv, None, None, True, 0.1, 1e-5)
    ref32 = torch.nn.functional.linear(q.float(), wr.float())
    tol = {torch.float32: 1e-4, torch.bfloat16: 2e-2, torch.float16: 2e-2}[dtype]
    torch.testing.assert_close(logits.float().cpu(), ref32.to(dtype).float(), rtol=tol, atol=tol)
    # fp32 logits against the CPU oracle: its 16-bit batch-norm keeps mean and 1/std in 16 bits, so the normalised
    # activations differ by a 16-bit rounding
    fro = ((logits32.cpu() - ref32).norm() / ref32.norm()).item()
    assert fro < {torch.float32: 1e-5, torch.bfloat16: 6e-3, torch.float16: 1e-3}[dtype], fro
    # ... and against torch's batch-norm on this device (fp32 statistics, the routine the reference module calls):
    # only a rare one-ulp difference of a normalised activation remains
    q_dev = torch.nn.functional.batch_norm(x.cuda(), None, None, None, None, True, 0.1, 1e-5)
    ref_dev = torch.nn.functional.linear(q_dev.float().cpu(), wr.float())
    fro = ((logits32.cpu() - ref_dev).norm() / ref_dev.norm()).item()
    assert fro < {torch.float32: 1e-5, torch.bfloat16: 5e-4, torch.float16: 1e-4}[dtype], fro
    # running statistics follow nn.BatchNorm1d (momentum 0.1, unbiased variance), counter incremented
    torch.testing.assert_close(bn.running_mean.float().cpu(), rm.float(), rtol=2e-2, atol=2e-3)
    torch.testing.assert_close(bn.running_var.float().cpu(), rv.float(), rtol=2e-2, atol=2e-3)
    assert int(bn.num_batches_tracked) == 1
    # routing stage on identical input: oracle log-softmax + top-k of the fp32 logits the kernel produced
    lp = torch.log_softmax(logits32.cpu().view(T, 2, nk), -1).transpose(0, 1).contiguous()
    o_s, o_i = oracle_topk_chunked(lp, nk, min(K + 1, nk * nk))
    torch.testing.assert_close(scores.cpu(), o_s[:, :K], rtol=0, atol=2e-6)
    same = (indices.cpu().sort(-1).values == o_i[:, :K].sort(-1).values).all(-1)
    tie = (o_s[:, K - 1] - o_s[:, K]).abs() < 2e-6 if o_s.shape[1] > K else torch.zeros(T, dtype=torch.bool)
    assert (same | tie).all()
    g_tol = {torch.float32: 1e-5, torch.bfloat16: 8e-3, torch.float16: 1e-3}[dtype]
    # fp16 gates below 6.1e-5 are subnormal: their spacing is 6e-8 whatever the value
    g_atol = 6e-8 if dtype == torch.float16 else 1e-10
    torch.testing.assert_close(gates.float().cpu(), orc.routing_weights(o_s[:, :K], False), rtol=g_tol, atol=g_atol)


def test_fused_router_eval_mode_and_normalised_gates():
    T, H, nk, K = 300, 128, 64, 32
    g = torch.Generator().manual_seed(5)
    x = torch.randn(T, H, generator=g) * 2 + 1
    wr = torch.randn(2 * nk, H, generator=g) * 0.05
    rm, rv = torch.randn(H, generator=g), torch.rand(H, generator=g) + 0.5
    (logits, scores, indices, gates, logits32), bn = _fused(x, wr, nk, K, True, torch.float32, training=False, rm=rm, rv=rv)
    ref_logits, ref_lp = orc.router_prologue(x, wr, nk, rm.clone(), rv.clone(), training=False)
    torch.testing.assert_close(logits.cpu().view(T, 2, nk).transpose(0, 1), ref_logits, rtol=1e-4, atol=1e-4)
    # the buffers are untouched in eval mode
    torch.testing.assert_close(bn.running_mean.cpu(), rm, rtol=0, atol=0)
    torch.testing.assert_close(bn.running_var.cpu(), rv, rtol=0, atol=0)
    assert int(bn.num_batches_tracked) == 0
    torch.testing.assert_close(gates.sum(-1).cpu(), torch.ones(T), rtol=1e-5, atol=1e-5)
    o_s, o_i = orc.router_topk(ref_lp, nk, K)
    overlap = sum(len(set(a.tolist()) & set(b.tolist())) for a, b in zip(indices.cpu(), o_i)) / o_i.numel()
    assert overlap > 0.999


def test_fused_router_statistics_are_stable_for_offset_data():
    # a large common offset must not cancel in the variance
    T, H, nk, K = 2048, 64, 16, 4
    g = torch.Generator().manual_seed(6)
    x = torch.randn(T, H, generator=g) * 0.01 + 100.0
    wr = torch.randn(2 * nk, H, generator=g)
    (logits, *_), bn = _fused(x, wr, nk, K, False, torch.float32)
    ref_logits, _ = orc.router_prologue(x.double(), wr.double(), nk)
    err = (logits.cpu().double().view(T, 2, nk).transpose(0, 1) - ref_logits).abs().max().item()
    assert err < 2e-2 * ref_logits.abs().max().item(), err


def test_fused_router_rejects_single_token_in_training():
    from flash_moe.ops.hip.flash_router import router_forward

    bn = torch.nn.BatchNorm1d(64, affine=False).cuda()
    with pytest.raises(ValueError, match="more than 1 value per channel"):
        router_forward(torch.randn(1, 64, device="cuda"), torch.randn(16, 64, device="cuda"), bn, 8, 4)
    bn.eval()
    out = router_forward(torch.randn(1, 64, device="cuda"), torch.randn(16, 64, device="cuda"), bn, 8, 4)
    assert out[2].shape == (1, 4)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,H,nk,K", [(8192, 1024, 128, 64), (300, 256, 64, 16)])
def test_split_query_router_equals_a_block_diagonal_gate(dtype, T, H, nk, K):
    """Two sub-key tables [nk, H/2], each scoring its own half of the query (the router benchmark configuration as worded),
    against the general routing stage with the block-diagonal gate they stand for: the zero blocks add exact zeros, so
    logits, scores and indices agree bit for bit; and the logits against the oracle's prologue on that gate."""
    from flash_moe.ops.hip.flash_router import router_forward

    g = torch.Generator().manual_seed(T + H)
    x = (torch.randn(T, H, generator=g) * 1.2 + 0.1).to(dtype)
    tables = (torch.randn(2 * nk, H // 2, generator=g) * 0.02).to(dtype)
    dense = torch.zeros(2 * nk, H, dtype=dtype)
    dense[:nk, : H // 2] = tables[:nk]
    dense[nk:, H // 2:] = tables[nk:]

    def run(weight, split):
        bn = torch.nn.BatchNorm1d(H, affine=False).to(device="cuda", dtype=dtype)
        return router_forward(x.cuda(), weight.cuda(), bn, nk, K, True, return_logits32=True, split_query=split), bn

    (logits, scores, indices, gates, logits32), bn = run(tables, True)
    (d_logits, d_scores, d_indices, d_gates, d_logits32), d_bn = run(dense, False)
    assert torch.equal(logits32, d_logits32) and torch.equal(logits, d_logits)
    assert torch.equal(scores, d_scores) and torch.equal(indices, d_indices) and torch.equal(gates, d_gates)
    assert torch.equal(bn.running_mean, d_bn.running_mean) and torch.equal(bn.running_var, d_bn.running_var)
    ref_logits, _ = orc.router_prologue(x.float(), dense.float(), nk)
    tol = {torch.float32: 1e-4, torch.bfloat16: 2e-2, torch.float16: 2e-2}[dtype]
    torch.testing.assert_close(logits.float().cpu().view(T, 2, nk).transpose(0, 1), ref_logits, rtol=tol, atol=tol)
    # each half only sees its half of the query: changing the other half of x leaves its logits untouched (eval mode,
    # so that the statistics of the untouched columns stay what they were)
    x2 = x.clone()
    x2[:, H // 2:] += 1.0
    bn_e = torch.nn.BatchNorm1d(H, affine=False).to(device="cuda", dtype=dtype).eval()
    a = router_forward(x.cuda(), tables.cuda(), bn_e, nk, K, False, return_logits32=True, split_query=True)[4]
    b = router_forward(x2.cuda(), tables.cuda(), bn_e, nk, K, False, return_logits32=True, split_query=True)[4]
    assert torch.equal(a[:, :nk], b[:, :nk]) and not torch.equal(a[:, nk:], b[:, nk:])
