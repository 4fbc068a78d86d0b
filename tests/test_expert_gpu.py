"""Parity of the HIP routed-expert op with the CPU oracle, through the op (and so the C ABI)."""
import pytest
import torch

from helpers import assert_output_close, cuda, rel_fro
from oracle import flashmoe_oracle as orc

pytestmark = pytest.mark.gpu


ALGOS = {"auto": 0, "rows": 1, "slices": 2, "buckets": 3}
SCHEDULES = ["rows", "slices", "buckets"]


def run(x, wd, wu, idx, g, algo="auto"):
    from flash_moe.ops.hip.flash_expert import expert_forward

    return expert_forward(*cuda(x, wd, wu, idx, g), algo=ALGOS[algo]).cpu()


def truth64(x, wd, wu, idx, g):
    """The oracle evaluated in float64 on the (already rounded) inputs."""
    return orc.expert_forward(x.double(), wd.double(), wu.double(), idx, g.double())


@pytest.mark.parametrize("algo", SCHEDULES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,H,E,K", [
    (512, 256, 1024, 16),        # C1
    (1024, 1024, 16384, 64),     # C3 / C4 row shape, fewer tokens
    (256, 2048, 4096, 128),      # C5 row shape
    (37, 72, 50, 5),             # ragged: rows of 9 packets, token count not a multiple of the block
    (3, 8, 4, 1),
    (130, 1000, 300, 70),        # K not a multiple of the 64 pairs a wave handles per round; last slice partial
    (200, 264, 20000, 40),       # more than 16384 rows: the narrower (128-byte) column slices, last one partial
])
def test_expert_matches_oracle(dtype, T, H, E, K, algo):
    x, wd, wu, idx, g = orc.make_expert_inputs(T, H, E, K, seed=T + K)
    x, wd, wu, g = (t.to(dtype) for t in (x, wd, wu, g))
    if algo == "buckets" and (H * x.element_size()) % 128 != 0:
        # the bucketed schedule works on whole 128-byte column bands: forcing it on other rows is refused
        with pytest.raises(ValueError, match="bucketed schedule"):
            run(x, wd, wu, idx, g, algo)
        return
    got = run(x, wd, wu, idx, g, algo)
    assert got.dtype == dtype and got.shape == (T, H)
    # (1) the stated bar: against the oracle run in the same dtype
    assert_output_close(got, orc.expert_forward(x, wd, wu, idx, g), dtype, "expert vs oracle")
    # (2) against the float64 evaluation of the same rounded inputs: only the final rounding remains
    fro = rel_fro(got, truth64(x, wd, wu, idx, g))
    assert fro < {torch.float32: 2e-6, torch.bfloat16: 4e-3, torch.float16: 5e-4}[dtype], fro


@pytest.mark.parametrize("dtype,H", [(torch.bfloat16, 8192), (torch.bfloat16, 5120), (torch.float16, 4104), (torch.float32, 2304)])
def test_expert_long_rows_take_the_column_slices(dtype, H):
    # rows of more than 8192 bytes do not fit the registers of the one-wave-per-token kernel: the op takes the column-slice
    # kernels for them whatever the problem size (the reference has no limit on hidden_size); forcing rows is refused
    T, E, K = 24, 96, 6
    x, wd, wu, idx, g = orc.make_expert_inputs(T, H, E, K, seed=H)
    x, wd, wu, g = (t.to(dtype) for t in (x, wd, wu, g))
    got = run(x, wd, wu, idx, g, "auto")
    assert_output_close(got, orc.expert_forward(x, wd, wu, idx, g), dtype, "expert, long rows")
    fro = rel_fro(got, truth64(x, wd, wu, idx, g))
    assert fro < {torch.float32: 2e-6, torch.bfloat16: 4e-3, torch.float16: 5e-4}[dtype], fro
    with pytest.raises(ValueError, match="elements per row"):
        run(x, wd, wu, idx, g, "rows")


@pytest.mark.parametrize("algo", ["slices", "auto"])
def test_expert_single_token_with_an_ill_conditioned_score(algo):
    """One token, rows of 3136 fp32 elements, 3 of 7 experts: the pair that carries 96 % of the gate has a score of
    -0.016 that is the sum of 3136 products whose absolute values sum to 39, so any fp32 summation of it is uncertain by
    eps * 39 = 2e-6 absolute, 1.5e-4 relative, and that error reaches the output through silu'(s) * gate.  Every fp32
    evaluation (this op in any schedule, the oracle run in fp32) lands a few 1e-6 from the float64 result in relative
    Frobenius norm, above the bar the well-conditioned cases meet (2e-6).  The bar here comes from the condition of the
    scores: a quarter of the worst-case bound for one rounding per product."""
    x, wd, wu, idx, g = orc.make_expert_inputs(1, 3136, 7, 3, seed=54)
    xd, wdd, wud, gd = x.double(), wd.double(), wu.double(), g.double()
    prod = xd[0][None, :] * wdd[idx[0]]
    s, s_abs = prod.sum(-1), prod.abs().sum(-1)
    assert float((s_abs / s.abs()).max()) > 1e3                       # the case is what the docstring says it is
    sig = torch.sigmoid(s)
    dsilu = sig * (1 + s * (1 - sig))
    err_coef = dsilu.abs() * gd[0] * s_abs * 2.0 ** -24               # |d out coefficient| for one ulp of each product
    ref = truth64(x, wd, wu, idx, g)
    bound = float(((err_coef[:, None] * wud[idx[0]].abs()).sum(0).norm() / ref.norm()))
    bar = 2e-6 + 0.25 * bound
    assert 5e-6 < bar < 5e-5, bar
    got = run(x, wd, wu, idx, g, algo)
    fro, fro_oracle32 = rel_fro(got, ref), rel_fro(orc.expert_forward(x, wd, wu, idx, g), ref)
    print(f"\nill-conditioned score: HIP ({algo}) {fro:.2e}, fp32 oracle {fro_oracle32:.2e}, bar {bar:.2e}")
    assert fro < bar and fro_oracle32 < bar
    assert_output_close(got, orc.expert_forward(x, wd, wu, idx, g), torch.float32, "expert, ill-conditioned score")


@pytest.mark.parametrize("algo", SCHEDULES)
def test_expert_reference_test_distribution(algo):
    # distributions of the reference's expert benchmark (tests/test_expert.py:160-175): x ~ N(0,0.5),
    # tables ~ N(0,0.1), ids drawn WITH replacement, gates ~ N(0,0.1) (negative values allowed)
    g0 = torch.Generator().manual_seed(0)
    T, H, E, K = 256, 1024, 4096, 512
    x = (torch.randn(T, H, generator=g0) * 0.5).bfloat16()
    wd = (torch.randn(E, H, generator=g0) * 0.1).bfloat16()
    wu = (torch.randn(E, H, generator=g0) * 0.1).bfloat16()
    idx = torch.randint(0, E, (T, K), generator=g0)
    g = (torch.randn(T, K, generator=g0) * 0.1).bfloat16()
    got = run(x, wd, wu, idx, g, algo)
    assert rel_fro(got, truth64(x, wd, wu, idx, g)) < 4e-3


@pytest.mark.parametrize("algo", SCHEDULES)
def test_expert_properties_full_size(algo):
    # C3 at full size: size-independent properties instead of a CPU evaluation of all 1M pairs
    import functools

    T, H, E, K = 16384, 1024, 16384, 64
    x, wd, wu, idx, g = orc.make_expert_inputs(T, H, E, K, seed=0)
    x, wd, wu, g = (t.bfloat16() for t in (x, wd, wu, g))
    xc, wdc, wuc, idxc, gc = cuda(x, wd, wu, idx, g)
    from flash_moe.ops.hip.flash_expert import expert_forward

    flash_expert_func = functools.partial(expert_forward, algo=ALGOS[algo])
    out = flash_expert_func(xc, wdc, wuc, idxc, gc)
    assert torch.isfinite(out).all()
    # deterministic: no atomics, so a second run is bit-identical
    assert torch.equal(out, flash_expert_func(xc, wdc, wuc, idxc, gc))
    # zero gates -> exact zeros (also proves the output is written, not accumulated into)
    assert flash_expert_func(xc, wdc, wuc, idxc, torch.zeros_like(gc)).abs().max() == 0
    # linear in the gates (power-of-two factor: exact in bf16)
    assert torch.equal(flash_expert_func(xc, wdc, wuc, idxc, gc * 2), out * 2)
    # permuting the K slots of every token only changes the fp32 summation order
    perm = torch.randperm(K, generator=torch.Generator().manual_seed(1)).cuda()
    out_p = flash_expert_func(xc, wdc, wuc, idxc[:, perm].contiguous(), gc[:, perm].contiguous())
    assert rel_fro(out_p, out) < 4e-3
    # a slice of tokens against the oracle
    sl = slice(5000, 5512)
    assert_output_close(out[sl].cpu(), orc.expert_forward(x[sl], wd, wu, idx[sl], g[sl]), torch.bfloat16, "C3 slice")
    assert rel_fro(out[sl].cpu(), truth64(x[sl], wd, wu, idx[sl], g[sl])) < 4e-3


def test_expert_schedules_agree():
    # the schedules on the same inputs: same pairs, different summation order (and, for bf16, the
    # slice schedule rounds silu(s)*g to bf16 before the packed dot product)
    T, H, E, K = 2048, 1024, 16384, 64
    x, wd, wu, idx, g = orc.make_expert_inputs(T, H, E, K, seed=9)
    for dtype, tol in ((torch.float32, 2e-6), (torch.bfloat16, 5e-3)):
        args = tuple(t.to(dtype) if t.is_floating_point() else t for t in (x, wd, wu, idx, g))
        rows = run(*args, algo="rows")
        assert rel_fro(run(*args, algo="slices"), rows) < tol
        assert rel_fro(run(*args, algo="buckets"), rows) < tol


def test_expert_large_table_takes_the_bucketed_schedule():
    """A table far beyond what the column-slice schedule keeps in L2: with about a dozen pairs per expert or more the
    default schedule is the bucketed one (each table row then serves many pairs), with fewer it gathers whole rows.
    Both against the oracle (on a sample of the tokens: tokens are independent) and against each other."""
    from flash_moe import _C

    lib = _C.lib()
    H, E, K = 256, 131072, 128
    T = 12 * E // K                                    # 12 pairs per expert
    assert lib.fmoe_expert_workspace_bytes(T, H, E, K, _C.BF16) == lib.fmoe_expert_workspace_bytes_algo(
        T, H, E, K, _C.BF16, _C.EXPERT_BUCKETS) > 0
    assert lib.fmoe_expert_workspace_bytes(T // 2, H, E, K, _C.BF16) == 0          # 6 pairs per expert: whole rows
    x, wd, wu, idx, g = orc.make_expert_inputs(T, H, E, K, seed=21)
    x, wd, wu, g = (t.bfloat16() for t in (x, wd, wu, g))
    got = run(x, wd, wu, idx, g, "auto")
    assert torch.equal(got, run(x, wd, wu, idx, g, "buckets"))
    assert rel_fro(got, run(x, wd, wu, idx, g, "rows")) < 4e-3
    sample = torch.arange(0, T, 37)
    xs, ids, gs = x[sample], idx[sample], g[sample]
    assert_output_close(got[sample], orc.expert_forward(xs, wd, wu, ids, gs), torch.bfloat16, "bucketed schedule vs oracle")
    assert rel_fro(got[sample], truth64(xs, wd, wu, ids, gs)) < 4e-3
    few = run(x[: T // 2], wd, wu, idx[: T // 2], g[: T // 2], "auto")
    assert torch.equal(few, run(x[: T // 2], wd, wu, idx[: T // 2], g[: T // 2], "rows"))


@pytest.mark.parametrize("algo", SCHEDULES)
def test_expert_duplicates_and_single_expert(algo):
    T, H, E = 64, 256, 32
    x, wd, wu, _, _ = orc.make_expert_inputs(T, H, E, 4, seed=5, std=0.2)
    e = torch.full((T, 4), 7, dtype=torch.int64)
    one = run(x, wd, wu, e[:, :1].contiguous(), torch.ones(T, 1), algo)
    rep = run(x, wd, wu, e, torch.full((T, 4), 0.25), algo)
    torch.testing.assert_close(rep, one, rtol=1e-5, atol=1e-7)
    s = x @ wd[7]
    torch.testing.assert_close(one, (torch.nn.functional.silu(s)).unsqueeze(-1) * wu[7], rtol=1e-4, atol=1e-6)


@pytest.mark.parametrize("algo", SCHEDULES)
def test_expert_out_of_range_ids_contribute_nothing(algo):
    T, H, E, K = 32, 64, 16, 4
    x, wd, wu, idx, g = orc.make_expert_inputs(T, H, E, K, seed=6, std=0.2)
    bad = idx.clone()
    bad[:, 0] = E + 3
    bad[::2, 1] = -1
    g2 = g.clone()
    g2[:, 0] = 0
    g2[::2, 1] = 0
    wd[0] = float("inf")   # the slice schedule reads row 0 as a stand-in for an invalid id: it must not leak
    wu[0] = float("nan")
    idx[idx == 0] = 1
    bad[bad == 0] = 1
    got = run(x, wd, wu, bad, g, algo)
    assert torch.isfinite(got).all()
    torch.testing.assert_close(got, run(x, wd, wu, idx, g2, algo), rtol=1e-6, atol=1e-8)


@pytest.mark.parametrize("E", [1000, 5000, 70000])
def test_expert_bucketed_grouping_by_partition_with_a_hot_expert_and_invalid_ids(E):
    """From 65536 pairs on the bucketed schedule groups the pairs with two partition passes (coarse buckets of 1, 8 and 128
    experts here, the last one partial): one expert chosen six times by every token (12288 pairs: more than a workgroup
    orders in LDS), ids outside [0, E) in two columns, fp32 against the row schedule and the float64 oracle."""
    T, H, K = 2048, 128, 32
    x, wd, wu, idx, g = orc.make_expert_inputs(T, H, E, K, seed=31, std=0.3)
    idx[:, 0] = 3
    idx[:, 4:9] = 3
    idx[::3, 1] = E + 5
    idx[1::4, 2] = -1
    idx[:, 3] = E - 1
    got = run(x, wd, wu, idx, g, "buckets")
    assert torch.isfinite(got).all() and torch.equal(got, run(x, wd, wu, idx, g, "buckets"))
    assert rel_fro(got, run(x, wd, wu, idx, g, "rows")) < 2e-6
    valid = (idx >= 0) & (idx < E)
    ref = truth64(x, wd, wu, idx.clamp(0, E - 1), g * valid)
    assert rel_fro(got, ref) < 2e-6


def test_expert_bucketed_grouping_with_the_largest_coarse_buckets():
    """Six million experts (rows of 128 bytes): the partition passes use coarse buckets of 2^13 experts, whose counters
    fill 32 KiB of a workgroup's LDS, and the second phase is the row kernel (the table is beyond the sweep's key range).
    Against the row schedule on the GPU and, for a sample of tokens, the float64 oracle on the rows those tokens use."""
    from flash_moe.ops.hip.flash_expert import expert_forward

    T, H, E, K = 2048, 64, 6_000_000, 32
    g0 = torch.Generator(device="cuda").manual_seed(5)
    x = (torch.randn(T, H, device="cuda", generator=g0) * 0.5).bfloat16()
    wd = (torch.randn(E, H, device="cuda", generator=g0) * 0.3).bfloat16()
    wu = (torch.randn(E, H, device="cuda", generator=g0) * 0.3).bfloat16()
    idx = torch.randint(0, E, (T, K), device="cuda", generator=g0)
    idx[:, 0] = E - 1                      # the last (partial) coarse bucket, chosen by every token
    idx[::5, 1] = E                        # out of range
    idx[:, 2] = idx[:, 3]                  # duplicates add
    g = torch.rand(T, K, device="cuda", generator=g0).bfloat16()
    got = expert_forward(x, wd, wu, idx, g, algo=ALGOS["buckets"])
    assert torch.isfinite(got).all() and torch.equal(got, expert_forward(x, wd, wu, idx, g, algo=ALGOS["buckets"]))
    rows = expert_forward(x, wd, wu, idx, g, algo=ALGOS["rows"])
    assert rel_fro(got.cpu(), rows.cpu()) < 4e-3
    sample = torch.arange(0, T, 97, device="cuda")
    ids = idx[sample]
    valid = (ids >= 0) & (ids < E)
    used, inverse = torch.unique(ids.clamp(0, E - 1), return_inverse=True)
    ref = orc.expert_forward(x[sample].double().cpu(), wd[used].double().cpu(), wu[used].double().cpu(), inverse.cpu(),
                             (g[sample].double() * valid).cpu())
    assert rel_fro(got[sample].cpu(), ref) < 4e-3


def test_expert_empty_and_noncontiguous():
    from flash_moe.ops import flash_expert_func

    T, H, E, K = 16, 64, 16, 4
    x, wd, wu, idx, g = cuda(*orc.make_expert_inputs(T, H, E, K, seed=7))
    assert flash_expert_func(x[:0], wd, wu, idx[:0], g[:0]).shape == (0, H)
    z = flash_expert_func(x, wd, wu, idx[:, :0], g[:, :0])
    assert z.shape == (T, H) and z.abs().max() == 0
    xt = x.t().contiguous().t()
    assert not xt.is_contiguous()
    assert torch.equal(flash_expert_func(xt, wd, wu, idx, g), flash_expert_func(x, wd, wu, idx, g))


def test_expert_on_router_produced_ids_at_the_block_size():
    """Ids as the block's router emits them (4096 tokens, 128 x 128 product keys, top-64: structured, not uniformly random)
    through every schedule, against the oracle on a sample of tokens and against each other."""
    from flash_moe.ops import flash_router_func

    T, H, nk, K = 4096, 1024, 128, 64
    E = nk * nk
    lp = orc.make_router_inputs(T, nk, seed=17)
    scores, idx = flash_router_func(lp.cuda(), nk, K)
    idx = idx.cpu()
    assert int(idx.min()) >= 0 and int(idx.max()) < E
    g = torch.exp(scores.cpu()).bfloat16()
    x, wd, wu, _, _ = orc.make_expert_inputs(T, H, E, K, seed=18)
    x, wd, wu = (t.bfloat16() for t in (x, wd, wu))
    outs = {algo: run(x, wd, wu, idx, g, algo) for algo in SCHEDULES}
    sample = torch.arange(0, T, 16)
    ref = truth64(x[sample], wd, wu, idx[sample], g[sample])
    for algo, out in outs.items():
        assert rel_fro(out[sample], ref) < 4e-3, algo
        assert_output_close(out[sample], orc.expert_forward(x[sample], wd, wu, idx[sample], g[sample]), torch.bfloat16, algo)
    assert rel_fro(outs["slices"], outs["rows"]) < 5e-3 and rel_fro(outs["buckets"], outs["rows"]) < 5e-3
