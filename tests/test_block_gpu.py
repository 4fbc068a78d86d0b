"""Whole-block parity: FlashMoE (HIP path) against the CPU oracle of FlashMoE_Pytorch.forward."""
import pytest
import torch

from helpers import assert_mostly_close, assert_output_close, cuda, rel_fro
from oracle import flashmoe_oracle as orc

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def fused_forward_path():
    """These tests are about the fused forward, which the module takes when no gradient is being recorded."""
    with torch.no_grad():
        yield


def build(H, I, E, K, norm, dtype, seed=0, std=0.02):
    from flash_moe.modules.flash_moe import FlashMoE, FlashMoEConfig

    w = orc.make_block_weights(H, I, E, seed=seed, std=std).to(dtype)
    m = FlashMoE(FlashMoEConfig(H, I, "silu", E, K, norm))
    m.load_state_dict({"gate_proj.weight": w.gate_proj, "up_proj.weight": w.up_proj, "down_proj.weight": w.down_proj,
                       "router_gate.weight": w.router_gate, "down_embed.weight": w.down_embed,
                       "up_embed.weight": w.up_embed}, strict=False)
    return m.to(device="cuda", dtype=dtype), w


def stagewise_check(m, w, x, K, norm, dtype):
    """End-to-end comparison plus a stage-by-stage one that feeds the oracle the HIP path's own
    intermediates, so that one flipped near-tie in the router cannot hide or fake an error downstream."""
    H = x.shape[-1]
    T = x.shape[0] * x.shape[1]
    nk = w.num_keys
    y, logits = m(x.cuda())
    assert y.shape == x.shape and y.dtype == dtype and logits.shape == (2, T, nk) and logits.dtype == dtype
    w.running_mean.zero_(); w.running_var.fill_(1.0)
    ref = orc.block_forward(x, w, K, norm_topk_prob=norm, training=True, routing_fp32=True, token_chunk=256)
    assert_output_close(logits, ref["router_logits"], dtype, "router_logits")
    outliers = 0.0
    if dtype == torch.float32:
        assert_output_close(y, ref["y"], dtype, "block output")
    else:
        outliers = assert_mostly_close(y, ref["y"], dtype, "block output vs same-dtype oracle")
    # running statistics follow nn.BatchNorm1d
    torch.testing.assert_close(m.router_norm.running_mean.float().cpu(), w.running_mean.float(), rtol=2e-2, atol=1e-3)
    torch.testing.assert_close(m.router_norm.running_var.float().cpu(), w.running_var.float(), rtol=2e-2, atol=1e-3)

    # stage by stage on the HIP path's intermediates
    m.router_norm.reset_running_stats()
    tokens = x.cuda().view(-1, H)
    _, scores, indices, gates, logits32 = m.route(tokens, return_logits32=True)
    idx_cpu, gates_cpu = indices.cpu(), gates.float().cpu()
    # router stage on identical input: the oracle's log-softmax and top-k of the HIP path's own fp32 gate output
    lp_cpu = torch.log_softmax(logits32.cpu().view(T, 2, nk), dim=-1).transpose(0, 1).contiguous()
    Kx = K + 1
    o_s = torch.cat([orc.router_topk(lp_cpu[:, lo:lo + 256].contiguous(), nk, Kx)[0] for lo in range(0, T, 256)])
    o_i = torch.cat([orc.router_topk(lp_cpu[:, lo:lo + 256].contiguous(), nk, Kx)[1] for lo in range(0, T, 256)])
    torch.testing.assert_close(scores.cpu(), o_s[:, :K], rtol=0, atol=2e-6)     # log-softmax differs in the last ulp
    set_equal = (idx_cpu.sort(-1).values == o_i[:, :K].sort(-1).values).all(-1)
    tie_at_cut = (o_s[:, K - 1] - o_s[:, K]).abs() < 2e-6
    assert (set_equal | tie_at_cut).all()
    g_tol = {torch.float32: 1e-5, torch.bfloat16: 8e-3, torch.float16: 1e-3}[dtype]
    torch.testing.assert_close(gates_cpu, orc.routing_weights(o_s[:, :K], norm), rtol=g_tol, atol=1e-10)
    # end to end the selection is chaotic: a one-ulp difference in a 16-bit batch-norm output moves a logit
    # by ~1e-4 and can swap the experts around the cut, so only the overlap with the oracle's sets is bounded
    hit = torch.tensor([len(set(a.tolist()) & set(b.tolist())) for a, b in zip(idx_cpu, ref["indices"])]).float()
    same = (hit / K).mean().item()
    assert same > (0.999 if dtype == torch.float32 else 0.97), f"mean overlap with the oracle's expert sets {same:.4f}"
    # experts: oracle on the HIP path's own indices and gates
    from flash_moe.ops.hip.flash_expert import expert_forward

    e_hip = expert_forward(tokens, m.down_embed.weight, m.up_embed.weight, indices, gates).cpu()
    e_ref = orc.expert_forward(x.view(-1, H).double(), w.down_embed.double(), w.up_embed.double(), idx_cpu,
                               gates.cpu().double(), token_chunk=256)
    fro = rel_fro(e_hip, e_ref)
    assert fro < {torch.float32: 2e-6, torch.bfloat16: 4e-3, torch.float16: 1e-3}[dtype], f"experts: {fro:.3e}"
    # block output against a float64 evaluation of MLP + experts on the HIP path's own routing: only the
    # HIP path's two roundings (the [T,I] activation and the result) remain, so the bar holds everywhere
    y64 = orc.mlp_forward(x.view(-1, H).double(), w.gate_proj.double(), w.up_proj.double(), w.down_proj.double()) + e_hip.double()
    assert_output_close(y.view(-1, H), y64.to(dtype), dtype, "block output vs float64 oracle")
    return dict(overlap_fp32_routing=same, outlier_fraction=outliers, indices=idx_cpu)


@pytest.mark.parametrize("norm", [False, True])
def test_block_c1_fp32(norm):
    # C1: fp32, 1 x 512 tokens, H=256, I=1024, E=1024 (32x32 keys), K=16
    m, w = build(256, 1024, 1024, 16, norm, torch.float32)
    x = torch.randn(1, 512, 256, generator=torch.Generator().manual_seed(0))
    stagewise_check(m, w, x, 16, norm, torch.float32)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_block_c4_shape_fewer_tokens(dtype):
    # C4 weights (H=1024, I=4096, E=16384, K=64) on 512 tokens so that the CPU oracle finishes in seconds
    m, w = build(1024, 4096, 16384, 64, False, dtype)
    x = torch.randn(1, 512, 1024, generator=torch.Generator().manual_seed(0)).to(dtype)
    res = stagewise_check(m, w, x, 64, False, dtype)
    # How far the expert sets are from the reference's literal 16-bit routing (logits, log-softmax and pair sums all
    # rounded to the dtype, where many sums tie and the choice among ties is the library's): measured, and bounded
    # from below so that a regression of the routing shows.
    w.running_mean.zero_(); w.running_var.fill_(1.0)
    literal = orc.block_forward(x, w, 64, norm_topk_prob=False, training=True, routing_fp32=False, token_chunk=256)
    hit = torch.tensor([len(set(a.tolist()) & set(b.tolist())) for a, b in zip(res["indices"], literal["indices"])]).float()
    overlap_literal = (hit / 64).mean().item()
    print(f"\n[{dtype}] 512 tokens of C4: expert-set overlap with the oracle's fp32 routing {res['overlap_fp32_routing']:.4f}, "
          f"with its literal 16-bit routing {overlap_literal:.4f}; elements of y outside rtol = atol = 2e-2 against the "
          f"same-dtype oracle: {res['outlier_fraction']:.2e} (budget 1e-4)")
    assert res["outlier_fraction"] <= 1e-4
    assert overlap_literal > 0.5, overlap_literal


def test_block_c4_full_size_properties():
    # C4 at full size (README configuration): structure and size-independent properties
    dtype = torch.bfloat16
    m, w = build(1024, 4096, 16384, 64, False, dtype)
    x = torch.randn(1, 4096, 1024, generator=torch.Generator().manual_seed(0)).to(dtype).cuda()
    y, logits = m(x)
    assert y.shape == (1, 4096, 1024) and logits.shape == (2, 4096, 128)
    assert torch.isfinite(y).all() and torch.isfinite(logits).all()
    m.eval()
    y1, _ = m(x)
    y2, _ = m(x)
    assert torch.equal(y1, y2)                               # deterministic
    # in eval mode tokens are independent: a slice of the batch gives the same rows
    ys, _ = m(x[:, 1000:1512])
    assert rel_fro(ys, y1[:, 1000:1512]) < 1e-3
    # block = shared MLP + routed experts
    from flash_moe.ops import flash_mlp_func
    from flash_moe.ops.hip.flash_expert import expert_forward

    tokens = x.view(-1, 1024)
    _, _, indices, gates = m.route(tokens)
    parts = flash_mlp_func(tokens, m.gate_proj.weight, m.up_proj.weight, m.down_proj.weight).float() + expert_forward(
        tokens, m.down_embed.weight, m.up_embed.weight, indices, gates).float()
    assert rel_fro(y1.view(-1, 1024), parts) < 6e-3
    # gates are probabilities p_x * p_y of distinct experts
    assert (gates > 0).all() and (gates.sum(-1) <= 1 + 1e-3).all()
    assert (indices.sort(-1).values.diff(dim=-1) != 0).all() and indices.max() < 16384


def test_block_c5_shape_fewer_tokens():
    # C5 weights scaled to fit a quick run: H=2048, I=8192, 512x512 keys, K=128, normalised gates, 256 tokens
    dtype = torch.bfloat16
    m, w = build(2048, 8192, 262144, 128, True, dtype)
    x = torch.randn(1, 256, 2048, generator=torch.Generator().manual_seed(0)).to(dtype)
    stagewise_check(m, w, x, 128, True, dtype)


def test_block_with_more_than_256_experts_per_token():
    # num_experts_per_tok may be anything up to the number of keys in the reference (flash_router.py:261-263); beyond 256
    # the router takes its workgroup-per-token kernel
    m, w = build(256, 512, 320 * 320, 300, True, torch.float32)
    x = torch.randn(1, 48, 256, generator=torch.Generator().manual_seed(0))
    stagewise_check(m, w, x, 300, True, torch.float32)


def test_block_with_long_rows():
    # hidden_size 5120: rows of 10240 bytes, longer than one wavefront's registers hold; the expert stage takes column slices
    dtype = torch.bfloat16
    m, w = build(5120, 1024, 1024, 8, False, dtype)
    x = torch.randn(1, 40, 5120, generator=torch.Generator().manual_seed(0)).to(dtype)
    stagewise_check(m, w, x, 8, False, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,H,I,E,K", [(1024, 256, 512, 4096, 64),     # column-slice expert schedule
                                       (96, 128, 256, 1024, 8),        # row-gather expert schedule
                                       (33, 64, 192, 400, 5)])         # ragged: E not a square, odd T and K
@pytest.mark.parametrize("training", [True, False])
def test_single_call_block_equals_the_three_stage_calls(dtype, T, H, I, E, K, training):
    """fmoe_block_forward runs the same kernels as router -> expert -> mlp called one by one: bit-identical."""
    from flash_moe.ops.hip.flash_block import block_forward

    m, _ = build(H, I, E, K, True, dtype, seed=3)
    m.train(training)
    x = torch.randn(1, T, H, generator=torch.Generator().manual_seed(5)).to(dtype).cuda()
    y1, l1 = m(x)
    stats1 = (m.router_norm.running_mean.clone(), m.router_norm.running_var.clone(), int(m.router_norm.num_batches_tracked))
    m.router_norm.reset_running_stats()
    y2, l2 = m.forward_staged(x)
    assert torch.equal(y1, y2) and torch.equal(l1, l2)
    assert torch.equal(stats1[0], m.router_norm.running_mean) and torch.equal(stats1[1], m.router_norm.running_var)
    assert stats1[2] == int(m.router_norm.num_batches_tracked) == (1 if training else 0)
    m.router_norm.reset_running_stats()
    _, _, idx_ref, gates_ref = m.route(x.view(T, H))
    m.router_norm.reset_running_stats()
    y3, _, idx, gates = block_forward(x.view(T, H), m.gate_proj.weight, m.up_proj.weight, m.down_proj.weight,
                                      m.router_gate.weight, m.router_norm, m.down_embed.weight, m.up_embed.weight,
                                      m.num_keys, K, True, return_routing=True)
    assert torch.equal(idx, idx_ref) and torch.equal(gates, gates_ref) and torch.equal(y3.view_as(y1), y1)


def test_single_call_block_without_routed_experts():
    """num_experts_per_tok = 0: the block is the shared MLP alone."""
    from flash_moe.ops.hip.flash_mlp import mlp_forward

    m, _ = build(128, 256, 1024, 0, False, torch.bfloat16, seed=1)
    x = torch.randn(2, 32, 128, generator=torch.Generator().manual_seed(2)).to(torch.bfloat16).cuda()
    y, logits = m(x)
    ref = mlp_forward(x.view(-1, 128), m.gate_proj.weight, m.up_proj.weight, m.down_proj.weight)
    assert torch.equal(y.view(-1, 128), ref) and logits.shape == (2, 64, 32)


def test_block_c5_full_size_sampled_tokens():
    """C5 at full size (32768 tokens, two 1 GiB tables, top-128, normalised gates), evaluation mode so that tokens are
    independent: the single call equals the staged calls bit for bit, and 48 sampled tokens are checked stage by stage
    against the oracle (router on the HIP path's fp32 gate output, experts + MLP in float64 on its routing)."""
    from flash_moe.modules.flash_moe import FlashMoE, FlashMoEConfig
    from flash_moe.ops.hip.flash_block import block_forward

    dtype, T, H, I, E, K, nk = torch.bfloat16, 32768, 2048, 8192, 262144, 128, 512
    with torch.device("cuda"):
        m = FlashMoE(FlashMoEConfig(H, I, "silu", E, K, True)).to(dtype)
    g = torch.Generator(device="cuda").manual_seed(0)
    with torch.no_grad():
        for p in m.parameters():
            p.normal_(0.0, 0.02, generator=g)
        m.router_norm.running_mean.normal_(0.0, 0.1, generator=g)
        m.router_norm.running_var.uniform_(0.5, 1.5, generator=g)
    m.eval()
    x = torch.randn(8, 4096, H, device="cuda", generator=g).to(dtype)
    tokens = x.view(T, H)
    y, logits, indices, gates = block_forward(tokens, m.gate_proj.weight, m.up_proj.weight, m.down_proj.weight,
                                              m.router_gate.weight, m.router_norm, m.down_embed.weight, m.up_embed.weight,
                                              nk, K, True, return_routing=True)
    assert torch.isfinite(y).all() and torch.isfinite(logits).all()
    y2, logits2 = m.forward_staged(x)
    assert torch.equal(y.view_as(y2), y2) and torch.equal(logits.view(T, 2, nk).transpose(0, 1), logits2)
    assert int(m.router_norm.num_batches_tracked) == 0
    torch.testing.assert_close(gates.float().sum(-1), torch.ones(T, device="cuda"), rtol=0, atol=2e-2)
    assert (indices.sort(-1).values.diff(dim=-1) != 0).all() and 0 <= int(indices.min()) and int(indices.max()) < E

    pick = torch.randperm(T, generator=torch.Generator().manual_seed(1))[:48].sort().values.cuda()
    xs = tokens[pick]
    _, s_scores, s_idx, s_gates, s_logits32 = m.route(xs, return_logits32=True)
    assert torch.equal(s_idx, indices[pick]) and torch.equal(s_gates, gates[pick])          # tokens are independent
    # router: the oracle's exhaustive top-k of the HIP path's own fp32 gate output
    lp = torch.log_softmax(s_logits32.cpu().view(-1, 2, nk), dim=-1).transpose(0, 1).contiguous()
    o_s, o_i = orc.router_topk(lp, nk, K + 1)
    torch.testing.assert_close(s_scores.cpu(), o_s[:, :K], rtol=0, atol=2e-6)
    set_equal = (s_idx.cpu().sort(-1).values == o_i[:, :K].sort(-1).values).all(-1)
    assert (set_equal | ((o_s[:, K - 1] - o_s[:, K]).abs() < 2e-6)).all()
    torch.testing.assert_close(s_gates.float().cpu(), orc.routing_weights(o_s[:, :K], True), rtol=8e-3, atol=1e-10)
    # experts + MLP in float64 on the sampled tokens, with only the table rows they use
    rows, remap = torch.unique(s_idx, return_inverse=True)
    wd_s, wu_s = m.down_embed.weight[rows].cpu().double(), m.up_embed.weight[rows].cpu().double()
    e64 = orc.expert_forward(xs.cpu().double(), wd_s, wu_s, remap.cpu(), s_gates.cpu().double())
    y64 = e64 + orc.mlp_forward(xs.cpu().double(), m.gate_proj.weight.cpu().double(), m.up_proj.weight.cpu().double(),
                                m.down_proj.weight.cpu().double())
    assert_output_close(y[pick], y64.to(dtype), dtype, "C5 block output vs float64 oracle on sampled tokens")


def test_block_c5_full_size_train_mode_batch_statistics():
    """C5 at full size in training mode: the batch statistics over all 32768 tokens (what couples the tokens) against
    float64 column statistics, the running-statistics update, and 32 sampled tokens through router, experts and MLP
    against the oracle fed those statistics."""
    from flash_moe.modules.flash_moe import FlashMoE, FlashMoEConfig
    from flash_moe.ops.hip.flash_block import block_forward
    from flash_moe.ops.hip.flash_router import router_forward

    dtype, T, H, I, E, K, nk = torch.bfloat16, 32768, 2048, 8192, 262144, 128, 512
    with torch.device("cuda"):
        m = FlashMoE(FlashMoEConfig(H, I, "silu", E, K, True)).to(dtype)
    g = torch.Generator(device="cuda").manual_seed(3)
    with torch.no_grad():
        for p in m.parameters():
            p.normal_(0.0, 0.02, generator=g)
    m.train()
    x = (torch.randn(8, 4096, H, device="cuda", generator=g) * 1.3 + 0.2).to(dtype)
    tokens = x.view(T, H)
    # statistics: mean and 1/sqrt(var + eps) the kernels normalise with, against float64
    out = router_forward(tokens, m.router_gate.weight, m.router_norm, nk, K, True, return_logits32=True, return_stats=True)
    logits, scores, indices, gates, logits32, stats = out
    mean64, var64 = tokens.double().mean(0), tokens.double().var(0, unbiased=False)
    torch.testing.assert_close(stats[:H].double(), mean64, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(stats[H:].double(), (var64 + 1e-5).rsqrt(), rtol=1e-5, atol=0)
    assert int(m.router_norm.num_batches_tracked) == 1
    torch.testing.assert_close(m.router_norm.running_mean.double(), 0.1 * mean64, rtol=2e-2, atol=2e-3)
    torch.testing.assert_close(m.router_norm.running_var.double(), 0.9 + 0.1 * var64 * T / (T - 1), rtol=2e-2, atol=2e-3)
    # the block in training mode: single call equals the staged routing on the same statistics
    m.router_norm.reset_running_stats()
    y, b_logits, b_idx, b_gates = block_forward(tokens, m.gate_proj.weight, m.up_proj.weight, m.down_proj.weight,
                                                m.router_gate.weight, m.router_norm, m.down_embed.weight, m.up_embed.weight,
                                                nk, K, True, return_routing=True)
    assert torch.equal(b_idx, indices) and torch.equal(b_gates, gates) and torch.equal(b_logits, logits)
    assert torch.isfinite(y).all()
    # sampled tokens: gate logits from the normalised activations rounded to bf16, as a stand-alone batch-norm emits them
    pick = torch.randperm(T, generator=torch.Generator().manual_seed(2))[:32].sort().values.cuda()
    xs = tokens[pick]
    q = ((xs.float() - stats[:H]) * stats[H:]).to(dtype)
    ref32 = q.float() @ m.router_gate.weight.float().t()
    assert rel_fro(logits32[pick], ref32) < 5e-4
    lp = torch.log_softmax(logits32[pick].cpu().view(-1, 2, nk), dim=-1).transpose(0, 1).contiguous()
    o_s, o_i = orc.router_topk(lp, nk, K + 1)
    torch.testing.assert_close(scores[pick].cpu(), o_s[:, :K], rtol=0, atol=2e-6)
    set_equal = (indices[pick].cpu().sort(-1).values == o_i[:, :K].sort(-1).values).all(-1)
    assert (set_equal | ((o_s[:, K - 1] - o_s[:, K]).abs() < 2e-6)).all()
    s_idx, s_gates = indices[pick], gates[pick]
    rows, remap = torch.unique(s_idx, return_inverse=True)
    wd_s, wu_s = m.down_embed.weight[rows].cpu().double(), m.up_embed.weight[rows].cpu().double()
    e64 = orc.expert_forward(xs.cpu().double(), wd_s, wu_s, remap.cpu(), s_gates.cpu().double())
    y64 = e64 + orc.mlp_forward(xs.cpu().double(), m.gate_proj.weight.cpu().double(), m.up_proj.weight.cpu().double(),
                                m.down_proj.weight.cpu().double())
    assert_output_close(y[pick], y64.to(dtype), dtype, "C5 train-mode block output vs float64 oracle on sampled tokens")


def test_block_of_an_empty_batch():
    m, _ = build(128, 256, 1024, 8, False, torch.bfloat16)
    m.eval()
    y, logits = m(torch.zeros(2, 0, 128, device="cuda", dtype=torch.bfloat16))
    assert y.shape == (2, 0, 128) and logits.shape == (2, 0, 32)


@pytest.mark.parametrize("T", [64, 1024])
def test_block_forward_under_hip_graph_capture(T):
    """The single-call forward only launches kernels on the caller's stream (no allocation, no memset, no host
    synchronisation inside the library), so it can be captured in a HIP graph: every replay equals the eager result."""
    dtype = torch.bfloat16
    m, _ = build(256, 512, 4096, 16, True, dtype, seed=4)
    m.eval()
    static_x = torch.randn(1, T, 256, generator=torch.Generator().manual_seed(1)).to(dtype).cuda()
    eager = [m(static_x)[0].clone()]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            m(static_x)                                  # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_y, static_logits = m(static_x)
    for step in range(3):
        new_x = torch.randn(1, T, 256, generator=torch.Generator().manual_seed(10 + step)).to(dtype).cuda()
        expect, expect_logits = m(new_x)                  # eager work between the replays
        torch.cuda.synchronize()
        static_x.copy_(new_x)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(static_y, expect) and torch.equal(static_logits, expect_logits), f"replay {step}"
