#!/usr/bin/env python3
"""Benchmark of the FlashMoE forward path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline]

A step is one forward pass of the FlashMoE block (README configuration: bf16, batch 1 x seq 4096,
hidden 1024, intermediate 4096, 16384 experts, top-64, norm_topk_prob False) over one synthetic batch
that is already resident in HBM.  The last line printed is one JSON object:

  value          tokens/s of the whole block: 4096 tokens / ms_per_step, the median over the K timed steps of the HIP-event
                 time of one step (step_ms has min / median / max / mean; wall_ms_per_step is the host clock over the K steps)
  stages_us      median duration of each C-ABI call of the block, one HIP-event pair per call on the launch stream
                 (stages_spread_us: min / median / max / mean)
  roofline       the slowest C-ABI call of the block (its kernels are named in `launches`) against the roofline
                 that bounds it; rooflines_all has every call
  expert_c3      the routed-expert kernel alone on its own benchmark shape (16384 tokens), as HBM GB/s
  router_c2      the routing stage alone on the router benchmark shape: module semantics (every half scores the full
                 query) and the configuration as worded (two sub-key tables on the two halves of the query)
  block_c5       the largest block (32768 tokens, 262144 experts), with its stages and the expert op's roofline entry
  block_c1       the reference's CPU-runnable configuration (fp32, 512 tokens, 1024 experts) on the GPU, next to cpu_baseline_c1
  mlp_fp32       the shared MLP of the same shape in fp32 (v_mfma_f32_32x32x2_f32) against the dense fp32 matrix peak
  cpu_baseline   the CPU restatement of the reference's eager path (oracle/) on the same block, timed on
                 this machine's host cores; cpu_baseline_c1 / cpu_baseline_c4_fp32: the reference's own CPU
                 configuration (fp32, 512 tokens) and the README block in fp32
  `traffic` figures are fabric-side bytes per launch (L2 misses, whether the Infinity Cache or HBM serves them) from
  rocprofv3 FETCH_SIZE / WRITE_SIZE runs kept under profiles/; the calibration is stated in traffic_source.

Only one GPU is used; --gpus N with N > 1 exits with a message.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "flash-moe_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16
MFMA_FP32_PEAK_TFLOPS = 157.3   # MI355X dense fp32 matrix

C1 = dict(batch=1, seq=512, hidden=256, inter=1024, experts=1024, top_k=16, norm=False)
C4 = dict(batch=1, seq=4096, hidden=1024, inter=4096, experts=16384, top_k=64, norm=False)
C3 = dict(tokens=16384, hidden=1024, experts=16384, top_k=64)
C2 = dict(tokens=8192, hidden=1024, keys=128, top_k=64)
C5 = dict(batch=8, seq=4096, hidden=2048, inter=8192, experts=262144, top_k=128, norm=True)


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def synthetic_block(cfg, dtype, device):
    """FlashMoE module with seeded N(0, 0.02) weights and a seeded N(0, 1) input."""
    import torch

    from flash_moe.modules.flash_moe import FlashMoE, FlashMoEConfig

    g = torch.Generator(device="cpu").manual_seed(0)
    m = FlashMoE(FlashMoEConfig(cfg["hidden"], cfg["inter"], "silu", cfg["experts"], cfg["top_k"], cfg["norm"]))
    with torch.no_grad():
        for p in m.parameters():
            p.copy_(torch.randn(p.shape, generator=g) * 0.02)
    x = torch.randn(cfg["batch"], cfg["seq"], cfg["hidden"], generator=g)
    return m.to(device=device, dtype=dtype), x.to(device=device, dtype=dtype)


def event_times_ms(fn, iters, warmup=3):
    """Duration of each of `iters` back-to-back calls of fn(), from one HIP-event pair per call on the current stream
    (the calls are queued without host synchronisation in between; one synchronisation at the end)."""
    import torch

    for _ in range(warmup):
        fn()
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
    torch.cuda.synchronize()
    for start, stop in pairs:
        start.record()
        fn()
        stop.record()
    torch.cuda.synchronize()
    return [start.elapsed_time(stop) for start, stop in pairs]


def spread(times_ms, scale=1e3, digits=2):
    """min / median / max / mean of a list of durations (ms), scaled (default: to microseconds)."""
    return dict(min=round(min(times_ms) * scale, digits), median=round(statistics.median(times_ms) * scale, digits),
                max=round(max(times_ms) * scale, digits), mean=round(statistics.fmean(times_ms) * scale, digits))


def event_time_ms(fn, iters, warmup=3):
    """Median duration of fn() over `iters` back-to-back calls (one HIP-event pair per call)."""
    return statistics.median(event_times_ms(fn, iters, warmup))


def expert_bytes(T, H, K, touched, elt):
    """Algorithmic bytes of the routed-expert op: x in and out, each touched down/up row once,
    int64 indices and gates."""
    return 2 * T * H * elt + 2 * touched * H * elt + T * K * (8 + elt)


def stage_kernels(m, x):
    """Callables that launch exactly one stage each through the C ABI (no allocation inside)."""
    import torch

    from flash_moe import _C

    L = _C.lib()
    dev = x.device
    stream = lambda: _C.current_stream(dev)
    tokens = x.view(-1, m.hidden_size)
    T, H, I, K, nk = tokens.shape[0], m.hidden_size, m.intermediate_size, m.top_k, m.num_keys
    code = _C.dtype_code(x.dtype)
    from flash_moe.ops.hip.flash_router import router_forward

    was_training = m.training
    m.eval()   # keep the running statistics untouched while setting up
    with torch.no_grad():
        _, _, _, _, logits32 = router_forward(tokens, m.router_gate.weight, m.router_norm, nk, K, m.norm_topk_prob, True)
    m.train(was_training)
    lp = torch.log_softmax(logits32.view(T, 2, nk), dim=-1).transpose(0, 1).contiguous()
    scores = torch.empty(T, K, device=dev, dtype=torch.float32)
    indices = torch.empty(T, K, device=dev, dtype=torch.int64)
    gates32 = torch.empty(T, K, device=dev, dtype=torch.float32)
    L.fmoe_router_topk(lp.data_ptr(), T, nk, K, _C.F32, scores.data_ptr(), indices.data_ptr(), gates32.data_ptr(),
                       int(m.norm_topk_prob), stream())
    gates = gates32.to(x.dtype)
    experts = torch.empty_like(tokens)
    act = torch.empty(T, I, device=dev, dtype=x.dtype)
    out = torch.empty_like(tokens)
    wd_t, wu_t = m.down_embed.weight, m.up_embed.weight
    E = wd_t.shape[0]
    ws_bytes = L.fmoe_expert_workspace_bytes(T, H, E, K, code)
    ws = torch.empty(max(ws_bytes, 1), device=dev, dtype=torch.uint8)

    def check(rc):
        if rc != 0:
            raise RuntimeError(L.fmoe_last_error().decode())

    # the fused router (batch statistics, finalize, normalise + gate GEMM, top-k): running statistics are given as
    # NULL so that timing it does not drift the module's buffers
    r_logits = torch.empty(T, 2 * nk, device=dev, dtype=x.dtype)
    r_logits32 = torch.empty(T, 2 * nk, device=dev, dtype=torch.float32)
    r_gates = torch.empty(T, K, device=dev, dtype=x.dtype)
    r_ws_bytes = L.fmoe_router_workspace_bytes(T, H, nk)
    r_ws = torch.empty(max(r_ws_bytes, 1), device=dev, dtype=torch.uint8)
    gate_w = m.router_gate.weight

    fns = {
        "router_forward": lambda: check(L.fmoe_router_forward(
            tokens.data_ptr(), gate_w.data_ptr(), None, None, None, code, 1, 0.1, 1e-5, T, H, nk, K, code,
            int(m.norm_topk_prob), r_logits.data_ptr(), r_logits32.data_ptr(), scores.data_ptr(), indices.data_ptr(),
            r_gates.data_ptr(), r_ws.data_ptr(), r_ws_bytes, stream())),
        "router_topk": lambda: check(L.fmoe_router_topk(lp.data_ptr(), T, nk, K, _C.F32, scores.data_ptr(),
                                                        indices.data_ptr(), gates32.data_ptr(),
                                                        int(m.norm_topk_prob), stream())),
        "expert": lambda: check(L.fmoe_expert_forward(tokens.data_ptr(), wd_t.data_ptr(), wu_t.data_ptr(),
                                                      indices.data_ptr(), gates.data_ptr(), T, H, E, K, code,
                                                      experts.data_ptr(), ws.data_ptr(), ws_bytes, stream())),
        "mlp_gate_up": lambda: check(L.fmoe_mlp_gate_up(tokens.data_ptr(), m.gate_proj.weight.data_ptr(),
                                                        m.up_proj.weight.data_ptr(), T, H, I, code, act.data_ptr(),
                                                        stream())),
        "mlp_down": lambda: check(L.fmoe_mlp_down(act.data_ptr(), m.down_proj.weight.data_ptr(), T, H, I, code,
                                                  experts.data_ptr(), out.data_ptr(), stream())),
    }
    touched = int(torch.unique(indices).numel())
    elt = x.element_size()
    work = {
        "router_forward": dict(bound="hbm", bytes=T * H * elt + 2 * nk * H * elt + T * 2 * nk * (elt + 4) + T * K * (4 + 8 + elt),
                               flops=2 * T * H * 2 * nk),
        "router_topk": dict(bound="hbm", bytes=2 * T * nk * 4 + T * K * (4 + 8 + 4)),
        "expert": dict(bound="hbm", bytes=expert_bytes(T, H, K, touched, elt), touched_experts=touched),
        "mlp_gate_up": dict(bound="mfma", flops=2 * T * H * 2 * I),
        "mlp_down": dict(bound="mfma", flops=2 * T * I * H),
    }
    keep = (lp, scores, indices, gates32, gates, experts, act, out, ws, r_logits, r_logits32, r_gates, r_ws)
    return fns, work, keep


# kernels behind each timed C-ABI call, as they appear in the rocprofv3 summaries under profiles/
LAUNCHES = {
    "router_forward": ["bn_block_stats_kernel", "router_gate_kernel", "router_select_kernel"],
    "router_topk": ["router_select_kernel"],
    "expert": ["expert_scores_slice_kernel", "expert_gate_kernel", "expert_states_slice_kernel"],
    "expert_c5": ["partition_count_kernel", "bucket_scan_kernel", "partition_scatter_kernel", "partition_local_kernel",
                  "expert_band_copy_kernel", "expert_scores_bucketed_kernel", "expert_gate_sorted_kernel",
                  "expert_owner_sort_kernel", "expert_states_sweep_kernel"],
    "mlp_gate_up": ["gemm_dma_kernel<256x256 tiles, SwiGLU epilogue>"],
    "mlp_down": ["gemm_dma_kernel<128x128 tiles, residual epilogue>"],
}


def roofline_entry(name, ms, w, traffic, launches=None, spread_us=None):
    if w["bound"] == "hbm":
        achieved = w["bytes"] / (ms * 1e-3) / 1e9
        peak, unit = HBM_PEAK_GBS, "GB/s"
    else:
        achieved = w["flops"] / (ms * 1e-3) / 1e12
        peak, unit = MFMA_BF16_PEAK_TFLOPS, "TFLOP/s"
    entry = dict(kernel=name, launches=LAUNCHES.get(launches or name, [name]), bound=w["bound"], achieved=round(achieved, 2),
                 peak=peak, unit=unit, frac=round(achieved / peak, 4), avg_launch_us=round(ms * 1e3, 2),
                 algorithmic=w.get("bytes", w.get("flops")), traffic=traffic)
    if spread_us is not None:
        entry["median_launch_us"], entry["min_launch_us"], entry["max_launch_us"] = (spread_us["median"], spread_us["min"],
                                                                                      spread_us["max"])
    clock = measured_traffic(name, "clock_ghz_c4")
    if clock is not None:
        # shader clock while this kernel runs, from the kept counter summary (profiles/mlp_c4_counters.txt): the peak above
        # is quoted at 2.4 GHz
        entry["clock_ghz"] = clock
    if w["bound"] == "hbm" and "flops" in w:
        # a contraction below the MFMA ridge: the matrix-core fraction next to the binding (HBM) one
        tf = w["flops"] / (ms * 1e-3) / 1e12
        entry["mfma_TFLOPs"] = round(tf, 2)
        entry["mfma_frac"] = round(tf / MFMA_BF16_PEAK_TFLOPS, 4)
    return entry


TRAFFIC_SOURCE = ("fabric-side bytes per launch (L2 misses, served by the Infinity Cache or HBM) = 2.000 x FETCH_SIZE + 1.000 x "
                  "WRITE_SIZE in KiB per dispatch from two rocprofv3 --pmc runs; the factors are what the same counters read "
                  "for a 256 MiB device copy (profiles/hbm_traffic_counters.txt)")


def measured_traffic(kernel, workload):
    """Fabric-side bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs, if a summary is committed."""
    path = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    try:
        with open(path) as f:
            return json.load(f).get(workload, {}).get(kernel)
    except (OSError, ValueError):
        return None


def bench_expert_c3(dtype, iters):
    import torch

    from flash_moe import _C

    cfg = C3
    T, H, E, K = cfg["tokens"], cfg["hidden"], cfg["experts"], cfg["top_k"]
    g = torch.Generator(device="cpu").manual_seed(0)
    x = torch.randn(T, H, generator=g).to(dtype).cuda()
    wd = (torch.randn(E, H, generator=g) * 0.02).to(dtype).cuda()
    wu = (torch.randn(E, H, generator=g) * 0.02).to(dtype).cuda()
    gidx = torch.Generator(device="cuda").manual_seed(0)
    idx = torch.rand(T, E, device="cuda", generator=gidx).topk(K, dim=-1).indices.contiguous()   # K distinct ids per token
    gates = torch.softmax(torch.randn(T, K, generator=g), -1).to(dtype).cuda()
    out = torch.empty_like(x)
    L = _C.lib()
    code = _C.dtype_code(dtype)
    ws_bytes = L.fmoe_expert_workspace_bytes(T, H, E, K, code)
    ws = torch.empty(max(ws_bytes, 1), device="cuda", dtype=torch.uint8)
    stream = lambda: _C.current_stream(x.device)

    def run():
        rc = L.fmoe_expert_forward(x.data_ptr(), wd.data_ptr(), wu.data_ptr(), idx.data_ptr(), gates.data_ptr(), T, H,
                                   E, K, code, out.data_ptr(), ws.data_ptr(), ws_bytes, stream())
        if rc:
            raise RuntimeError(L.fmoe_last_error().decode())

    ms = event_time_ms(run, iters)
    touched = int(torch.unique(idx).numel())
    nbytes = expert_bytes(T, H, K, touched, x.element_size())
    gbs = nbytes / (ms * 1e-3) / 1e9
    return dict(workload=f"expert kernel only: bf16, {T} tokens, hidden {H}, {E} experts, top-{K}, distinct ids per token",
                avg_launch_us=round(ms * 1e3, 2), algorithmic_bytes=nbytes, touched_experts=touched,
                achieved_GBps=round(gbs, 1), peak_GBps=HBM_PEAK_GBS, frac=round(gbs / HBM_PEAK_GBS, 4),
                tokens_per_s=round(T / (ms * 1e-3)), traffic=measured_traffic("expert", "c3"))


def bench_router_c2(dtype, iters):
    """The routing stage alone on its own shape: the fused call (batch norm, gate, log-softmax, top-k, gates) and the
    top-k op on ready-made fp32 log-probabilities."""
    import torch

    from flash_moe import _C

    T, H, nk, K = C2["tokens"], C2["hidden"], C2["keys"], C2["top_k"]
    g = torch.Generator(device="cpu").manual_seed(0)
    x = torch.randn(T, H, generator=g).to(dtype).cuda()
    w = (torch.randn(2 * nk, H, generator=g) * 0.02).to(dtype).cuda()
    lp = torch.log_softmax(torch.randn(2, T, nk, generator=g), -1).cuda()
    L = _C.lib()
    code = _C.dtype_code(dtype)
    logits = torch.empty(T, 2 * nk, device="cuda", dtype=dtype)
    logits32 = torch.empty(T, 2 * nk, device="cuda", dtype=torch.float32)
    scores = torch.empty(T, K, device="cuda", dtype=torch.float32)
    indices = torch.empty(T, K, device="cuda", dtype=torch.int64)
    gates = torch.empty(T, K, device="cuda", dtype=dtype)
    ws_bytes = L.fmoe_router_workspace_bytes(T, H, nk)
    ws = torch.empty(max(ws_bytes, 1), device="cuda", dtype=torch.uint8)
    stream = lambda: _C.current_stream(x.device)

    def fused():
        rc = L.fmoe_router_forward(x.data_ptr(), w.data_ptr(), None, None, None, code, 1, 0.1, 1e-5, T, H, nk, K, code, 0,
                                   logits.data_ptr(), logits32.data_ptr(), scores.data_ptr(), indices.data_ptr(),
                                   gates.data_ptr(), ws.data_ptr(), ws_bytes, stream())
        if rc:
            raise RuntimeError(L.fmoe_last_error().decode())

    def topk():
        rc = L.fmoe_router_topk(lp.data_ptr(), T, nk, K, _C.F32, scores.data_ptr(), indices.data_ptr(), None, 0, stream())
        if rc:
            raise RuntimeError(L.fmoe_last_error().decode())

    # the configuration as worded: two sub-key tables [nk, H/2], each on its own half of the query
    w_split = (torch.randn(2 * nk, H // 2, generator=g) * 0.02).to(dtype).cuda()

    def split():
        rc = L.fmoe_router_forward_split(x.data_ptr(), w_split.data_ptr(), None, None, None, code, 1, 0.1, 1e-5, T, H, nk, K,
                                         code, 0, logits.data_ptr(), logits32.data_ptr(), scores.data_ptr(),
                                         indices.data_ptr(), gates.data_ptr(), ws.data_ptr(), ws_bytes, stream())
        if rc:
            raise RuntimeError(L.fmoe_last_error().decode())

    ms_fused, ms_topk, ms_split = event_time_ms(fused, iters), event_time_ms(topk, iters), event_time_ms(split, iters)
    elt = x.element_size()
    nbytes = T * H * elt + 2 * nk * H * elt + T * 2 * nk * elt + T * K * (elt + 8)
    nbytes_split = nbytes - nk * H * elt
    flops, flops_split = 2 * T * H * 2 * nk, T * H * 2 * nk
    return dict(workload=f"router only: bf16, {T} tokens, hidden {H}, 2x{nk} keys, top-{K}, train-mode batch norm",
                fused_us=round(ms_fused * 1e3, 2), topk_only_us=round(ms_topk * 1e3, 2),
                tokens_per_s=round(T / (ms_fused * 1e-3)), algorithmic_bytes=nbytes,
                achieved_GBps=round(nbytes / (ms_fused * 1e-3) / 1e9, 1), peak_GBps=HBM_PEAK_GBS,
                frac=round(nbytes / (ms_fused * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                gemm_TFLOPs=round(flops / (ms_fused * 1e-3) / 1e12, 2),
                mfma_frac=round(flops / (ms_fused * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
                as_worded=dict(workload=f"two sub-key tables {nk} x {H // 2}, each on its own half of the {H}-wide query "
                                        "(fmoe_router_forward_split)",
                               fused_us=round(ms_split * 1e3, 2), tokens_per_s=round(T / (ms_split * 1e-3)),
                               algorithmic_bytes=nbytes_split,
                               achieved_GBps=round(nbytes_split / (ms_split * 1e-3) / 1e9, 1),
                               frac=round(nbytes_split / (ms_split * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                               gemm_TFLOPs=round(flops_split / (ms_split * 1e-3) / 1e12, 2),
                               mfma_frac=round(flops_split / (ms_split * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4)))


def bench_block_c5(dtype, iters):
    """The largest single-GPU configuration: 262144 experts of width 2048 (two 1 GiB tables), top-128, renormalised."""
    import torch

    from flash_moe.modules.flash_moe import FlashMoE, FlashMoEConfig

    cfg = C5
    with torch.device("cuda"):
        m = FlashMoE(FlashMoEConfig(cfg["hidden"], cfg["inter"], "silu", cfg["experts"], cfg["top_k"], cfg["norm"])).to(dtype)
    g = torch.Generator(device="cuda").manual_seed(0)
    with torch.no_grad():
        for p in m.parameters():
            p.normal_(0.0, 0.02, generator=g)
    x = torch.randn(cfg["batch"], cfg["seq"], cfg["hidden"], device="cuda", generator=g).to(dtype)
    T = cfg["batch"] * cfg["seq"]
    with torch.no_grad():
        ms = event_time_ms(lambda: m(x), iters, warmup=2)
        fns, work, keep = stage_kernels(m, x)
        times = {n: event_time_ms(fn, iters, warmup=2) for n, fn in fns.items()}
    expert = roofline_entry("expert", times["expert"], work["expert"], measured_traffic("expert", "c5"), launches="expert_c5")
    expert["touched_experts"] = work["expert"]["touched_experts"]
    del keep, fns
    return dict(workload=f"C5 full block: bf16, {T} tokens, hidden {cfg['hidden']}, intermediate {cfg['inter']}, "
                         f"{cfg['experts']} experts, top-{cfg['top_k']}, norm_topk_prob True, train-mode batch norm",
                ms_per_step=round(ms, 3), tokens_per_s=round(T / (ms * 1e-3)),
                stages_us={n: round(t * 1e3, 1) for n, t in times.items()},
                expert=expert,
                mlp_TFLOPs=round(6 * T * cfg["hidden"] * cfg["inter"] / ((times["mlp_gate_up"] + times["mlp_down"]) * 1e-3) / 1e12, 1))


def bench_block_c1(iters):
    """The reference's own CPU-runnable configuration (fp32, 512 tokens, 1024 experts, top-16) on the GPU: launch-bound."""
    import torch

    m, x = synthetic_block(C1, torch.float32, "cuda:0")
    T = C1["batch"] * C1["seq"]
    with torch.no_grad():
        per_call = event_times_ms(lambda: m(x), iters, warmup=5)
    ms = statistics.median(per_call)
    return dict(workload=f"C1 full block: fp32, {T} tokens, hidden {C1['hidden']}, intermediate {C1['inter']}, "
                         f"{C1['experts']} experts, top-{C1['top_k']}, train-mode batch norm",
                ms_per_step=round(ms, 4), step_us=spread(per_call), tokens_per_s=round(T / (ms * 1e-3)))


def bench_mlp_fp32(iters):
    """The C4 shared MLP in fp32: both GEMMs on v_mfma_f32_32x32x2_f32, priced against the dense fp32 matrix peak."""
    import torch

    from flash_moe.ops.hip.flash_mlp import mlp_forward

    T, H, I = C4["batch"] * C4["seq"], C4["hidden"], C4["inter"]
    g = torch.Generator(device="cuda").manual_seed(0)
    x = torch.randn(T, H, device="cuda", generator=g)
    wg, wu = (torch.randn(I, H, device="cuda", generator=g) * 0.02 for _ in range(2))
    wd = torch.randn(H, I, device="cuda", generator=g) * 0.02
    per_call = event_times_ms(lambda: mlp_forward(x, wg, wu, wd), iters, warmup=3)
    ms = statistics.median(per_call)
    tf = 6.0 * T * H * I / (ms * 1e-3) / 1e12
    return dict(workload=f"C4 shared MLP in fp32: {T} tokens, hidden {H}, intermediate {I} (gate/up + down launches)",
                bound="mfma", dtype="f32", us=spread(per_call), achieved=round(tf, 1), peak=MFMA_FP32_PEAK_TFLOPS,
                unit="TFLOP/s", frac=round(tf / MFMA_FP32_PEAK_TFLOPS, 4))


def bench_backward_c4(dtype, iters):
    """Forward + backward of the C4 block through autograd (the differentiable composition of the three ops)."""
    import torch

    m, x = synthetic_block(C4, dtype, "cuda:0")
    wy = torch.randn_like(x)
    T = C4["batch"] * C4["seq"]

    def step():
        for p in m.parameters():
            p.grad = None
        y, _ = m(x.detach().requires_grad_(True))
        y.backward(wy)

    def forward_only():
        with torch.no_grad():
            m.forward_autograd(x)

    ms, ms_fwd = event_time_ms(step, iters, warmup=3), event_time_ms(forward_only, iters, warmup=3)
    return dict(workload="C4 block, forward + backward through autograd (train-mode batch norm), gradients of the input "
                         "and of every parameter", ms_per_step=round(ms, 3), tokens_per_s=round(T / (ms * 1e-3)),
                forward_autograd_ms=round(ms_fwd, 3))


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(cfg, dtype, budget_s=20.0, label="C4"):
    """The oracle's block forward on the same workload, on the host cores (checker timed as a baseline)."""
    import torch

    from oracle import flashmoe_oracle as orc

    threads = torch.get_num_threads()
    w = orc.make_block_weights(cfg["hidden"], cfg["inter"], cfg["experts"], seed=0).to(dtype)
    x = torch.randn(cfg["batch"], cfg["seq"], cfg["hidden"], generator=torch.Generator().manual_seed(0)).to(dtype)
    T = cfg["batch"] * cfg["seq"]
    times = []
    t_begin = time.perf_counter()
    with torch.no_grad():
        orc.block_forward(x, w, cfg["top_k"], cfg["norm"], token_chunk=512)   # warm-up
        while len(times) < 5 or (time.perf_counter() - t_begin < budget_s and len(times) < 50):
            t0 = time.perf_counter()
            orc.block_forward(x, w, cfg["top_k"], cfg["norm"], token_chunk=512)
            times.append(time.perf_counter() - t0)
            if time.perf_counter() - t_begin > 3 * budget_s:
                break
    med = statistics.median(times)
    return dict(value=round(T / med, 1), unit="tokens/s", cores=threads, kind="port",
                sample=f"whole {label} batch ({T} tokens, {str(dtype).replace('torch.', '')}), median of {len(times)} "
                       f"forward passes of the torch CPU restatement of FlashMoE_Pytorch.forward, {threads} threads "
                       f"of {os.cpu_count()} logical CPUs ({cpu_model()})",
                ms_per_step=round(med * 1e3, 2))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-c3", action="store_true")
    ap.add_argument("--only-c3", action="store_true", help="run only the routed-expert kernel on its own shape (for profiling)")
    ap.add_argument("--only-backward", action="store_true", help="run only forward + backward of the C4 block (for profiling)")
    ap.add_argument("--only-c5", action="store_true", help="run only the largest block (C5) and its stages (for profiling)")
    ap.add_argument("--no-extras", action="store_true", help="skip the router-only (C2) and largest-block (C5) side measurements")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run a 256 MiB device copy, as the known-size reference for FETCH_SIZE / WRITE_SIZE counters")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: --gpus {args.gpus} is not supported (the path is single-GPU: tokens would be "
              "split across devices with one all-reduce of the batch-norm statistics, or the tables sharded by expert)", file=sys.stderr)
        sys.exit(2)

    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a ROCm GPU", file=sys.stderr)
        sys.exit(1)
    from flash_moe import _C

    _C.lib()   # fail loudly here if the HIP library is missing
    dtype = torch.bfloat16
    torch.cuda.set_device(0)
    if args.copy_probe:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda:0").fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if args.only_c3:
        res = bench_expert_c3(dtype, max(10, min(50, args.steps)))
        log("expert C3:", res)
        print(json.dumps({"metric": "expert kernel HBM GB/s", "value": res["achieved_GBps"], "unit": "GB/s", "n_gpus": 1,
                          "steps": args.steps, "warmup": args.warmup, "expert_c3": res}), flush=True)
        return
    if args.only_c5:
        res = bench_block_c5(dtype, max(3, min(10, args.steps)))
        log("block C5:", res)
        print(json.dumps({"metric": "FlashMoE fwd tokens/s (h2048, 256K experts, top-128)", "value": res["tokens_per_s"],
                          "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "block_c5": res}),
              flush=True)
        return
    if args.only_backward:
        res = bench_backward_c4(dtype, max(5, min(20, args.steps)))
        log("backward C4:", res)
        print(json.dumps({"metric": "FlashMoE fwd+bwd tokens/s (h1024, 16K experts, top-64)", "value": res["tokens_per_s"],
                          "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "backward_c4": res}),
              flush=True)
        return
    m, x = synthetic_block(C4, dtype, "cuda:0")
    T = C4["batch"] * C4["seq"]

    # K timed steps between two device synchronisations; inside, one HIP-event pair per step on the launch stream
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    with torch.no_grad():
        for _ in range(args.warmup):
            m(x)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for start, stop in pairs:
            start.record()
            m(x)
            stop.record()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
    step_ms = [start.elapsed_time(stop) for start, stop in pairs]
    wall_ms_per_step = (t1 - t0) * 1e3 / args.steps
    ms_per_step = statistics.median(step_ms)
    log(f"block: median {ms_per_step:.4f} ms/step (min {min(step_ms):.4f}, max {max(step_ms):.4f}; host clock over the "
        f"{args.steps} steps {wall_ms_per_step:.4f}) -> {T / ms_per_step * 1e3:.0f} tokens/s")

    # per-stage durations (HIP events on the launch stream), kernels launched through the C ABI
    fns, work, keep = stage_kernels(m, x)
    iters = max(20, min(200, args.steps))
    stages = {}
    times = {}
    stage_spread = {}
    for name, fn in fns.items():
        per_call = event_times_ms(fn, iters)
        times[name] = statistics.fmean(per_call)          # the roofline entries use the average launch duration
        stage_spread[name] = spread(per_call)
        stages[name] = stage_spread[name]["median"]
    log("stage durations (us, min / median / max / mean):", stage_spread)
    rooflines = {n: roofline_entry(n, times[n], work[n], measured_traffic(n, "c4"), spread_us=stage_spread[n]) for n in fns}
    # router_topk is part of router_forward: it is listed, but only whole launches compete for "dominant"
    dominant = max((n for n in times if n != "router_topk"), key=times.get)

    result = {
        "metric": "FlashMoE fwd tokens/s (h1024, 16K experts, top-64)",
        "value": round(T / ms_per_step * 1e3, 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        # ms_per_step is the median over the K steps of the HIP-event time of one step; wall_ms_per_step is the host clock
        # between the two synchronisations divided by K
        "step_ms": spread(step_ms, scale=1.0, digits=4),
        "wall_ms_per_step": round(wall_ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "C4 full FlashMoE block (README config): bf16, batch 1 x seq 4096, hidden 1024, "
                               "intermediate 4096, silu, 16384 experts, top-64, norm_topk_prob False, train-mode batch norm",
                   "tokens": T, "hidden": C4["hidden"], "intermediate": C4["inter"], "num_experts": C4["experts"],
                   "top_k": C4["top_k"]},
        "roofline": rooflines[dominant],
        "stages_us": stages,
        "stages_spread_us": stage_spread,
        # the block's own launches: the stages without the stand-alone top-k and without the expert op's id -> offset
        # pass (inside the block the router writes the offsets); what is left of ms_per_step is launch gaps
        "stages_sum_us": round(sum(v for k, v in stages.items() if k != "router_topk"), 2),
        "rooflines_all": rooflines,
        "traffic_source": TRAFFIC_SOURCE,
    }
    if not args.no_c3:
        result["expert_c3"] = bench_expert_c3(dtype, max(10, min(50, args.steps)))
        log("expert C3:", result["expert_c3"])
    del keep
    if not args.no_extras:
        result["router_c2"] = bench_router_c2(dtype, max(10, min(50, args.steps)))
        log("router C2:", result["router_c2"])
        del m, x, fns
        torch.cuda.empty_cache()
        result["block_c5"] = bench_block_c5(dtype, 5)
        log("block C5:", result["block_c5"])
        torch.cuda.empty_cache()
        result["block_c1"] = bench_block_c1(50)
        log("block C1:", result["block_c1"])
        result["mlp_fp32"] = result["rooflines_all"]["mlp_fp32"] = bench_mlp_fp32(10)
        log("mlp fp32:", result["mlp_fp32"])
        result["backward_c4"] = bench_backward_c4(dtype, 10)
        log("backward C4:", result["backward_c4"])
        torch.cuda.empty_cache()
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(C4, dtype, budget_s=12.0)
        log("cpu baseline:", result["cpu_baseline"])
        # the reference's own CPU configuration (fp32, 512 tokens, 1024 experts, top-16) and the README block in fp32
        result["cpu_baseline_c1"] = cpu_baseline(C1, torch.float32, budget_s=4.0, label="C1")
        log("cpu baseline C1:", result["cpu_baseline_c1"])
        result["cpu_baseline_c4_fp32"] = cpu_baseline(C4, torch.float32, budget_s=6.0)
        log("cpu baseline C4 fp32:", result["cpu_baseline_c4_fp32"])
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
