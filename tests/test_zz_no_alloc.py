"""The router entry point that allocates nothing (``fmoe_router_forward_noalloc``: its scratch is a static array in device
memory) against ``fmoe_router_forward`` with a caller-provided workspace, through the C ABI: bit-identical outputs, on two
calls in a row, the second with a smaller input (the static scratch keeps the first call's contents)."""
import pytest
import torch

from flash_moe import _C

pytestmark = pytest.mark.gpu


def _route(entry, x, w, nk, K, training, norm_flag):
    T, H = x.shape
    dev = x.device
    rm = torch.zeros(H, device=dev, dtype=torch.float32)
    rv = torch.ones(H, device=dev, dtype=torch.float32)
    nbt = torch.zeros(1, device=dev, dtype=torch.int64)
    logits = torch.empty(T, 2 * nk, device=dev, dtype=x.dtype)
    logits32 = torch.empty(T, 2 * nk, device=dev, dtype=torch.float32)
    scores = torch.empty(T, K, device=dev, dtype=torch.float32)
    indices = torch.empty(T, K, device=dev, dtype=torch.int64)
    gates = torch.empty(T, K, device=dev, dtype=x.dtype)
    L = _C.lib()
    common = (_C.ptr(x), _C.ptr(w), _C.ptr(rm), _C.ptr(rv), _C.ptr(nbt), _C.F32, int(training), 0.1, 1e-5, T, H, nk, K,
              _C.dtype_code(x.dtype), int(norm_flag), _C.ptr(logits), _C.ptr(logits32), _C.ptr(scores), _C.ptr(indices),
              _C.ptr(gates))
    stream = _C.current_stream(dev)
    with torch.cuda.device(dev):
        if entry == "noalloc":
            status = L.fmoe_router_forward_noalloc(*common, stream)
        else:
            need = L.fmoe_router_workspace_bytes(T, H, nk)
            ws = torch.empty(need, device=dev, dtype=torch.uint8)
            status = L.fmoe_router_forward(*common, _C.ptr(ws), need, stream)
    _C.check(status, entry)
    torch.cuda.synchronize()
    return logits, logits32, scores, indices, gates, rm, rv, nbt


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("training", [True, False])
def test_noalloc_router_equals_the_workspace_entry_point_on_two_calls(dtype, training):
    g = torch.Generator().manual_seed(11)
    cases = [(2048, 1024, 128, 64), (300, 256, 32, 16)]      # the second call is smaller in every extent
    for T, H, nk, K in cases:
        x = (torch.randn(T, H, generator=g) * 1.3 + 0.2).to(dtype).cuda()
        w = (torch.randn(2 * nk, H, generator=g) * 0.02).to(dtype).cuda()
        got = _route("noalloc", x, w, nk, K, training, True)
        ref = _route("workspace", x, w, nk, K, training, True)
        for a, b, name in zip(got, ref, ("logits", "logits32", "scores", "indices", "gates", "mean", "var", "count")):
            assert torch.equal(a, b), f"{name} differs at T={T} H={H}"
        assert int(got[3].min()) >= 0 and int(got[3].max()) < nk * nk


@pytest.mark.parametrize("dtype,training", [(torch.bfloat16, True), (torch.float16, False)])
def test_noalloc_router_equals_the_workspace_entry_point_where_that_one_takes_the_tiled_gate_product(dtype, training):
    """With at least one 256 x 256 tile of logits per compute unit the workspace entry point normalises x into its workspace
    and runs the gate product on the shared MLP's tiled kernel; the no-allocation entry point has no room for that copy and
    keeps the 64 x 64 gate kernel.  Both add the products in ascending k, 16 per matrix instruction: bit-identical."""
    T, H, nk, K = 16384, 256, 512, 16
    L = _C.lib()
    assert L.fmoe_router_workspace_bytes(T, H, nk) >= T * H * 2 > L.fmoe_router_workspace_bytes(T // 2, H, nk)
    g = torch.Generator().manual_seed(12)
    x = (torch.randn(T, H, generator=g) * 1.3 + 0.2).to(dtype).cuda()
    w = (torch.randn(2 * nk, H, generator=g) * 0.05).to(dtype).cuda()
    got = _route("noalloc", x, w, nk, K, training, False)
    ref = _route("workspace", x, w, nk, K, training, False)
    for a, b, name in zip(got, ref, ("logits", "logits32", "scores", "indices", "gates", "mean", "var", "count")):
        assert torch.equal(a, b), f"{name} differs"


def test_noalloc_router_rejects_sizes_beyond_its_scratch():
    L = _C.lib()
    x = torch.zeros(4, 4096, device="cuda", dtype=torch.bfloat16)
    a = _C.ptr(x)
    status = L.fmoe_router_forward_noalloc(a, a, a, a, a, _C.F32, 1, 0.1, 1e-5, 4, 4096, 8, 2, _C.BF16, 0, a, a, a, a, a, None)
    assert status == -5 and b"2048" in L.fmoe_last_error()


def test_noalloc_router_in_a_hip_graph_after_one_warm_up_call():
    """The first call on a device looks up the address of the static scratch and the device geometry (host-side queries,
    not stream work), so one eager call precedes the capture; after it the entry point only launches kernels, and every
    replay of a graph that holds it equals the eager workspace entry point on the same input."""
    dtype, T, H, nk, K = torch.bfloat16, 1024, 512, 64, 32
    g = torch.Generator().manual_seed(5)
    dev = torch.device("cuda")
    w = (torch.randn(2 * nk, H, generator=g) * 0.02).to(dtype).cuda()
    static_x = torch.randn(T, H, generator=g).to(dtype).cuda()
    _route("noalloc", static_x, w, nk, K, False, True)                      # the warm-up call
    rm, rv = torch.zeros(H, device=dev), torch.ones(H, device=dev)
    nbt = torch.zeros(1, device=dev, dtype=torch.int64)
    logits = torch.empty(T, 2 * nk, device=dev, dtype=dtype)
    logits32 = torch.empty(T, 2 * nk, device=dev, dtype=torch.float32)
    scores = torch.empty(T, K, device=dev, dtype=torch.float32)
    indices = torch.empty(T, K, device=dev, dtype=torch.int64)
    gates = torch.empty(T, K, device=dev, dtype=dtype)
    L = _C.lib()

    def call():
        _C.check(L.fmoe_router_forward_noalloc(_C.ptr(static_x), _C.ptr(w), _C.ptr(rm), _C.ptr(rv), _C.ptr(nbt), _C.F32, 0, 0.1,
                                               1e-5, T, H, nk, K, _C.BF16, 1, _C.ptr(logits), _C.ptr(logits32), _C.ptr(scores),
                                               _C.ptr(indices), _C.ptr(gates), _C.current_stream(dev)), "noalloc in capture")

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    for step in range(3):
        new_x = torch.randn(T, H, generator=torch.Generator().manual_seed(20 + step)).to(dtype).cuda()
        ref = _route("workspace", new_x, w, nk, K, False, True)              # eager work between the replays
        static_x.copy_(new_x)
        graph.replay()
        torch.cuda.synchronize()
        for a, b, name in zip((logits, logits32, scores, indices, gates), ref, ("logits", "logits32", "scores", "indices", "gates")):
            assert torch.equal(a, b), f"replay {step}: {name} differs"
