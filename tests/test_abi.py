"""The C-ABI library: loads without a GPU, exports every symbol the header declares, and rejects bad
arguments with the documented status codes before touching the device."""
import ctypes
import os
import re

import pytest
import torch

from flash_moe import _C

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "flashmoe_hip.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fmoe_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = declared_functions()
    for must in ("fmoe_router_topk", "fmoe_expert_forward", "fmoe_mlp_forward", "fmoe_last_error", "fmoe_abi_version"):
        assert must in names


def test_library_exports_every_declared_symbol():
    lib = _C.lib()
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} declared in flashmoe_hip.h but not exported by {_C.lib_path()}"
    # and the Python binding table names exactly the declared functions
    assert sorted(_C.SIGNATURES) == declared_functions()
    assert lib.fmoe_abi_version() == _C.ABI_VERSION


def test_citations_in_header_point_at_the_reference_interface():
    text = open(HEADER).read()
    for cite in ("flash_router.py:381-382", "flash_expert.py:831-836", "flash_mlp.py:169-181", "flash_moe.py:101"):
        assert cite in text


def _buf(n=4096):
    b = ctypes.create_string_buffer(n + 256)
    addr = (ctypes.addressof(b) + 255) // 256 * 256
    return b, addr


def test_router_argument_checks():
    lib = _C.lib()
    keep, a = _buf()
    # top_k outside [0, nk]: the reference's assertion (flash_router.py:261-263)
    assert lib.fmoe_router_topk(a, 4, 8, 9, _C.F32, a, a, None, 0, None) == -3
    assert b"[0, 8]" in lib.fmoe_last_error()
    assert lib.fmoe_router_topk(a, 4, 8, -1, _C.F32, a, a, None, 0, None) == -3
    assert lib.fmoe_router_topk(a, 4, 8, 4, 7, a, a, None, 0, None) == -4          # dtype
    assert lib.fmoe_router_topk(a, -1, 8, 4, _C.F32, a, a, None, 0, None) == -2     # shape
    assert lib.fmoe_router_topk(None, 4, 8, 4, _C.F32, a, a, None, 0, None) == -1   # null
    assert lib.fmoe_router_topk(a, 4, 8192, 4097, _C.F32, a, a, None, 0, None) == -5  # top_k > 4096
    assert lib.fmoe_router_topk(a, 4, 70000, 4, _C.F32, a, a, None, 0, None) == -5    # num_keys > 65535
    # empty problems succeed without a launch
    assert lib.fmoe_router_topk(None, 0, 8, 4, _C.F32, None, None, None, 0, None) == 0
    assert lib.fmoe_router_topk(a, 4, 8, 0, _C.F32, a, a, None, 0, None) == 0
    assert lib.fmoe_last_error() == b""


def test_fused_router_argument_checks():
    lib = _C.lib()
    keep, a = _buf()
    f = lib.fmoe_router_forward
    need = lib.fmoe_router_workspace_bytes(64, 128, 16)
    assert need > 0 and need % 256 == 0
    ok_args = dict(x=a, w=a, rm=a, rv=a, nbt=a)
    call = lambda **kw: f(kw.get("x", a), a, a, a, a, _C.F32, kw.get("training", 1), 0.1, 1e-5, kw.get("T", 64), 128, 16,
                          kw.get("K", 4), kw.get("dtype", _C.BF16), 0, a, a, a, a, a, kw.get("ws", a), kw.get("wsb", need), None)
    assert call(K=17) == -3                       # top_k > num_keys
    assert call(dtype=9) == -4
    assert call(T=-1) == -2
    assert call(T=1) == -2                        # one token in training mode, as nn.BatchNorm1d
    assert b"more than 1 value per channel" in lib.fmoe_last_error()
    assert call(x=None) == -1
    assert call(wsb=need - 1) == -7
    assert call(T=0) == 0


def test_expert_argument_checks():
    lib = _C.lib()
    keep, a = _buf()
    f = lib.fmoe_expert_forward
    assert f(a, a, a, a, a, 4, 64, 16, 2, 9, a, None, 0, None) == -4
    assert f(a, a, a, a, a, 4, 0, 16, 2, _C.BF16, a, None, 0, None) == -2
    assert f(None, a, a, a, a, 4, 64, 16, 2, _C.BF16, a, None, 0, None) == -1
    assert f(a, a, a, None, a, 4, 64, 16, 2, _C.BF16, a, None, 0, None) == -1
    assert f(a, a, a, a, a, 4, 60, 16, 2, _C.BF16, a, None, 0, None) == -6          # row not 16-byte multiple
    assert f(a + 2, a, a, a, a, 4, 64, 16, 2, _C.BF16, a, None, 0, None) == -6      # misaligned pointer
    # rows too long for the row kernels take the column slices, which need their workspace; forcing rows is refused
    assert f(a, a, a, a, a, 4, 1 << 20, 16, 2, _C.BF16, a, None, 0, None) == -7
    assert lib.fmoe_expert_workspace_bytes(4, 1 << 20, 16, 2, _C.BF16) > 0
    assert lib.fmoe_expert_forward_algo(a, a, a, a, a, 4, 1 << 20, 16, 2, _C.BF16, a, None, 0, _C.EXPERT_ROWS, None) == -5
    assert f(None, None, None, None, None, 0, 64, 16, 2, _C.BF16, None, None, 0, None) == 0
    assert isinstance(lib.fmoe_expert_workspace_bytes(1024, 1024, 16384, 64, _C.BF16), int)
    # the size follows the schedule: column slices when a slice of the table fits L2 and there are enough pairs, else none
    sliced = lib.fmoe_expert_workspace_bytes(4096, 1024, 16384, 64, _C.BF16)
    assert sliced >= 4096 * 64 * (4 + 4 + 8 * 4) and sliced % 256 == 0               # 8 slices of 256 bytes
    wide = lib.fmoe_expert_workspace_bytes(4096, 1024, 32768, 64, _C.BF16)
    assert wide >= 4096 * 64 * (4 + 4 + 16 * 4) and wide % 256 == 0                   # 16 slices of 128 bytes
    # a table whose slices are too large for L2 takes the bucketed schedule: bucketing state, grouped order, band-major x,
    # 32 bands of partial scores, the per-owner lists of the sweep
    big = lib.fmoe_expert_workspace_bytes(32768, 2048, 262144, 128, _C.BF16)
    assert big >= 32768 * 128 * 4 * (4 + 32 + 2) + 32768 * 2048 * 2 and big % 256 == 0
    assert big == lib.fmoe_expert_workspace_bytes_algo(32768, 2048, 262144, 128, _C.BF16, _C.EXPERT_BUCKETS)
    assert lib.fmoe_expert_workspace_bytes_algo(32768, 2048, 262144, 128, _C.BF16, _C.EXPERT_ROWS) == 0
    assert lib.fmoe_expert_workspace_bytes(64, 1024, 16384, 8, _C.BF16) == 0            # too few pairs
    assert lib.fmoe_expert_workspace_bytes_algo(64, 1024, 16384, 8, _C.BF16, _C.EXPERT_SLICES) > 0
    assert lib.fmoe_expert_workspace_bytes_algo(4096, 1024, 16384, 64, _C.BF16, _C.EXPERT_ROWS) == 0
    assert lib.fmoe_expert_workspace_bytes_algo(4096, 1024, 16384, 64, _C.BF16, _C.EXPERT_AUTO) == sliced
    # a product-key memory has no score phase: it never takes the bucketed plan's workspace (the reference's PKM
    # benchmark shape, tests/test_pkm.py: 16384 tokens, top-2500, would ask for gigabytes of partial scores there)
    assert lib.fmoe_pkm_workspace_bytes(4096, 1024, 16384, 64, _C.BF16) == sliced
    assert lib.fmoe_pkm_workspace_bytes(32768, 2048, 262144, 128, _C.BF16) == 0
    assert lib.fmoe_pkm_workspace_bytes(16384, 1024, 1 << 20, 2500, _C.BF16) == 0 < lib.fmoe_expert_workspace_bytes(
        16384, 1024, 1 << 20, 2500, _C.BF16)
    assert lib.fmoe_pkm_workspace_bytes(0, 1024, 16, 4, _C.BF16) == 0 and lib.fmoe_pkm_workspace_bytes(4, 1024, 16, 4, 9) == 0


def test_mlp_argument_checks():
    lib = _C.lib()
    keep, a = _buf()
    f = lib.fmoe_mlp_forward
    need = lib.fmoe_mlp_workspace_bytes(8, 64, 128, _C.BF16)
    assert need >= 8 * 128 * 2 and need % 256 == 0
    assert lib.fmoe_mlp_workspace_bytes(8, 64, 128, _C.F32) >= 8 * 128 * 4
    assert f(a, a, a, a, 8, 64, 128, 5, None, a, a, need, None) == -4
    assert f(a, a, a, a, 8, 64, -1, _C.BF16, None, a, a, need, None) == -2
    assert f(a, None, a, a, 8, 64, 128, _C.BF16, None, a, a, need, None) == -1
    assert f(a, a, a, a, 8, 64, 128, _C.BF16, None, a, a, need - 1, None) == -7
    assert f(a, a, a, a, 8, 64, 128, _C.BF16, None, a, None, need, None) == -7
    assert f(a, a, a, a, 8, 60, 128, _C.BF16, None, a, a, need, None) == -6
    assert f(None, None, None, None, 0, 64, 128, _C.BF16, None, None, None, 0, None) == 0


def test_block_argument_checks():
    lib = _C.lib()
    keep, a = _buf()
    f = lib.fmoe_block_forward
    T, H, I, E, nk, K = 8, 64, 128, 1024, 32, 4
    need = lib.fmoe_block_workspace_bytes(T, H, I, nk, E, K, _C.BF16)
    parts = (lib.fmoe_router_workspace_bytes(T, H, nk) + lib.fmoe_expert_workspace_bytes(T, H, E, K, _C.BF16)
             + lib.fmoe_mlp_workspace_bytes(T, H, I, _C.BF16))
    assert need >= parts + T * 2 * nk * 4 + T * K * (4 + 8 + 2) + T * H * 2 and need % 256 == 0
    assert lib.fmoe_block_workspace_bytes(T, H, I, nk, E, K, 9) == 0

    def call(T=T, H=H, I=I, E=E, nk=nk, K=K, dtype=_C.BF16, x=a, ws=a, ws_bytes=need):
        return f(x, a, a, a, a, a, a, a, a, a, _C.F32, 1, 0.1, 1e-5, T, H, I, E, nk, K, dtype, 0, a, a, None, None,
                 ws, ws_bytes, None)

    assert call(dtype=6) == -4
    assert call(I=0) == -2
    assert call(nk=33) == -2                      # nk*nk > E
    assert call(K=33) == -3 and b"[0, 32]" in lib.fmoe_last_error()
    assert call(x=None) == -1
    assert call(H=60) == -6
    assert call(I=100) == -6
    assert call(ws_bytes=need - 1) == -7
    assert call(ws=None) == -7
    assert call(T=0, x=None, ws=None, ws_bytes=0) == 0


def test_backward_argument_checks():
    lib = _C.lib()
    keep, a = _buf()
    rb = lib.fmoe_router_topk_backward
    assert rb(a, a, 4, 8, 2, 9, a, None) == -4
    assert rb(a, a, 4, 0, 2, _C.F32, a, None) == -2
    assert rb(a, a, 4, 70000, 2, _C.F32, a, None) == -5                          # the forward op's own key limit
    assert rb(a, None, 4, 8, 2, _C.F32, a, None) == -1
    assert rb(None, None, 0, 8, 2, _C.F32, None, None) == 0
    rt = lib.fmoe_route_backward
    assert rt(a, a, a, None, 4, 8, 2, 9, 0, a, None) == -4                       # dtype
    assert rt(a, a, a, None, 4, 0, 2, _C.BF16, 0, a, None) == -2                 # num_keys
    assert rt(a, a, a, None, 4, 40000, 2, _C.BF16, 0, a, None) == -5             # the fused router's own key limit
    assert rt(a, a, None, None, 4, 8, 2, _C.BF16, 0, a, None) == -1              # logits
    assert rt(None, None, a, None, 4, 8, 2, _C.BF16, 0, a, None) == -1           # gate gradient with top_k > 0
    assert rt(None, None, None, None, 0, 8, 2, _C.BF16, 1, None, None) == 0      # empty batch
    off = lib.fmoe_router_workspace_stats_offset(64, 128, 16)
    assert 0 < off < lib.fmoe_router_workspace_bytes(64, 128, 16) and off % 256 == 0
    pneed = lib.fmoe_router_prologue_backward_workspace_bytes(64, 128, 16, _C.BF16)
    assert pneed >= 64 * 32 * 2 + 2 * 64 * 128 * 2 and pneed % 256 == 0
    pb = lib.fmoe_router_prologue_backward
    assert pb(a, a, a, a, 1, 64, 128, 16, 4, a, a, a, pneed, None) == -4
    assert pb(a, a, a, a, 1, 0, 128, 16, _C.BF16, a, a, a, pneed, None) == -2
    assert pb(a, a, a, a, 1, 64, 124, 16, _C.BF16, a, a, a, pneed, None) == -6
    assert pb(None, a, a, a, 1, 64, 128, 16, _C.BF16, a, a, a, pneed, None) == -1
    assert pb(a, a, a, a, 1, 64, 128, 16, _C.BF16, a, a, a, pneed - 1, None) == -7
    sb = lib.fmoe_swiglu_backward
    assert sb(a, a, a, 4, 64, 7, a, a, None) == -4
    assert sb(a, a, a, 4, 0, _C.BF16, a, a, None) == -2
    assert sb(a, a, a, 4, 60, _C.BF16, a, a, None) == -6
    assert sb(a, None, a, 4, 64, _C.BF16, a, a, None) == -1
    assert sb(None, None, None, 0, 64, _C.BF16, None, None, None) == 0
    need = lib.fmoe_expert_backward_workspace_bytes(8, 64, 256, 4, _C.BF16)
    assert need >= 8 * 4 * 24 + 257 * 4 and need % 256 == 0
    eb = lib.fmoe_expert_backward

    def ecall(T=8, H=64, E=256, K=4, dtype=_C.BF16, dout=a, ws=a, ws_bytes=need):
        return eb(dout, a, a, a, a, a, T, H, E, K, dtype, a, a, a, a, ws, ws_bytes, None)

    assert ecall(dtype=3) == -4
    assert ecall(H=0) == -2
    assert ecall(H=60) == -6
    assert ecall(H=8192) == -7                     # long rows take the column-slice kernels: a larger workspace
    assert ecall(H=8192, E=1 << 19) == -5          # ... which cannot address tables of 4 GiB or more
    assert ecall(dout=None) == -1
    assert ecall(ws_bytes=need - 1) == -7
    mneed = lib.fmoe_mlp_backward_workspace_bytes(8, 64, 128, _C.BF16)
    assert mneed >= 6 * 8 * 128 * 2 and mneed % 256 == 0
    mb = lib.fmoe_mlp_backward

    def mcall(T=8, H=64, I=128, dtype=_C.BF16, dy=a, ws_bytes=mneed):
        return mb(dy, a, a, a, a, None, T, H, I, dtype, a, a, a, a, a, ws_bytes, None)

    assert mcall(dtype=5) == -4
    assert mcall(T=0) == -2
    assert mcall(I=100) == -6
    assert mcall(dy=None) == -1
    assert mcall(ws_bytes=mneed - 1) == -7


def test_python_wrappers_refuse_cpu_tensors():
    from flash_moe.ops import flash_expert_func, flash_mlp_func, flash_router_func

    with pytest.raises(RuntimeError, match="no CPU path"):
        flash_router_func(torch.zeros(2, 4, 8), 8, 2)
    with pytest.raises(RuntimeError, match="no CPU path"):
        flash_expert_func(torch.zeros(4, 8), torch.zeros(16, 8), torch.zeros(16, 8), torch.zeros(4, 2, dtype=torch.int64), torch.zeros(4, 2))
    with pytest.raises(RuntimeError, match="no CPU path"):
        flash_mlp_func(torch.zeros(4, 8), torch.zeros(16, 8), torch.zeros(16, 8), torch.zeros(8, 16))
