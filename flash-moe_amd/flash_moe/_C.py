"""ctypes binding of ``libflashmoe_hip.so`` (the C ABI declared in ``include/flashmoe_hip.h``).

The library is loaded from ``flash_moe/lib/`` next to this file.  It is never built at import or call
time, and there is no fallback: if it is missing, the first op call raises.
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional

import torch

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libflashmoe_hip.so")
_lib: Optional[ctypes.CDLL] = None

ABI_VERSION = 1

F32, BF16, F16 = 0, 1, 2
_DTYPE_CODE = {torch.float32: F32, torch.bfloat16: BF16, torch.float16: F16}

ERR_TOPK_RANGE = -3

EXPERT_AUTO, EXPERT_ROWS, EXPERT_SLICES, EXPERT_BUCKETS = 0, 1, 2, 3

_vp, _i64, _int, _sz = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_size_t

# name -> (restype, argtypes); mirrors include/flashmoe_hip.h one to one
SIGNATURES = {
    "fmoe_abi_version": (_int, []),
    "fmoe_last_error": (ctypes.c_char_p, []),
    "fmoe_router_topk": (_int, [_vp, _i64, _int, _int, _int, _vp, _vp, _vp, _int, _vp]),
    "fmoe_router_workspace_bytes": (_sz, [_i64, _int, _int]),
    "fmoe_router_forward": (_int, [_vp, _vp, _vp, _vp, _vp, _int, _int, ctypes.c_float, ctypes.c_float, _i64, _int, _int,
                                   _int, _int, _int, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "fmoe_router_forward_split": (_int, [_vp, _vp, _vp, _vp, _vp, _int, _int, ctypes.c_float, ctypes.c_float, _i64, _int, _int,
                                         _int, _int, _int, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "fmoe_router_forward_noalloc": (_int, [_vp, _vp, _vp, _vp, _vp, _int, _int, ctypes.c_float, ctypes.c_float, _i64, _int, _int,
                                           _int, _int, _int, _vp, _vp, _vp, _vp, _vp, _vp]),
    "fmoe_expert_workspace_bytes": (_sz, [_i64, _int, _i64, _int, _int]),
    "fmoe_expert_workspace_bytes_algo": (_sz, [_i64, _int, _i64, _int, _int, _int]),
    "fmoe_expert_forward": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _int, _i64, _int, _int, _vp, _vp, _sz, _vp]),
    "fmoe_expert_forward_algo": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _int, _i64, _int, _int, _vp, _vp, _sz, _int, _vp]),
    "fmoe_expert_bucket_workspace_bytes": (_sz, [_i64]),
    "fmoe_expert_bucket": (_int, [_vp, _i64, _int, _i64, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "fmoe_mlp_workspace_bytes": (_sz, [_i64, _int, _int, _int]),
    "fmoe_mlp_forward": (_int, [_vp, _vp, _vp, _vp, _i64, _int, _int, _int, _vp, _vp, _vp, _sz, _vp]),
    "fmoe_block_workspace_bytes": (_sz, [_i64, _int, _int, _int, _i64, _int, _int]),
    "fmoe_block_forward": (_int, [_vp] * 10 + [_int, _int, ctypes.c_float, ctypes.c_float, _i64, _int, _int, _i64, _int, _int,
                                  _int, _int, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "fmoe_mlp_gate_up": (_int, [_vp, _vp, _vp, _i64, _int, _int, _int, _vp, _vp]),
    "fmoe_mlp_gate_up_save": (_int, [_vp, _vp, _vp, _i64, _int, _int, _int, _vp, _vp, _vp]),
    "fmoe_mlp_down": (_int, [_vp, _vp, _i64, _int, _int, _int, _vp, _vp, _vp]),
    "fmoe_peer_forward": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _int, _i64, _int, _int, _vp, _vp, _sz, _vp]),
    "fmoe_pkm_workspace_bytes": (_sz, [_i64, _int, _i64, _int, _int]),
    "fmoe_pkm_forward": (_int, [_vp, _vp, _vp, _i64, _int, _i64, _int, _int, _vp, _vp, _sz, _vp]),
    "fmoe_router_topk_backward": (_int, [_vp, _vp, _i64, _int, _int, _int, _vp, _vp]),
    "fmoe_route_backward": (_int, [_vp, _vp, _vp, _vp, _i64, _int, _int, _int, _int, _vp, _vp]),
    "fmoe_router_workspace_stats_offset": (_sz, [_i64, _int, _int]),
    "fmoe_router_prologue_backward_workspace_bytes": (_sz, [_i64, _int, _int, _int]),
    "fmoe_router_prologue_backward": (_int, [_vp, _vp, _vp, _vp, _int, _i64, _int, _int, _int, _vp, _vp, _vp, _sz, _vp]),
    "fmoe_swiglu_backward": (_int, [_vp, _vp, _vp, _i64, _int, _int, _vp, _vp, _vp]),
    "fmoe_mlp_backward_workspace_bytes": (_sz, [_i64, _int, _int, _int]),
    "fmoe_mlp_backward": (_int, [_vp] * 6 + [_i64, _int, _int, _int] + [_vp] * 5 + [_sz, _vp]),
    "fmoe_expert_backward_workspace_bytes": (_sz, [_i64, _int, _i64, _int, _int]),
    "fmoe_expert_backward": (_int, [_vp] * 6 + [_i64, _int, _i64, _int, _int] + [_vp] * 5 + [_sz, _vp]),
}


def lib_path() -> str:
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    """Load (once) and return the shared library; raise if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError(
                f"{_LIB_PATH} not found: build it with `make -C flash-moe_amd/csrc` "
                "(hipcc, --offload-arch=gfx950); there is no fallback path"
            )
        handle = ctypes.CDLL(_LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype, fn.argtypes = res, args
        got = handle.fmoe_abi_version()
        if got != ABI_VERSION:
            raise RuntimeError(f"{_LIB_PATH}: ABI version {got}, this package expects {ABI_VERSION}")
        _lib = handle
    return _lib


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise TypeError(f"unsupported dtype {dtype}; expected float32, bfloat16 or float16") from None


def require_gpu(*tensors: torch.Tensor) -> torch.device:
    """All tensors must live on one HIP device; returns it."""
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError("flash_moe HIP ops need tensors on a ROCm GPU (got a CPU tensor); there is no CPU path")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError(f"tensors on different devices: {dev} and {t.device}")
    return dev


def ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def current_stream(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def check(status: int, what: str) -> None:
    """Turn a C status into the exception the reference's call site would have raised."""
    if status == 0:
        return
    msg = lib().fmoe_last_error().decode() or f"status {status}"
    if status == ERR_TOPK_RANGE:
        raise AssertionError(msg)
    if status < 0:
        raise ValueError(f"{what}: {msg}")
    raise RuntimeError(f"{what}: HIP error {status}: {msg}")
