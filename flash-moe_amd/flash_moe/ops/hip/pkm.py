"""Product-key-memory value lookup: ``out[t] = sum_k w[t,k] * values[idx[t,k]]``.

Same call signature and return value as ``triton_pkm_func`` (flash_moe/ops/triton/pkm.py:195-200); the work is done
by ``fmoe_pkm_forward`` in libflashmoe_hip.so (the second phase of the routed-expert kernels, with the routing weight as
the coefficient).  Forward only, as in the reference (pkm.py:190-192).
"""
from __future__ import annotations

import torch

from flash_moe import _C
from flash_moe.ops.utils import ensure_contiguous


def pkm_forward(values, routing_weights, indices) -> torch.Tensor:
    if values.dim() != 2 or indices.dim() != 2 or routing_weights.shape != indices.shape:
        raise ValueError("expected values [E, H] and routing_weights / indices [T, topk]")
    if indices.dtype != torch.int64:
        raise TypeError(f"indices must be int64 (got {indices.dtype})")
    if routing_weights.dtype != values.dtype:
        raise TypeError(f"routing_weights has dtype {routing_weights.dtype}, values has {values.dtype}")
    dev = _C.require_gpu(values, routing_weights, indices)
    v, w, idx = values.contiguous(), routing_weights.contiguous(), indices.contiguous()
    (num_experts, hidden), (num_tokens, top_k), code = v.shape, idx.shape, _C.dtype_code(v.dtype)
    out = torch.empty((num_tokens, hidden), device=dev, dtype=v.dtype)
    L = _C.lib()
    ws_bytes = L.fmoe_pkm_workspace_bytes(num_tokens, hidden, num_experts, top_k, code)
    ws = torch.empty(max(ws_bytes, 1), device=dev, dtype=torch.uint8)
    with torch.cuda.device(dev):
        status = L.fmoe_pkm_forward(_C.ptr(v), _C.ptr(w), _C.ptr(idx), num_tokens, hidden, num_experts, top_k, code, _C.ptr(out),
                                    _C.ptr(ws), ws_bytes, _C.current_stream(dev))
    _C.check(status, "pkm")
    return out


class PKMFunc(torch.autograd.Function):
    @staticmethod
    @ensure_contiguous
    def forward(ctx, values, routing_weights, indices):
        return pkm_forward(values, routing_weights, indices)

    @staticmethod
    def backward(ctx, grad_output):
        raise NotImplementedError("PKM backward is not implemented (nor is it in the reference)")


def pkm_func(values, routing_weights, indices):
    return PKMFunc.apply(values, routing_weights, indices)
