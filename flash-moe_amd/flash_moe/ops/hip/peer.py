"""PEER op: ``out[t] = sum_k gelu(<x_t, Wd[idx[t,k]]>) * w[t,k] * Wu[idx[t,k]]`` (erf GELU).

Same call signature and return value as ``triton_peer_func`` (flash_moe/ops/triton/peer.py:246-255; note the
argument order: routing weights before indices); the work is done by ``fmoe_peer_forward`` in libflashmoe_hip.so,
which runs the routed-expert kernels with GELU in place of SiLU.  Forward only, as in the reference (peer.py:241-243).
"""
from __future__ import annotations

import torch

from flash_moe import _C
from flash_moe.ops.utils import ensure_contiguous


def peer_forward(hidden_states, down_embed, up_embed, routing_weights, indices) -> torch.Tensor:
    if hidden_states.dim() != 2 or down_embed.dim() != 2 or up_embed.shape != down_embed.shape:
        raise ValueError("expected hidden_states [T, H] and down_embed / up_embed [E, H]")
    if indices.dim() != 2 or routing_weights.shape != indices.shape or indices.shape[0] != hidden_states.shape[0]:
        raise ValueError("indices and routing_weights must both be (num_tokens, topk)")
    if indices.dtype != torch.int64:
        raise TypeError(f"indices must be int64 (got {indices.dtype})")
    dtype = hidden_states.dtype
    if any(t.dtype != dtype for t in (down_embed, up_embed, routing_weights)):
        raise TypeError(f"down_embed, up_embed and routing_weights must have the dtype of hidden_states ({dtype})")
    num_tokens, hidden = hidden_states.shape
    if down_embed.shape[1] != hidden:
        raise ValueError("down_embed / up_embed rows must have hidden_size elements")
    dev = _C.require_gpu(hidden_states, down_embed, up_embed, routing_weights, indices)
    x, wd, wu, w, idx = (t.contiguous() for t in (hidden_states, down_embed, up_embed, routing_weights, indices))
    num_experts, top_k, code = wd.shape[0], idx.shape[1], _C.dtype_code(dtype)
    out = torch.empty_like(x)
    L = _C.lib()
    ws_bytes = L.fmoe_expert_workspace_bytes(num_tokens, hidden, num_experts, top_k, code)
    ws = torch.empty(max(ws_bytes, 1), device=dev, dtype=torch.uint8)
    with torch.cuda.device(dev):
        status = L.fmoe_peer_forward(_C.ptr(x), _C.ptr(wd), _C.ptr(wu), _C.ptr(w), _C.ptr(idx), num_tokens, hidden, num_experts,
                                     top_k, code, _C.ptr(out), _C.ptr(ws), ws_bytes, _C.current_stream(dev))
    _C.check(status, "peer")
    return out


class PEERFunc(torch.autograd.Function):
    @staticmethod
    @ensure_contiguous
    def forward(ctx, hidden_states, down_embed, up_embed, routing_weights, indices):
        return peer_forward(hidden_states, down_embed, up_embed, routing_weights, indices)

    @staticmethod
    def backward(ctx, grad_output):
        raise NotImplementedError("PEER backward is not implemented (nor is it in the reference)")


def peer_func(hidden_states, down_embed, up_embed, routing_weights, indices):
    return PEERFunc.apply(hidden_states, down_embed, up_embed, routing_weights, indices)
