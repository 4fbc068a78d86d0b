"""Routed-expert op: ``out[t] = sum_k silu(<x_t, Wd[idx[t,k]]>) * g[t,k] * Wu[idx[t,k]]``.

Same call signature and return value as ``triton_flash_expert_func``
(flash_moe/ops/triton/flash_expert.py:831-836; contract docs/flash_expert.md:17-58); the work is done
by ``fmoe_expert_forward`` in libflashmoe_hip.so.
"""
from __future__ import annotations

import torch

from flash_moe import _C
from flash_moe.ops.utils import ensure_contiguous


def expert_forward(hidden_states, down_weights, up_weights, indices, routing_weights, algo: int = _C.EXPERT_AUTO) -> torch.Tensor:
    """``algo`` picks the schedule (``_C.EXPERT_AUTO`` / ``EXPERT_ROWS`` / ``EXPERT_SLICES``); the result is the same."""
    if hidden_states.dim() != 2 or down_weights.dim() != 2 or up_weights.dim() != 2:
        raise ValueError("hidden_states, down_weights and up_weights must be 2-D")
    if indices.dim() != 2 or routing_weights.shape != indices.shape:
        raise ValueError("indices and routing_weights must both be (num_tokens, num_experts_per_tok)")
    num_tokens, hidden = hidden_states.shape
    num_experts = down_weights.shape[0]
    if down_weights.shape != (num_experts, hidden) or up_weights.shape != (num_experts, hidden):
        raise ValueError("down_weights and up_weights must be (num_experts, hidden_size)")
    if indices.shape[0] != num_tokens:
        raise ValueError("indices has a different number of tokens than hidden_states")
    if indices.dtype != torch.int64:
        raise TypeError(f"indices must be int64 (got {indices.dtype})")
    dtype = hidden_states.dtype
    for name, t in (("down_weights", down_weights), ("up_weights", up_weights), ("routing_weights", routing_weights)):
        if t.dtype != dtype:
            raise TypeError(f"{name} has dtype {t.dtype}, hidden_states has {dtype}")
    dev = _C.require_gpu(hidden_states, down_weights, up_weights, indices, routing_weights)
    x, wd, wu, idx, g = (t.contiguous() for t in (hidden_states, down_weights, up_weights, indices, routing_weights))
    top_k = idx.shape[1]
    code = _C.dtype_code(dtype)
    out = torch.empty_like(x)
    L = _C.lib()
    ws_bytes = L.fmoe_expert_workspace_bytes_algo(num_tokens, hidden, num_experts, top_k, code, algo)
    ws = torch.empty(ws_bytes, device=dev, dtype=torch.uint8) if ws_bytes else None
    with torch.cuda.device(dev):
        status = L.fmoe_expert_forward_algo(
            _C.ptr(x), _C.ptr(wd), _C.ptr(wu), _C.ptr(idx), _C.ptr(g), num_tokens, hidden, num_experts, top_k,
            code, _C.ptr(out), _C.ptr(ws), ws_bytes, algo, _C.current_stream(dev),
        )
    _C.check(status, "flash_expert")
    return out


def expert_bucketing(indices: torch.Tensor, num_experts: int):
    """Expert-centric grouping of the (token, k) pairs on the GPU (``fmoe_expert_bucket``): returns
    ``(sorted_token_ids, expert_offsets, sorted_pair_ids, sorted_expert_ids)``, all int32; the first three are what
    ``_preprocess_expert_centric_indices_pytorch`` of the reference computes with sort / bincount / cumsum
    (flash_moe/ops/triton/flash_expert.py:528-577).  Pairs of expert ``e`` occupy slots ``[offsets[e], offsets[e+1])`` in
    ascending flattened position; ids outside ``[0, num_experts)`` are left out, so the three per-slot tensors have
    ``T*K`` entries of which the first ``offsets[-1]`` are meaningful.  No host synchronisation."""
    if indices.dim() != 2 or indices.dtype != torch.int64:
        raise ValueError("indices must be an int64 tensor (num_tokens, num_experts_per_tok)")
    dev = _C.require_gpu(indices)
    idx = indices.contiguous()
    num_tokens, top_k = idx.shape
    pairs = num_tokens * top_k
    offsets = torch.empty(num_experts + 1, device=dev, dtype=torch.int32)
    sorted_pairs, sorted_tokens, sorted_experts = (torch.empty(pairs, device=dev, dtype=torch.int32) for _ in range(3))
    L = _C.lib()
    ws_bytes = L.fmoe_expert_bucket_workspace_bytes(num_experts)
    ws = torch.empty(max(ws_bytes, 1), device=dev, dtype=torch.uint8)
    with torch.cuda.device(dev):
        status = L.fmoe_expert_bucket(_C.ptr(idx), num_tokens, top_k, num_experts, _C.ptr(offsets), _C.ptr(sorted_pairs),
                                      _C.ptr(sorted_tokens), _C.ptr(sorted_experts), _C.ptr(ws), ws_bytes,
                                      _C.current_stream(dev))
    _C.check(status, "flash_expert bucketing")
    return sorted_tokens, offsets, sorted_pairs, sorted_experts


def preprocess_expert_centric_indices(indices: torch.Tensor, routing_weights: torch.Tensor, num_experts: int):
    """Same return tuple as the reference's ``_preprocess_expert_centric_indices_pytorch(Indices, G, num_experts)``
    (flash_moe/ops/triton/flash_expert.py:528-577): ``(sorted_token_ids, sorted_G, expert_offsets, max_pairs_per_expert,
    sorted_pair_ids)``, for callers written against it.  ``max_pairs_per_expert`` is a host integer, so this helper
    synchronises like the reference does; the library's own forward and backward never need it.  Every id must lie in
    ``[0, num_experts)`` (the reference's contract)."""
    sorted_tokens, offsets, sorted_pairs, _ = expert_bucketing(indices, num_experts)
    sorted_g = routing_weights.reshape(-1)[sorted_pairs.long()]
    max_pairs = int((offsets[1:] - offsets[:-1]).max().item()) if num_experts > 0 else 0
    return sorted_tokens, sorted_g, offsets, max_pairs, sorted_pairs


def expert_backward(dexperts_states, hidden_states, down_weights, up_weights, indices, routing_weights):
    """Gradients ``(dhidden_states, ddown_weights, dup_weights, drouting_weights)`` of ``expert_forward``
    (``fmoe_expert_backward``; the reference's _flash_expert_backward, flash_moe/ops/triton/flash_expert.py:654-745).
    Deterministic; the scores are recomputed rather than saved."""
    dev = _C.require_gpu(dexperts_states, hidden_states, down_weights, up_weights, indices, routing_weights)
    do, x, wd, wu, idx, g = (t.contiguous() for t in (dexperts_states, hidden_states, down_weights, up_weights, indices,
                                                      routing_weights))
    if do.shape != x.shape or do.dtype != x.dtype:
        raise ValueError("the output gradient must have the shape and dtype of hidden_states")
    num_tokens, hidden = x.shape
    num_experts, top_k = wd.shape[0], idx.shape[1]
    code = _C.dtype_code(x.dtype)
    dx, dwd, dwu, dg = torch.empty_like(x), torch.empty_like(wd), torch.empty_like(wu), torch.empty_like(g)
    L = _C.lib()
    ws_bytes = L.fmoe_expert_backward_workspace_bytes(num_tokens, hidden, num_experts, top_k, code)
    ws = torch.empty(max(ws_bytes, 1), device=dev, dtype=torch.uint8)
    with torch.cuda.device(dev):
        status = L.fmoe_expert_backward(
            _C.ptr(do), _C.ptr(x), _C.ptr(wd), _C.ptr(wu), _C.ptr(idx), _C.ptr(g), num_tokens, hidden, num_experts, top_k,
            code, _C.ptr(dx), _C.ptr(dwd), _C.ptr(dwu), _C.ptr(dg), _C.ptr(ws), ws_bytes, _C.current_stream(dev),
        )
    _C.check(status, "flash_expert backward")
    return dx, dwd, dwu, dg


class FlashExpertFunc(torch.autograd.Function):
    @staticmethod
    @ensure_contiguous
    def forward(ctx, hidden_states, down_weights, up_weights, indices, routing_weights):
        ctx.save_for_backward(hidden_states, down_weights, up_weights, indices, routing_weights)
        return expert_forward(hidden_states, down_weights, up_weights, indices, routing_weights)

    @staticmethod
    @ensure_contiguous
    def backward(ctx, dexperts_states):
        dx, dwd, dwu, dg = expert_backward(dexperts_states, *ctx.saved_tensors)
        return dx, dwd, dwu, None, dg


def flash_expert_func(hidden_states, down_weights, up_weights, indices, routing_weights):
    return FlashExpertFunc.apply(hidden_states, down_weights, up_weights, indices, routing_weights)
