"""Shared SwiGLU MLP op: ``(silu(x Wg^T) * (x Wu^T)) Wd^T``.

Same call signature and return value as ``triton_flash_mlp_func``
(flash_moe/ops/triton/flash_mlp.py:169-181); the work is done by ``fmoe_mlp_forward`` in
libflashmoe_hip.so (two MFMA GEMMs, the activation fused into the first one's epilogue).
"""
from __future__ import annotations

from typing import Optional

import torch

from flash_moe import _C
from flash_moe.ops.utils import ensure_contiguous


def mlp_forward(x, gate_weight, up_weight, down_weight, residual: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``x`` may have any leading shape; the last dimension is the hidden size.  ``residual`` (same shape
    as the output) is added in the second GEMM's epilogue (the add of flash_moe/modules/flash_moe.py:101)."""
    hidden = x.shape[-1]
    inter = gate_weight.shape[0]
    if gate_weight.shape != (inter, hidden) or up_weight.shape != (inter, hidden) or down_weight.shape != (hidden, inter):
        raise ValueError("expected gate_weight/up_weight (intermediate, hidden) and down_weight (hidden, intermediate)")
    dtype = x.dtype
    for name, t in (("gate_weight", gate_weight), ("up_weight", up_weight), ("down_weight", down_weight)):
        if t.dtype != dtype:
            raise TypeError(f"{name} has dtype {t.dtype}, x has {dtype}")
    dev = _C.require_gpu(x, gate_weight, up_weight, down_weight, residual)
    x2 = x.contiguous().view(-1, hidden)
    num_tokens = x2.shape[0]
    res = None
    if residual is not None:
        if residual.shape != x.shape or residual.dtype != dtype:
            raise ValueError("residual must have the shape and dtype of x")
        res = residual.contiguous().view(-1, hidden)
    wg, wu, wd = gate_weight.contiguous(), up_weight.contiguous(), down_weight.contiguous()
    code = _C.dtype_code(dtype)
    out = torch.empty_like(x2)
    L = _C.lib()
    ws_bytes = L.fmoe_mlp_workspace_bytes(num_tokens, hidden, inter, code)
    ws = torch.empty(max(ws_bytes, 1), device=dev, dtype=torch.uint8)
    with torch.cuda.device(dev):
        status = L.fmoe_mlp_forward(
            _C.ptr(x2), _C.ptr(wg), _C.ptr(wu), _C.ptr(wd), num_tokens, hidden, inter, code, _C.ptr(res),
            _C.ptr(out), _C.ptr(ws), ws_bytes, _C.current_stream(dev),
        )
    _C.check(status, "flash_mlp")
    return out.view(x.shape)


def mlp_forward_saving(x, gate_weight, up_weight, down_weight, residual: Optional[torch.Tensor] = None):
    """``mlp_forward`` that also returns the [2, T, I] gate and up products for ``mlp_backward`` (``fmoe_mlp_gate_up_save``
    then ``fmoe_mlp_down``), as the reference's SwiGLU function saves them (flash_moe/ops/triton/flash_mlp.py:153-159)."""
    hidden, inter = x.shape[-1], gate_weight.shape[0]
    if gate_weight.shape != (inter, hidden) or up_weight.shape != (inter, hidden) or down_weight.shape != (hidden, inter):
        raise ValueError("expected gate_weight/up_weight (intermediate, hidden) and down_weight (hidden, intermediate)")
    if any(t.dtype != x.dtype for t in (gate_weight, up_weight, down_weight)):
        raise TypeError(f"all weights must have the dtype of x ({x.dtype})")
    dev = _C.require_gpu(x, gate_weight, up_weight, down_weight, residual)
    x2 = x.contiguous().view(-1, hidden)
    res = None
    if residual is not None:
        if residual.shape != x.shape or residual.dtype != x.dtype:
            raise ValueError("residual must have the shape and dtype of x")
        res = residual.contiguous().view(-1, hidden)
    wg, wu, wd = gate_weight.contiguous(), up_weight.contiguous(), down_weight.contiguous()
    num_tokens, code = x2.shape[0], _C.dtype_code(x.dtype)
    act = torch.empty((num_tokens, inter), device=dev, dtype=x.dtype)
    saved = torch.empty((2, num_tokens, inter), device=dev, dtype=x.dtype)
    out = torch.empty_like(x2)
    L = _C.lib()
    with torch.cuda.device(dev):
        stream = _C.current_stream(dev)
        _C.check(L.fmoe_mlp_gate_up_save(_C.ptr(x2), _C.ptr(wg), _C.ptr(wu), num_tokens, hidden, inter, code, _C.ptr(act),
                                         _C.ptr(saved), stream), "flash_mlp")
        _C.check(L.fmoe_mlp_down(_C.ptr(act), _C.ptr(wd), num_tokens, hidden, inter, code, _C.ptr(res), _C.ptr(out), stream), "flash_mlp")
    return out.view(x.shape), saved


def mlp_backward(dout, x, gate_weight, up_weight, down_weight, saved=None):
    """Gradients ``(dx, dgate_weight, dup_weight, ddown_weight)`` of ``mlp_forward`` without residual
    (``fmoe_mlp_backward``): the gate and up products come from ``saved`` (``mlp_forward_saving``) or are recomputed, the
    SwiGLU gradient is the fused kernel behind ``swiglu_backward``, the transposed-operand GEMMs are rocBLAS calls
    inside the library."""
    hidden, inter = x.shape[-1], gate_weight.shape[0]
    dev = _C.require_gpu(dout, x, gate_weight, up_weight, down_weight)
    if dout.shape != x.shape or dout.dtype != x.dtype:
        raise ValueError("the output gradient must have the shape and dtype of x")
    x2, dy = x.contiguous().view(-1, hidden), dout.contiguous().view(-1, hidden)
    wg, wu, wd = gate_weight.contiguous(), up_weight.contiguous(), down_weight.contiguous()
    num_tokens = x2.shape[0]
    code = _C.dtype_code(x.dtype)
    if saved is not None and (saved.shape != (2, num_tokens, inter) or saved.dtype != x.dtype or not saved.is_contiguous()):
        raise ValueError("saved must be the contiguous [2, T, I] tensor mlp_forward_saving returned")
    # the two [I, H] gradients sit behind each other in one buffer: the library then forms them as one [2I, H] product
    dwgu = torch.empty((2 * inter, hidden), device=wg.device, dtype=wg.dtype)
    dwg, dwu = dwgu[:inter], dwgu[inter:]
    dx, dwd = torch.empty_like(x2), torch.empty_like(wd)
    if num_tokens == 0:
        return dx.view(x.shape), dwg.zero_(), dwu.zero_(), dwd.zero_()
    L = _C.lib()
    ws_bytes = L.fmoe_mlp_backward_workspace_bytes(num_tokens, hidden, inter, code)
    ws = torch.empty(max(ws_bytes, 1), device=dev, dtype=torch.uint8)
    with torch.cuda.device(dev):
        status = L.fmoe_mlp_backward(
            _C.ptr(dy), _C.ptr(x2), _C.ptr(wg), _C.ptr(wu), _C.ptr(wd), _C.ptr(saved), num_tokens, hidden, inter, code, _C.ptr(dx),
            _C.ptr(dwg), _C.ptr(dwu), _C.ptr(dwd), _C.ptr(ws), ws_bytes, _C.current_stream(dev),
        )
    _C.check(status, "flash_mlp backward")
    return dx.view(x.shape), dwg, dwu, dwd


def swiglu_backward(a: torch.Tensor, b: torch.Tensor, dc: torch.Tensor):
    """``(da, db)`` for ``c = silu(a) * b`` (``fmoe_swiglu_backward``; flash_moe/ops/triton/flash_mlp.py:126-150)."""
    if a.shape != b.shape or a.shape != dc.shape or a.dtype != b.dtype or a.dtype != dc.dtype:
        raise ValueError("a, b and dc must have one shape and dtype")
    dev = _C.require_gpu(a, b, dc)
    cols = a.shape[-1]
    a2, b2, dc2 = (t.contiguous().view(-1, cols) for t in (a, b, dc))
    da, db = torch.empty_like(a2), torch.empty_like(b2)
    with torch.cuda.device(dev):
        status = _C.lib().fmoe_swiglu_backward(_C.ptr(dc2), _C.ptr(a2), _C.ptr(b2), a2.shape[0], cols, _C.dtype_code(a.dtype),
                                               _C.ptr(da), _C.ptr(db), _C.current_stream(dev))
    _C.check(status, "swiglu backward")
    return da.view(a.shape), db.view(a.shape)


class FlashMLPFunc(torch.autograd.Function):
    @staticmethod
    @ensure_contiguous
    def forward(ctx, x, gate_weight, up_weight, down_weight):
        if not any(ctx.needs_input_grad):
            return mlp_forward(x, gate_weight, up_weight, down_weight)
        if x.numel() == 0:
            # nothing to keep for an empty batch: the backward returns zero gradients of the right shapes
            ctx.save_for_backward(x, gate_weight, up_weight, down_weight)
            return mlp_forward(x, gate_weight, up_weight, down_weight)
        out, saved = mlp_forward_saving(x, gate_weight, up_weight, down_weight)
        ctx.save_for_backward(x, gate_weight, up_weight, down_weight, saved)
        return out

    @staticmethod
    @ensure_contiguous
    def backward(ctx, dout):
        x, gate_weight, up_weight, down_weight, *rest = ctx.saved_tensors
        return mlp_backward(dout, x, gate_weight, up_weight, down_weight, rest[0] if rest else None)


def flash_mlp_func(x: torch.Tensor, gate_weight: torch.Tensor, up_weight: torch.Tensor, down_weight: torch.Tensor) -> torch.Tensor:
    return FlashMLPFunc.apply(x, gate_weight, up_weight, down_weight)
