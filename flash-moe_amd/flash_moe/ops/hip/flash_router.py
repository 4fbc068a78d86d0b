"""Product-key router op: top-k over the nk*nk pair sums of two per-token score vectors.

Same call signature, return values and argument checks as ``triton_flash_router_func``
(flash_moe/ops/triton/flash_router.py:381-382; contract docs/flash_router.md:16-40); the work is done
by ``fmoe_router_topk`` in libflashmoe_hip.so.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from flash_moe import _C
from flash_moe.ops.utils import ensure_contiguous


def router_topk_gates(
    router_logits: torch.Tensor,
    num_expert_keys: int,
    num_experts_per_tok: int,
    with_gates: bool = False,
    norm_topk_prob: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    """Launch the router kernel.  Returns ``(scores, indices, gates-or-None)``.

    ``gates = exp(scores)`` (divided by its per-token sum if ``norm_topk_prob``) is what
    FlashMoE.forward computes right after the router (flash_moe/modules/flash_moe.py:80-85); asking
    for it here saves two or three elementwise launches.
    """
    # the three checks of _flash_router_forward (flash_router.py:257-263), same exception type
    assert router_logits.dim() == 3, (
        "router_logits must be a 3D tensor of shape (2, batch_size * seq_len, num_expert_keys)"
    )
    assert router_logits.size(0) == 2, "The first dimension of router_logits must be 2"
    assert 0 <= num_experts_per_tok <= num_expert_keys, (
        f"num_experts_per_tok should be in [0, {num_expert_keys}], but got {num_experts_per_tok}"
    )
    if router_logits.size(2) != num_expert_keys:
        raise ValueError(
            f"router_logits.size(-1)={router_logits.size(2)} does not match num_expert_keys={num_expert_keys}"
        )
    dev = _C.require_gpu(router_logits)
    lp = router_logits.contiguous()
    num_tokens = lp.size(1)
    scores = torch.empty((num_tokens, num_experts_per_tok), device=dev, dtype=lp.dtype)
    indices = torch.empty((num_tokens, num_experts_per_tok), device=dev, dtype=torch.int64)
    gates = torch.empty_like(scores) if with_gates else None
    with torch.cuda.device(dev):
        status = _C.lib().fmoe_router_topk(
            _C.ptr(lp), num_tokens, num_expert_keys, num_experts_per_tok, _C.dtype_code(lp.dtype),
            _C.ptr(scores), _C.ptr(indices), _C.ptr(gates), int(bool(norm_topk_prob)), _C.current_stream(dev),
        )
    _C.check(status, "flash_router")
    return scores, indices, gates


def check_router_args(tokens, gate_weight, norm, num_expert_keys, num_experts_per_tok, split_query=False):
    """Argument checks of the fused routing stage; returns ``(device, training)``."""
    width = tokens.shape[1] // 2 if split_query else tokens.shape[1]
    if tokens.dim() != 2 or gate_weight.shape != (2 * num_expert_keys, width):
        raise ValueError("expected tokens [T, H] and a router gate weight [2*num_expert_keys, H] "
                         "([2*num_expert_keys, H/2] sub-key tables with split_query)")
    assert 0 <= num_experts_per_tok <= num_expert_keys, (
        f"num_experts_per_tok should be in [0, {num_expert_keys}], but got {num_experts_per_tok}"
    )
    if gate_weight.dtype != tokens.dtype:
        raise TypeError(f"router gate weight has dtype {gate_weight.dtype}, tokens have {tokens.dtype}")
    if norm.affine or norm.momentum is None or not norm.track_running_stats:
        raise ValueError("the fused router expects BatchNorm1d(affine=False, momentum=<float>, track_running_stats=True)")
    training = bool(norm.training)
    if training and tokens.shape[0] == 1:
        raise ValueError(f"Expected more than 1 value per channel when training, got input size {tuple(tokens.shape)}")
    rm, rv = norm.running_mean, norm.running_var
    if not (rm.is_contiguous() and rv.is_contiguous() and rm.dtype == rv.dtype):
        raise ValueError("running statistics must be contiguous and of one dtype")
    return _C.require_gpu(tokens, gate_weight, rm, rv), training


def router_forward(tokens: torch.Tensor, gate_weight: torch.Tensor, norm: torch.nn.BatchNorm1d, num_expert_keys: int,
                   num_experts_per_tok: int, norm_topk_prob: bool = False, return_logits32: bool = False,
                   return_stats: bool = False, split_query: bool = False):
    """The block's whole routing stage in one call of ``fmoe_router_forward``: batch-norm (training or evaluation
    mode, taken from ``norm.training``; its running statistics are updated in place), the router gate, the per-half
    log-softmax, the product-key top-k and the gates (flash_moe/modules/flash_moe.py:62-85).

    Returns ``(router_logits [T, 2*nk] in tokens.dtype, scores [T,K] fp32, indices [T,K] int64, gates [T,K] in
    tokens.dtype)``, plus the fp32 logits the routing was computed from when ``return_logits32`` is set, plus the
    batch-norm mean and 1/sqrt(var + eps) used ([2*H] fp32, a view of the call's workspace) when ``return_stats`` is set.
    ``split_query``: ``gate_weight`` is two sub-key tables [2*nk, H/2], each scoring its own half of the normalised query
    (``fmoe_router_forward_split``; equal to a block-diagonal [2*nk, H] gate); the module never uses this form.
    """
    dev, training = check_router_args(tokens, gate_weight, norm, num_expert_keys, num_experts_per_tok, split_query)
    T, H = tokens.shape
    x, w = tokens.contiguous(), gate_weight.contiguous()
    K = num_experts_per_tok
    logits = torch.empty((T, 2 * num_expert_keys), device=dev, dtype=x.dtype)
    logits32 = torch.empty((T, 2 * num_expert_keys), device=dev, dtype=torch.float32)
    scores = torch.empty((T, K), device=dev, dtype=torch.float32)
    indices = torch.empty((T, K), device=dev, dtype=torch.int64)
    gates = torch.empty((T, K), device=dev, dtype=x.dtype)
    L = _C.lib()
    ws_bytes = L.fmoe_router_workspace_bytes(T, H, num_expert_keys)
    ws = torch.empty(max(ws_bytes, 1), device=dev, dtype=torch.uint8)
    rm, rv, nbt = norm.running_mean, norm.running_var, norm.num_batches_tracked
    with torch.cuda.device(dev):
        status = (L.fmoe_router_forward_split if split_query else L.fmoe_router_forward)(
            _C.ptr(x), _C.ptr(w), _C.ptr(rm), _C.ptr(rv), _C.ptr(nbt), _C.dtype_code(rm.dtype), int(training),
            float(norm.momentum), float(norm.eps), T, H, num_expert_keys, K, _C.dtype_code(x.dtype),
            int(bool(norm_topk_prob)), _C.ptr(logits), _C.ptr(logits32), _C.ptr(scores), _C.ptr(indices), _C.ptr(gates),
            _C.ptr(ws), ws_bytes, _C.current_stream(dev),
        )
    _C.check(status, "flash_router")
    result = (logits, scores, indices, gates)
    if return_logits32:
        result += (logits32,)
    if return_stats:
        off = L.fmoe_router_workspace_stats_offset(T, H, num_expert_keys)
        result += (ws[off:off + 2 * H * 4].view(torch.float32),)
    return result


class RouterPrologueFunc(torch.autograd.Function):
    """Differentiable router prologue ``logits = BatchNorm1d(x) @ gate_weight.T`` (flash_moe/modules/flash_moe.py:62-67).

    Forward: the batch-norm and gate launches of ``fmoe_router_forward`` (top_k = 0); returns the fp32 logits the routing
    is computed from and their rounding to the activation dtype (what the module returns).  Backward:
    ``fmoe_router_prologue_backward``.  ``norm``'s running statistics are updated in training mode, as by any forward."""

    @staticmethod
    def forward(ctx, tokens, gate_weight, norm):
        num_expert_keys = gate_weight.shape[0] // 2
        dev, training = check_router_args(tokens, gate_weight, norm, num_expert_keys, 0)
        x, w = tokens.contiguous(), gate_weight.contiguous()
        T, H = x.shape
        logits = torch.empty((T, 2 * num_expert_keys), device=dev, dtype=x.dtype)
        logits32 = torch.empty((T, 2 * num_expert_keys), device=dev, dtype=torch.float32)
        L = _C.lib()
        ws_bytes = L.fmoe_router_workspace_bytes(T, H, num_expert_keys)
        ws = torch.empty(max(ws_bytes, 1), device=dev, dtype=torch.uint8)
        rm, rv, nbt = norm.running_mean, norm.running_var, norm.num_batches_tracked
        with torch.cuda.device(dev):
            status = L.fmoe_router_forward(
                _C.ptr(x), _C.ptr(w), _C.ptr(rm), _C.ptr(rv), _C.ptr(nbt), _C.dtype_code(rm.dtype), int(training),
                float(norm.momentum), float(norm.eps), T, H, num_expert_keys, 0, _C.dtype_code(x.dtype), 0, _C.ptr(logits),
                _C.ptr(logits32), None, None, None, _C.ptr(ws), ws_bytes, _C.current_stream(dev),
            )
        _C.check(status, "router prologue")
        off = L.fmoe_router_workspace_stats_offset(T, H, num_expert_keys)
        stats = ws[off:off + 2 * H * 4].view(torch.float32).clone()        # mean, 1/sqrt(var + eps): [2*H]
        ctx.save_for_backward(x, w, stats)
        ctx.training, ctx.num_expert_keys = training, num_expert_keys
        return logits32, logits

    @staticmethod
    def backward(ctx, dlogits32, dlogits):
        x, w, stats = ctx.saved_tensors
        grad = None
        for g in (dlogits32, dlogits):
            if g is not None:
                grad = g.float() if grad is None else grad + g.float()
        if grad is None:
            return None, None, None
        dx, dw = router_prologue_backward(grad, x, w, stats, ctx.training)
        return dx, dw, None


def router_prologue_backward(dlogits32: torch.Tensor, tokens: torch.Tensor, gate_weight: torch.Tensor, stats: torch.Tensor,
                             training: bool):
    """``(dtokens, dgate_weight)`` of ``logits = BatchNorm1d(tokens) @ gate_weight.T`` from the fp32 gradient of the logits
    [T, 2*nk] and the forward's batch-norm statistics ``stats`` ([2*H] fp32: mean, 1/sqrt(var + eps));
    ``fmoe_router_prologue_backward``."""
    x, w, grad = tokens.contiguous(), gate_weight.contiguous(), dlogits32.contiguous()
    T, H = x.shape
    num_expert_keys = w.shape[0] // 2
    if grad.shape != (T, 2 * num_expert_keys) or grad.dtype != torch.float32:
        raise ValueError("expected an fp32 gradient of shape [T, 2*num_expert_keys]")
    dev = _C.require_gpu(x, w, grad, stats)
    code = _C.dtype_code(x.dtype)
    dx, dw = torch.empty_like(x), torch.empty_like(w)
    L = _C.lib()
    ws_bytes = L.fmoe_router_prologue_backward_workspace_bytes(T, H, num_expert_keys, code)
    ws = torch.empty(max(ws_bytes, 1), device=dev, dtype=torch.uint8)
    with torch.cuda.device(dev):
        status = L.fmoe_router_prologue_backward(_C.ptr(grad), _C.ptr(x), _C.ptr(w), _C.ptr(stats), int(training), T, H,
                                                 num_expert_keys, code, _C.ptr(dx), _C.ptr(dw), _C.ptr(ws), ws_bytes,
                                                 _C.current_stream(dev))
    _C.check(status, "router prologue backward")
    return dx, dw


def route_backward(dgates: torch.Tensor, indices: torch.Tensor, logits32: torch.Tensor, num_expert_keys: int,
                   norm_topk_prob: bool = False, dlogits: torch.Tensor = None) -> torch.Tensor:
    """Gradient of the fp32 gate logits [T, 2*nk] from the gradient of the gates [T, K] (``fmoe_route_backward``): the
    backward of per-half log-softmax, product-key top-k, exp and optional renormalisation
    (flash_moe/modules/flash_moe.py:69-85) in one launch.  ``dlogits`` ([T, 2*nk] in the gates' dtype), the gradient of the
    router logits the block returns, is added when given."""
    if dgates.dim() != 2 or indices.shape != dgates.shape or indices.dtype != torch.int64:
        raise ValueError("expected dgates [T, K] and int64 indices of the same shape")
    T, K = dgates.shape
    if logits32.shape != (T, 2 * num_expert_keys) or logits32.dtype != torch.float32:
        raise ValueError("expected fp32 logits of shape [T, 2*num_expert_keys]")
    if dlogits is not None and (dlogits.shape != logits32.shape or dlogits.dtype != dgates.dtype):
        raise ValueError("dlogits must have the shape of the logits and the dtype of dgates")
    dev = _C.require_gpu(dgates, indices, logits32, dlogits)
    dg, idx, lg = dgates.contiguous(), indices.contiguous(), logits32.contiguous()
    extra = dlogits.contiguous() if dlogits is not None else None
    out = torch.empty_like(lg)
    with torch.cuda.device(dev):
        status = _C.lib().fmoe_route_backward(_C.ptr(dg), _C.ptr(idx), _C.ptr(lg), _C.ptr(extra), T, num_expert_keys, K,
                                              _C.dtype_code(dg.dtype), int(bool(norm_topk_prob)), _C.ptr(out),
                                              _C.current_stream(dev))
    _C.check(status, "route backward")
    return out


def router_prologue(tokens: torch.Tensor, gate_weight: torch.Tensor, norm: torch.nn.BatchNorm1d):
    """``(logits_fp32 [T, 2*nk], logits [T, 2*nk] in tokens.dtype)``, differentiable with respect to tokens and gate_weight."""
    return RouterPrologueFunc.apply(tokens, gate_weight, norm)


def router_topk_backward(dscores: torch.Tensor, indices: torch.Tensor, num_expert_keys: int) -> torch.Tensor:
    """Scatter of ``dscores`` [T, K] onto the two halves' keys -> [2, T, nk] in ``dscores.dtype`` (``fmoe_router_topk_backward``)."""
    if dscores.dim() != 2 or indices.shape != dscores.shape or indices.dtype != torch.int64:
        raise ValueError("expected dscores [T, K] and int64 indices of the same shape")
    dev = _C.require_gpu(dscores, indices)
    ds, idx = dscores.contiguous(), indices.contiguous()
    T, K = ds.shape
    out = torch.empty((2, T, num_expert_keys), device=dev, dtype=ds.dtype)
    with torch.cuda.device(dev):
        status = _C.lib().fmoe_router_topk_backward(_C.ptr(ds), _C.ptr(idx), T, num_expert_keys, K, _C.dtype_code(ds.dtype),
                                                    _C.ptr(out), _C.current_stream(dev))
    _C.check(status, "flash_router backward")
    return out


class FlashRouterFunc(torch.autograd.Function):
    @staticmethod
    @ensure_contiguous
    def forward(ctx, router_logits, num_expert_keys, num_experts_per_tok):
        """router_logits [2, T, nk] -> scores [T, K] (dtype of the input), indices [T, K] int64."""
        scores, indices, _ = router_topk_gates(router_logits, num_expert_keys, num_experts_per_tok)
        ctx.mark_non_differentiable(indices)
        ctx.save_for_backward(indices)
        ctx.num_expert_keys = num_expert_keys
        return scores, indices

    @staticmethod
    @ensure_contiguous
    def backward(ctx, dscores, dindices):
        """drouter_logits [2, T, nk]: each selected pair's gradient goes to its two keys
        (flash_moe/ops/triton/flash_router.py:317-344); no gradient for the two integers."""
        (indices,) = ctx.saved_tensors
        return router_topk_backward(dscores, indices, ctx.num_expert_keys), None, None


def flash_router_func(router_logits, num_expert_keys, num_experts_per_tok):
    return FlashRouterFunc.apply(router_logits, num_expert_keys, num_experts_per_tok)
