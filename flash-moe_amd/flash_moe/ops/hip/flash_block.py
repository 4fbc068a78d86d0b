"""The whole FlashMoE block forward as one call of ``fmoe_block_forward``.

``block_forward`` computes what FlashMoE.forward computes on the flattened tokens
(flash_moe/modules/flash_moe.py:55-105): router -> routed experts -> shared SwiGLU MLP + add.  It gives the same
results as calling ``router_forward``, ``expert_forward`` and ``mlp_forward(residual=...)`` in turn; the single call
keeps every intermediate in one workspace and skips the conversion of expert ids to table offsets.
"""
from __future__ import annotations

import torch

from flash_moe import _C
from flash_moe.ops.hip.flash_router import check_router_args


def block_forward(tokens: torch.Tensor, gate_proj: torch.Tensor, up_proj: torch.Tensor, down_proj: torch.Tensor,
                  router_gate: torch.Tensor, norm: torch.nn.BatchNorm1d, down_embed: torch.Tensor, up_embed: torch.Tensor,
                  num_expert_keys: int, num_experts_per_tok: int, norm_topk_prob: bool = False,
                  return_routing: bool = False):
    """tokens [T, H] -> ``(out [T, H], router_logits [T, 2*nk])`` in tokens.dtype, plus ``(indices int64, gates)``
    [T, K] when ``return_routing`` is set.  ``norm.training`` selects batch or running statistics; the running
    statistics are updated in place in training mode."""
    dev, training = check_router_args(tokens, router_gate, norm, num_expert_keys, num_experts_per_tok)
    T, H = tokens.shape
    I, E, K = gate_proj.shape[0], down_embed.shape[0], num_experts_per_tok
    if gate_proj.shape != (I, H) or up_proj.shape != (I, H) or down_proj.shape != (H, I):
        raise ValueError("expected gate/up projection weights [I, H] and a down projection weight [H, I]")
    if down_embed.shape != (E, H) or up_embed.shape != (E, H):
        raise ValueError("expected expert tables [E, H]")
    if num_expert_keys * num_expert_keys > E:
        raise ValueError(f"num_expert_keys**2 = {num_expert_keys ** 2} exceeds the {E} rows of the expert tables")
    weights = (gate_proj, up_proj, down_proj, router_gate, down_embed, up_embed)
    if any(w.dtype != tokens.dtype for w in weights):
        raise TypeError(f"all weights must have the tokens' dtype {tokens.dtype}")
    _C.require_gpu(tokens, *weights)
    x = tokens.contiguous()
    wg, wu, wd, wr, ed, eu = (w.contiguous() for w in weights)
    code = _C.dtype_code(x.dtype)
    out = torch.empty_like(x)
    logits = torch.empty((T, 2 * num_expert_keys), device=dev, dtype=x.dtype)
    indices = torch.empty((T, K), device=dev, dtype=torch.int64) if return_routing else None
    gates = torch.empty((T, K), device=dev, dtype=x.dtype) if return_routing else None
    L = _C.lib()
    ws_bytes = L.fmoe_block_workspace_bytes(max(T, 1), H, I, num_expert_keys, E, K, code)
    ws = torch.empty(max(ws_bytes, 1), device=dev, dtype=torch.uint8)
    rm, rv, nbt = norm.running_mean, norm.running_var, norm.num_batches_tracked
    with torch.cuda.device(dev):
        status = L.fmoe_block_forward(
            _C.ptr(x), _C.ptr(wg), _C.ptr(wu), _C.ptr(wd), _C.ptr(wr), _C.ptr(ed), _C.ptr(eu), _C.ptr(rm), _C.ptr(rv),
            _C.ptr(nbt), _C.dtype_code(rm.dtype), int(training), float(norm.momentum), float(norm.eps), T, H, I, E,
            num_expert_keys, K, code, int(bool(norm_topk_prob)), _C.ptr(out), _C.ptr(logits), _C.ptr(indices),
            _C.ptr(gates), _C.ptr(ws), ws_bytes, _C.current_stream(dev),
        )
    _C.check(status, "flash_moe block")
    if return_routing:
        return out, logits, indices, gates
    return out, logits


class FlashMoEBlockFunc(torch.autograd.Function):
    """The block with gradients for the tokens and every weight, library calls only.

    Forward: the three calls the single-call forward is made of (``fmoe_router_forward``, ``fmoe_expert_forward``,
    ``fmoe_mlp_gate_up_save`` + ``fmoe_mlp_down`` with the experts' output as residual), keeping what the backward needs:
    ids, gates, the fp32 gate logits, the batch-norm statistics and the MLP's gate / up products.  Backward:
    ``fmoe_mlp_backward``, ``fmoe_expert_backward``, ``fmoe_route_backward``, ``fmoe_router_prologue_backward`` and the
    sum of the three token gradients.  The reference reaches the same gradients through autograd of its eager ops
    around the three Triton functions (flash_moe/modules/flash_moe.py:55-105)."""

    @staticmethod
    def forward(ctx, tokens, gate_proj, up_proj, down_proj, router_gate, down_embed, up_embed, norm, num_expert_keys,
                num_experts_per_tok, norm_topk_prob):
        from flash_moe.ops.hip.flash_expert import expert_forward
        from flash_moe.ops.hip.flash_mlp import mlp_forward_saving
        from flash_moe.ops.hip.flash_router import router_forward

        x = tokens.contiguous()
        training = bool(norm.training)
        logits, _, indices, gates, logits32, stats = router_forward(
            x, router_gate, norm, num_expert_keys, num_experts_per_tok, norm_topk_prob, return_logits32=True, return_stats=True)
        experts = expert_forward(x, down_embed, up_embed, indices, gates)
        out, saved = mlp_forward_saving(x, gate_proj, up_proj, down_proj, residual=experts)
        ctx.save_for_backward(x, gate_proj, up_proj, down_proj, router_gate, down_embed, up_embed, indices, gates, logits32,
                              stats, saved)
        ctx.training, ctx.num_expert_keys, ctx.norm_topk_prob = training, num_expert_keys, bool(norm_topk_prob)
        return out, logits

    @staticmethod
    def backward(ctx, dout, dlogits):
        from flash_moe.ops.hip.flash_expert import expert_backward
        from flash_moe.ops.hip.flash_mlp import mlp_backward
        from flash_moe.ops.hip.flash_router import route_backward, router_prologue_backward

        x, wg, wu, wd, wr, ed, eu, indices, gates, logits32, stats, saved = ctx.saved_tensors
        if dout is None:
            dout = torch.zeros_like(x)
        dout = dout.contiguous()
        dx, dwg, dwu, dwd = mlp_backward(dout, x, wg, wu, wd, saved)
        dx_experts, ded, deu, dgates = expert_backward(dout, x, ed, eu, indices, gates)
        dlogits32 = route_backward(dgates, indices, logits32, ctx.num_expert_keys, ctx.norm_topk_prob, dlogits)
        dx_router, dwr = router_prologue_backward(dlogits32, x, wr, stats, ctx.training)
        dx.add_(dx_experts).add_(dx_router)
        return dx, dwg, dwu, dwd, dwr, ded, deu, None, None, None, None


def block_forward_autograd(tokens, gate_proj, up_proj, down_proj, router_gate, norm, down_embed, up_embed, num_expert_keys,
                           num_experts_per_tok, norm_topk_prob=False):
    """Differentiable ``block_forward``: ``(out [T, H], router_logits [T, 2*nk])``."""
    return FlashMoEBlockFunc.apply(tokens, gate_proj, up_proj, down_proj, router_gate, down_embed, up_embed, norm,
                                   num_expert_keys, num_experts_per_tok, norm_topk_prob)
