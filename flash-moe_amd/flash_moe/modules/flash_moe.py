"""``FlashMoE`` block on the HIP forward path.

Drop-in for ``flash_moe.modules.flash_moe`` of flash-algo/flash-moe: ``FlashMoEConfig`` takes the same
six arguments (flash_moe/modules/flash_moe.py:12-27), ``FlashMoE`` owns parameters and buffers under
the same ``state_dict`` names (:43-53) and ``forward`` returns the same ``(hidden_states, router_logits)``
pair (:55-105).

``forward`` is one call of ``fmoe_block_forward``, whose stages are those of the per-op entry points:
  batch-norm, router gate, log-softmax, product-key top-k, gates    ``fmoe_router_forward``
  routed experts                                                    ``fmoe_expert_forward``
  shared SwiGLU MLP + add                                           ``fmoe_mlp_forward`` (the add is the second
                                                                    GEMM's epilogue)
``forward_staged`` runs the same three stages as three calls.  When gradients are being recorded ``forward`` takes
``forward_autograd`` instead: one autograd node whose forward is those three calls (keeping what the backward needs)
and whose backward is the library's backward calls.  ``forward_autograd_ops`` is the reference's own composition
(batch norm + router gate, log-softmax, then the router, expert and MLP ops, flash_moe/modules/flash_moe.py:62-101) on the
differentiable per-op functions; both give the same gradients.

Routing is evaluated in fp32 whatever the module dtype: the normalised activations are rounded to the
module dtype exactly as the reference does, but their product with the router gate, the log-softmax
and the pair sums stay in fp32.  With 16-bit log-probabilities the pair sums of the reference are
tie-dominated (values near -10 are 2^-4 apart in bf16) and which of the tied experts it picks is not
defined; fp32 scores make the selection well defined.  The returned ``router_logits`` are rounded to
the module dtype as in the reference.
"""
from __future__ import annotations

import math

import torch
import torch.nn as nn
import torch.nn.functional as F

from flash_moe.ops.hip.flash_block import block_forward, block_forward_autograd
from flash_moe.ops.hip.flash_expert import expert_forward, flash_expert_func
from flash_moe.ops.hip.flash_mlp import flash_mlp_func, mlp_forward
from flash_moe.ops.hip.flash_router import flash_router_func, router_forward, router_prologue

_SILU_NAMES = ("silu", "swish")


class FlashMoEConfig:
    """Plain configuration record; argument order and names as in the reference."""

    def __init__(self, hidden_size: int, intermediate_size: int, hidden_act: str, num_experts: int,
                 num_experts_per_tok: int, norm_topk_prob: bool = False):
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.hidden_act = hidden_act
        self.num_experts = num_experts
        self.num_experts_per_tok = num_experts_per_tok
        self.norm_topk_prob = norm_topk_prob

    def __repr__(self) -> str:
        body = ", ".join(f"{k}={v!r}" for k, v in vars(self).items())
        return f"FlashMoEConfig({body})"


class FlashMoE(nn.Module):
    def __init__(self, config: FlashMoEConfig):
        super().__init__()
        if config.hidden_act not in _SILU_NAMES:
            # the fused kernels hard-code SiLU, as the reference's do (flash_expert.py:8-10, flash_mlp.py:8-10)
            raise ValueError(f"hidden_act={config.hidden_act!r}: the HIP kernels implement 'silu' only")
        H, I, E = config.hidden_size, config.intermediate_size, config.num_experts
        self.hidden_size, self.intermediate_size, self.num_experts = H, I, E
        self.act_fn = F.silu
        # experts are addressed by a pair of sub-keys; ids >= num_keys**2 are never selected (:38)
        self.num_keys = math.floor(math.sqrt(E))
        self.top_k = config.num_experts_per_tok
        self.norm_topk_prob = config.norm_topk_prob

        self.gate_proj = nn.Linear(H, I, bias=False)
        self.up_proj = nn.Linear(H, I, bias=False)
        self.down_proj = nn.Linear(I, H, bias=False)

        self.router_gate = nn.Linear(H, 2 * self.num_keys, bias=False)
        self.router_norm = nn.BatchNorm1d(H, affine=False)

        self.down_embed = nn.Embedding(E, H)
        self.up_embed = nn.Embedding(E, H)

    def route(self, tokens: torch.Tensor, return_logits32: bool = False):
        """[T, H] -> (router_logits [2, T, nk] in the module dtype, scores fp32, indices int64, gates); with
        ``return_logits32`` also the fp32 gate output [T, 2*nk] the routing was computed from.  Like any forward call
        this updates the batch-norm running statistics in training mode."""
        out = router_forward(tokens, self.router_gate.weight, self.router_norm, self.num_keys, self.top_k,
                             self.norm_topk_prob, return_logits32)
        router_logits = out[0].view(tokens.shape[0], 2, self.num_keys).transpose(0, 1)
        return (router_logits,) + tuple(out[1:])

    def forward(self, hidden_states: torch.Tensor, **kwargs):
        if torch.is_grad_enabled() and (hidden_states.requires_grad or any(p.requires_grad for p in self.parameters())):
            return self.forward_autograd(hidden_states)
        bsz, seq_len, _ = hidden_states.shape
        tokens = hidden_states.reshape(bsz * seq_len, self.hidden_size)
        out, logits = block_forward(
            tokens, self.gate_proj.weight, self.up_proj.weight, self.down_proj.weight, self.router_gate.weight,
            self.router_norm, self.down_embed.weight, self.up_embed.weight, self.num_keys, self.top_k, self.norm_topk_prob,
        )
        router_logits = logits.view(tokens.shape[0], 2, self.num_keys).transpose(0, 1)
        return out.view(bsz, seq_len, self.hidden_size), router_logits

    def forward_autograd(self, hidden_states: torch.Tensor):
        """Differentiable forward: one autograd node around the library's forward and backward calls."""
        bsz, seq_len, _ = hidden_states.shape
        tokens = hidden_states.reshape(bsz * seq_len, self.hidden_size)
        num_tokens = tokens.shape[0]
        if num_tokens == 0 or self.top_k == 0:
            return self.forward_autograd_ops(hidden_states)
        out, logits = block_forward_autograd(
            tokens, self.gate_proj.weight, self.up_proj.weight, self.down_proj.weight, self.router_gate.weight,
            self.router_norm, self.down_embed.weight, self.up_embed.weight, self.num_keys, self.top_k, self.norm_topk_prob,
        )
        router_logits = logits.view(num_tokens, 2, self.num_keys).transpose(0, 1)
        return out.view(bsz, seq_len, self.hidden_size), router_logits

    def forward_autograd_ops(self, hidden_states: torch.Tensor):
        """Differentiable forward op by op, as the reference composes it (flash_moe/modules/flash_moe.py:62-101): the
        differentiable router prologue, torch's log-softmax, then the router, expert and MLP functions.  Routing is
        evaluated in fp32 as on the fused path: the normalised activations are rounded to the module dtype, their product
        with the router gate and the log-softmax are fp32."""
        bsz, seq_len, _ = hidden_states.shape
        tokens = hidden_states.reshape(bsz * seq_len, self.hidden_size)
        num_tokens = tokens.shape[0]
        if num_tokens == 0:
            logits32 = F.linear(self.router_norm(tokens).float(), self.router_gate.weight.float())
            logits = logits32.to(tokens.dtype)
        else:
            logits32, logits = router_prologue(tokens, self.router_gate.weight, self.router_norm)
        router_logits = logits.view(num_tokens, 2, self.num_keys).transpose(0, 1)
        log_probs = F.log_softmax(logits32.view(num_tokens, 2, self.num_keys), dim=-1).transpose(0, 1)
        scores, indices = flash_router_func(log_probs, self.num_keys, self.top_k)
        gates = torch.exp(scores)
        if self.norm_topk_prob:
            gates = gates / gates.sum(dim=-1, keepdim=True)
        experts_states = flash_expert_func(tokens, self.down_embed.weight, self.up_embed.weight, indices, gates.to(tokens.dtype))
        out = flash_mlp_func(tokens, self.gate_proj.weight, self.up_proj.weight, self.down_proj.weight) + experts_states
        return out.view(bsz, seq_len, self.hidden_size), router_logits

    def forward_staged(self, hidden_states: torch.Tensor):
        """``forward`` as three library calls (router, experts, MLP) instead of one; same results."""
        bsz, seq_len, _ = hidden_states.shape
        tokens = hidden_states.reshape(bsz * seq_len, self.hidden_size)
        router_logits, _, indices, gates = self.route(tokens)
        experts_states = expert_forward(tokens, self.down_embed.weight, self.up_embed.weight, indices, gates)
        out = mlp_forward(
            tokens, self.gate_proj.weight, self.up_proj.weight, self.down_proj.weight, residual=experts_states
        )
        return out.view(bsz, seq_len, self.hidden_size), router_logits
