"""CPU oracle for the FlashMoE forward path.  TEST INFRASTRUCTURE ONLY.

This file restates, with stock ``torch`` routines on the CPU, the eager forward path of the
reference (flash-algo/flash-moe).  Only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import it; the product package never does.

Every function names the reference lines it follows.  What pins each function (so a dropped
term, a wrong sign or a transposed operand fails a test that does not retype the formula):

* ``router_prologue``   batch-norm closed forms (train: per-feature mean 0 / biased variance 1,
                        running-stat update rule; eval: running stats), ``logsumexp(lp) == 0``,
                        half h of the output equals features ``[h*nk, (h+1)*nk)`` of the gate.
* ``router_topk``       brute force over all nk*nk sums (independent C implementation in
                        ``oracle/bruteforce.c`` and a numpy argsort), closed-form cases (one
                        dominant key per half, K = 1, K = nk).
* ``routing_weights``   row sums equal 1 when normalised; equals ``p_x * p_y`` otherwise.
* ``expert_forward``    float64 loop implementation in ``oracle/bruteforce.c``; special cases
                        (zero gates, one expert repeated, linearity in the gates, permutation of k).
* ``mlp_forward``       float64 loop implementation in ``oracle/bruteforce.c``.
* ``expert_bucketing``  exhaustive C scan in ``oracle/bruteforce.c`` (for every expert, every pair in index
                        order), invariants (offsets monotone, ``offsets[E]`` = number of valid pairs, each
                        segment one expert, the pairs a permutation), a numpy ``argsort(kind="stable")``.
* ``peer_forward``, ``pkm_forward``   float64 loops in ``oracle/bruteforce.c`` (``erf`` of the C library),
                        closed forms (a unit weight copies a row; gelu(s) - gelu(-s) = s).
* ``block_forward``     composition of the above; equality with calling the stages one by one.

The reference holds no golden vectors or asserting tests for this path (its tests only print),
so the fixtures under ``tests/golden`` are written by this oracle after the pins above pass.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional, Tuple

import torch
import torch.nn.functional as F


# --------------------------------------------------------------------------------------
# router
# --------------------------------------------------------------------------------------
def router_prologue(
    hidden: torch.Tensor,
    router_gate_weight: torch.Tensor,
    num_keys: int,
    running_mean: Optional[torch.Tensor] = None,
    running_var: Optional[torch.Tensor] = None,
    training: bool = True,
    momentum: float = 0.1,
    eps: float = 1e-5,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """BatchNorm1d(affine=False) -> Linear(H, 2*nk, no bias) -> [2, T, nk] view -> log_softmax.

    Follows flash_moe/modules/flash_moe.py:147-156 (same statements as :65-72 of the fused
    module).  ``hidden`` is [T, H].  Returns ``(router_logits, router_log_probs)``, both
    [2, T, nk]; ``router_logits`` is the transposed view the module returns to its caller.
    In training mode the running statistics, when given, are updated in place exactly as
    ``torch.nn.BatchNorm1d`` does (momentum 0.1, unbiased variance in the running estimate).
    """
    q = F.batch_norm(
        hidden,
        running_mean,
        running_var,
        weight=None,
        bias=None,
        training=training or running_mean is None,
        momentum=momentum,
        eps=eps,
    )
    logits = F.linear(q, router_gate_weight)                      # [T, 2*nk]
    logits = logits.view(hidden.shape[0], 2, num_keys).transpose(0, 1)   # [2, T, nk]
    return logits, F.log_softmax(logits, dim=-1)


def router_topk(log_probs: torch.Tensor, num_keys: int, top_k: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Top-k over the nk*nk pair sums ``lp[0,t,i] + lp[1,t,j]``; flat index ``i*nk + j``.

    Follows flash_moe/modules/flash_moe.py:159-167 and tests/test_router.py:8-16: a full
    descending ``topk(nk)`` of each half, the dense [T, nk, nk] sums in the input dtype, then
    ``topk(K)`` and a gather of the flat indices.  Tie order is whatever ``torch.topk`` gives.
    """
    (sx, sy), (ix, iy) = log_probs.topk(num_keys, dim=-1)
    sums = sx.unsqueeze(-1) + sy.unsqueeze(-2)                    # [T, nk, nk]
    flat = ix.unsqueeze(-1) * num_keys + iy.unsqueeze(-2)
    sums = sums.reshape(sums.shape[0], -1)
    flat = flat.reshape(flat.shape[0], -1)
    scores, pos = sums.topk(top_k, dim=-1)
    return scores, flat.gather(-1, pos)


def routing_weights(scores: torch.Tensor, norm_topk_prob: bool) -> torch.Tensor:
    """``exp(scores)`` and the optional per-token renormalisation.

    Follows flash_moe/modules/flash_moe.py:170-175.
    """
    w = torch.exp(scores)
    if norm_topk_prob:
        w = w / w.sum(dim=-1, keepdim=True)
    return w


# --------------------------------------------------------------------------------------
# routed experts and shared MLP
# --------------------------------------------------------------------------------------
def expert_forward(
    hidden: torch.Tensor,
    down_table: torch.Tensor,
    up_table: torch.Tensor,
    indices: torch.Tensor,
    weights: torch.Tensor,
    token_chunk: int = 1024,
) -> torch.Tensor:
    """``out[t] = sum_k silu(<x_t, Wd[idx[t,k]]>) * g[t,k] * Wu[idx[t,k]]``.

    Follows flash_moe/modules/flash_moe.py:178-186 and tests/test_expert.py:21-29: two
    embedding gathers [T, K, H], a batched mat-vec, ``silu(.) * g`` and a batched vec-mat, all
    in the dtype of the inputs.  Tokens are processed in chunks only to bound the size of the
    two gathers; rows are independent so chunking does not change any value.
    """
    out = torch.empty_like(hidden)
    n = hidden.shape[0]
    for lo in range(0, n, token_chunk):
        hi = min(n, lo + token_chunk)
        idx = indices[lo:hi]
        wd = F.embedding(idx, down_table)                          # [c, K, H]
        wu = F.embedding(idx, up_table)
        s = torch.matmul(wd, hidden[lo:hi].unsqueeze(-1)).squeeze(-1)   # [c, K]
        a = F.silu(s) * weights[lo:hi]
        out[lo:hi] = torch.matmul(a.unsqueeze(-2), wu).squeeze(-2)
    return out


def expert_bucketing(indices: torch.Tensor, num_experts: int):
    """Token-centric (token, expert) pairs -> expert-centric segments.

    Follows ``_preprocess_expert_centric_indices_pytorch`` (flash_moe/ops/triton/flash_expert.py:528-577): flatten
    the pairs, sort them by expert id, permute the token ids, ``bincount`` + ``cumsum`` into ``expert_offsets``.
    Returns ``(sorted_token_ids int32 [P'], expert_offsets int32 [E+1], sorted_pair_ids int32 [P'],
    sorted_expert_ids int32 [P'])``.  Two points the reference leaves open are fixed here: the sort is stable
    (``torch.sort`` there is not), so a segment lists its pairs in ascending pair index, the canonical order every
    comparison uses; and ids outside ``[0, num_experts)`` are dropped (P' = number of valid pairs), where the
    reference would index out of bounds.
    """
    num_tokens, top_k = indices.shape
    expert_ids = indices.reshape(-1)
    valid = (expert_ids >= 0) & (expert_ids < num_experts)
    pair_ids = torch.arange(num_tokens * top_k, dtype=torch.int64)[valid]
    order = torch.sort(expert_ids[valid], stable=True)
    sorted_pair_ids = pair_ids[order.indices]
    sorted_token_ids = sorted_pair_ids // max(top_k, 1)
    counts = torch.bincount(order.values, minlength=num_experts)
    offsets = torch.zeros(num_experts + 1, dtype=torch.int32)
    offsets[1:] = torch.cumsum(counts, dim=0)
    return sorted_token_ids.int(), offsets, sorted_pair_ids.int(), order.values.int()


def peer_forward(hidden, down_table, up_table, weights, indices):
    """PEER: ``out[t] = sum_k gelu(<x_t, Wd[idx[t,k]]>) * w[t,k] * Wu[idx[t,k]]`` with the erf GELU.

    Follows the eager form of the reference's test (tests/test_peer.py:9-24): two embedding gathers, a batched
    mat-vec, ``F.gelu`` (exact, erf), the routing weight, a batched vec-mat; note the argument order (weights
    before indices) of ``triton_peer_func`` (flash_moe/ops/triton/peer.py:246-255).
    """
    wd = F.embedding(indices, down_table)
    wu = F.embedding(indices, up_table)
    s = torch.matmul(wd, hidden.unsqueeze(-1)).squeeze(-1)
    a = F.gelu(s) * weights
    return torch.matmul(a.unsqueeze(-2), wu).squeeze(-2)


def pkm_forward(values, weights, indices):
    """Product-key memory read-out ``out[t] = sum_k w[t,k] * values[idx[t,k]]``.

    Follows tests/test_pkm.py:9-20 (an embedding-bag with per-sample weights) and ``triton_pkm_func``
    (flash_moe/ops/triton/pkm.py:195-200).
    """
    return torch.matmul(weights.unsqueeze(-2), F.embedding(indices, values)).squeeze(-2)


def mlp_forward(x: torch.Tensor, gate_w: torch.Tensor, up_w: torch.Tensor, down_w: torch.Tensor) -> torch.Tensor:
    """Shared SwiGLU MLP ``(silu(x Wg^T) * (x Wu^T)) Wd^T``.

    Follows flash_moe/modules/flash_moe.py:187-189 and tests/test_mlp.py:9-19.
    """
    h = F.silu(F.linear(x, gate_w)) * F.linear(x, up_w)
    return F.linear(h, down_w)


# --------------------------------------------------------------------------------------
# whole block
# --------------------------------------------------------------------------------------
@dataclass
class BlockWeights:
    """Parameter set of one FlashMoE block, named as the module's ``state_dict`` names them
    (flash_moe/modules/flash_moe.py:43-53)."""

    gate_proj: torch.Tensor      # [I, H]
    up_proj: torch.Tensor        # [I, H]
    down_proj: torch.Tensor      # [H, I]
    router_gate: torch.Tensor    # [2*nk, H]
    down_embed: torch.Tensor     # [E, H]
    up_embed: torch.Tensor       # [E, H]
    running_mean: Optional[torch.Tensor] = None   # [H]
    running_var: Optional[torch.Tensor] = None    # [H]

    @property
    def num_keys(self) -> int:
        return self.router_gate.shape[0] // 2

    def to(self, dtype: torch.dtype) -> "BlockWeights":
        cast = lambda t: None if t is None else t.to(dtype)
        return BlockWeights(*(cast(getattr(self, f)) for f in self.__dataclass_fields__))


def make_block_weights(hidden: int, inter: int, num_experts: int, seed: int = 0, std: float = 0.02) -> BlockWeights:
    """Seeded fp32 weights ~ N(0, std) for a block; BatchNorm buffers at their initial values."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    nk = math.floor(math.sqrt(num_experts))
    rn = lambda *s: torch.randn(*s, generator=g) * std
    return BlockWeights(
        gate_proj=rn(inter, hidden),
        up_proj=rn(inter, hidden),
        down_proj=rn(hidden, inter),
        router_gate=rn(2 * nk, hidden),
        down_embed=rn(num_experts, hidden),
        up_embed=rn(num_experts, hidden),
        running_mean=torch.zeros(hidden),
        running_var=torch.ones(hidden),
    )


def block_forward(
    x: torch.Tensor,
    w: BlockWeights,
    top_k: int,
    norm_topk_prob: bool = False,
    training: bool = True,
    routing_fp32: bool = False,
    token_chunk: int = 1024,
):
    """One FlashMoE block, eager: flash_moe/modules/flash_moe.py:139-191.

    ``x`` is [B, S, H].  Returns a dict with every intermediate a parity test may want:
    ``y`` [B, S, H], ``router_logits`` [2, T, nk], ``scores``, ``indices``, ``gates``,
    ``experts`` [T, H], ``mlp`` [T, H].

    ``routing_fp32=True`` runs batch-norm as the reference does (result rounded to the dtype of
    ``x``) and then evaluates the rest of the routing stage (gate product, log-softmax, pair sums,
    exp) in fp32 on those values, rounding logits, scores and gates to the dtype of ``x`` only at
    the end.  With 16-bit log-probabilities the pair sums are tie-dominated and ``torch.topk``'s
    tie order is unspecified, so index parity is only meaningful on fp32 scores; the HIP path
    routes in fp32 and is compared in this mode.  For fp32 inputs both modes are identical.
    """
    B, S, H = x.shape
    hid = x.reshape(-1, H)
    nk = w.num_keys
    if routing_fp32:
        # batch-norm exactly as the reference runs it (output rounded to the dtype of x); everything
        # after it in fp32 on those values
        q = F.batch_norm(hid, w.running_mean, w.running_var, None, None,
                         training or w.running_mean is None, 0.1, 1e-5)
        logits = F.linear(q.float(), w.router_gate.float()).view(hid.shape[0], 2, nk).transpose(0, 1)
        lp = F.log_softmax(logits, dim=-1)
    else:
        logits, lp = router_prologue(hid, w.router_gate, nk, w.running_mean, w.running_var, training)
    scores, indices = router_topk(lp, nk, top_k)
    gates = routing_weights(scores, norm_topk_prob)
    logits, scores, gates = logits.to(x.dtype), scores.to(x.dtype), gates.to(x.dtype)
    experts = expert_forward(hid, w.down_embed, w.up_embed, indices, gates, token_chunk)
    mlp = mlp_forward(hid, w.gate_proj, w.up_proj, w.down_proj)
    y = (mlp + experts).view(B, S, H)
    return dict(y=y, router_logits=logits, scores=scores, indices=indices, gates=gates,
                experts=experts, mlp=mlp)


# --------------------------------------------------------------------------------------
# seeded synthetic inputs of the benchmark configurations (generated on the CPU in fp32, then
# cast, so that a CPU run and a GPU run see identical values)
# --------------------------------------------------------------------------------------
def make_router_inputs(num_tokens: int, num_keys: int, seed: int = 0, log_probs: bool = True) -> torch.Tensor:
    """[2, T, nk] fp32.  ``log_probs=False`` gives the raw normals tests/test_router.py:43-46 uses."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    z = torch.randn(2, num_tokens, num_keys, generator=g)
    return F.log_softmax(z, dim=-1) if log_probs else z


def make_expert_inputs(num_tokens: int, hidden: int, num_experts: int, top_k: int, seed: int = 0,
                       std: float = 0.02):
    """x ~ N(0,1); tables ~ N(0,std); per token K distinct expert ids; gates = softmax(N(0,1))."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    x = torch.randn(num_tokens, hidden, generator=g)
    wd = torch.randn(num_experts, hidden, generator=g) * std
    wu = torch.randn(num_experts, hidden, generator=g) * std
    # K distinct ids per token: top-K positions of iid uniforms == a uniform K-subset in random order
    idx = torch.rand(num_tokens, num_experts, generator=g).topk(top_k, dim=-1).indices \
        if num_tokens * num_experts <= (1 << 26) else _distinct_ids_chunked(num_tokens, num_experts, top_k, g)
    gates = torch.softmax(torch.randn(num_tokens, top_k, generator=g), dim=-1)
    return x, wd, wu, idx.to(torch.int64), gates


def _distinct_ids_chunked(num_tokens, num_experts, top_k, g, chunk=2048):
    parts = []
    for lo in range(0, num_tokens, chunk):
        n = min(chunk, num_tokens - lo)
        parts.append(torch.rand(n, num_experts, generator=g).topk(top_k, dim=-1).indices)
    return torch.cat(parts, 0)
