"""Expert-centric bucketing on the GPU (``fmoe_expert_bucket``) against the oracle's restatement of the reference's
sort / bincount / cumsum preprocessing (flash_moe/ops/triton/flash_expert.py:528-577): integer work, compared bit for
bit.  The oracle's order inside a segment (ascending pair index, a stable sort) is the library's contract too, so
nothing is canonicalised before comparing."""
import pytest
import torch

from oracle import flashmoe_oracle as orc

pytestmark = pytest.mark.gpu


def _check(idx, E):
    from flash_moe.ops.hip.flash_expert import expert_bucketing

    tok, offsets, pairs, experts = (t.cpu() for t in expert_bucketing(idx.cuda(), E))
    o_tok, o_offsets, o_pairs, o_experts = orc.expert_bucketing(idx, E)
    assert torch.equal(offsets, o_offsets), "expert_offsets"
    n = int(o_offsets[-1])
    assert torch.equal(pairs[:n], o_pairs), "sorted_pair_ids"
    assert torch.equal(tok[:n], o_tok), "sorted_token_ids"
    assert torch.equal(experts[:n], o_experts), "sorted_expert_ids"
    return offsets, pairs[:n]


@pytest.mark.parametrize("T,K,E,seed", [(64, 8, 32, 0), (1000, 16, 4096, 1), (4096, 64, 16384, 2), (333, 7, 100, 3),
                                        (5, 1, 3, 4), (2048, 128, 262144, 5), (700, 3, 1, 6)])
def test_bucketing_random_ids(T, K, E, seed):
    g = torch.Generator().manual_seed(seed)
    idx = torch.randint(0, E, (T, K), generator=g)
    offsets, pairs = _check(idx, E)
    assert int(offsets[-1]) == T * K and sorted(pairs.tolist()) == list(range(T * K))


def test_bucketing_ids_out_of_range_take_no_slot():
    g = torch.Generator().manual_seed(7)
    T, K, E = 500, 8, 64
    idx = torch.randint(0, E, (T, K), generator=g)
    idx[::7, 2] = -1
    idx[3::11, 5] = E
    idx[5::13, 0] = 1 << 40
    offsets, pairs = _check(idx, E)
    assert int(offsets[-1]) == int(((idx >= 0) & (idx < E)).sum())


@pytest.mark.parametrize("T,hot", [(100, 1.0), (3000, 1.0), (20000, 1.0), (20000, 0.3)])
def test_bucketing_with_a_hot_expert(T, hot):
    """Segments of 100 (one wave), 3000 (sorted in LDS) and 20000 / ~6000 pairs (compacted from the index array)."""
    g = torch.Generator().manual_seed(8)
    K, E = 4, 1024
    idx = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)])
    chosen = torch.rand(T, generator=g) < hot
    slot = torch.randint(0, K, (T,), generator=g)
    idx[chosen, slot[chosen]] = 77
    offsets, _ = _check(idx, E)
    assert int(offsets[78] - offsets[77]) >= int(chosen.sum())


def test_bucketing_of_router_produced_ids_and_the_reference_named_helper():
    from flash_moe.ops.hip.flash_expert import preprocess_expert_centric_indices
    from flash_moe.ops import flash_router_func

    T, nk, K = 2048, 64, 32
    lp = orc.make_router_inputs(T, nk, seed=3).cuda()
    _, idx = flash_router_func(lp, nk, K)
    _check(idx.cpu(), nk * nk)
    gates = torch.rand(T, K, device="cuda")
    tok, sorted_g, offsets, max_pairs, pairs = preprocess_expert_centric_indices(idx, gates, nk * nk)
    o_tok, o_offsets, o_pairs, _ = orc.expert_bucketing(idx.cpu(), nk * nk)
    assert torch.equal(sorted_g.cpu(), gates.cpu().reshape(-1)[o_pairs.long()])
    assert max_pairs == int((o_offsets[1:] - o_offsets[:-1]).max()) and torch.equal(pairs.cpu(), o_pairs)


def test_bucketing_of_an_empty_batch():
    from flash_moe.ops.hip.flash_expert import expert_bucketing

    tok, offsets, pairs, _ = expert_bucketing(torch.zeros(0, 4, dtype=torch.int64, device="cuda"), 10)
    assert tok.numel() == 0 and pairs.numel() == 0 and offsets.cpu().tolist() == [0] * 11
