"""Pins of the CPU oracle (oracle/flashmoe_oracle.py) that do not retype its formulas.

Each oracle function is checked against (a) the plain-C double-precision brute force in
oracle/bruteforce.c, which shares no routine with torch, and (b) closed forms / invariants chosen so
that a dropped term, a wrong sign or index, or a transposed operand fails at least one of them.
"""
import numpy as np
import pytest
import torch

from oracle import bruteforce as bf
from oracle import flashmoe_oracle as orc


# ----------------------------------------------------------------------------------------------
# router prologue
# ----------------------------------------------------------------------------------------------
def test_prologue_matches_bruteforce_training():
    g = torch.Generator().manual_seed(1)
    T, H, nk = 96, 40, 12
    x = torch.randn(T, H, generator=g, dtype=torch.float64) * 3 + 0.7
    wr = torch.randn(2 * nk, H, generator=g, dtype=torch.float64) * 0.3
    rm, rv = torch.zeros(H, dtype=torch.float64), torch.ones(H, dtype=torch.float64)
    logits, lp = orc.router_prologue(x, wr, nk, rm, rv, training=True)
    b_logits, b_lp, b_mean, b_var = bf.prologue(x.numpy(), wr.numpy(), nk, training=True)
    assert logits.shape == (2, T, nk) and lp.shape == (2, T, nk)
    np.testing.assert_allclose(logits.numpy(), b_logits, rtol=1e-10, atol=1e-10)
    np.testing.assert_allclose(lp.numpy(), b_lp, rtol=1e-10, atol=1e-10)
    # running statistics: momentum 0.1 from (0, 1), unbiased variance in the running estimate
    np.testing.assert_allclose(rm.numpy(), 0.1 * b_mean, rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(rv.numpy(), 0.9 + 0.1 * b_var * T / (T - 1), rtol=1e-10)


def test_prologue_matches_bruteforce_eval():
    g = torch.Generator().manual_seed(2)
    T, H, nk = 33, 24, 7
    x = torch.randn(T, H, generator=g, dtype=torch.float64)
    wr = torch.randn(2 * nk, H, generator=g, dtype=torch.float64)
    rm = torch.randn(H, generator=g, dtype=torch.float64)
    rv = torch.rand(H, generator=g, dtype=torch.float64) + 0.5
    logits, lp = orc.router_prologue(x, wr, nk, rm.clone(), rv.clone(), training=False)
    b_logits, b_lp, _, _ = bf.prologue(x.numpy(), wr.numpy(), nk, training=False, mean=rm.numpy(), var=rv.numpy())
    np.testing.assert_allclose(logits.numpy(), b_logits, rtol=1e-10, atol=1e-10)
    np.testing.assert_allclose(lp.numpy(), b_lp, rtol=1e-10, atol=1e-10)


def test_prologue_invariants():
    g = torch.Generator().manual_seed(3)
    T, H, nk = 64, 16, 8
    x = torch.randn(T, H, generator=g, dtype=torch.float64) * 5 - 2
    wr = torch.randn(2 * nk, H, generator=g, dtype=torch.float64)
    logits, lp = orc.router_prologue(x, wr, nk)
    # log-probabilities: logsumexp over the key axis is 0 for each half
    assert torch.logsumexp(lp, -1).abs().max() < 1e-12
    # half h of the output is gate features [h*nk, (h+1)*nk): zero the second half of the gate
    wr2 = wr.clone()
    wr2[nk:] = 0
    logits2, _ = orc.router_prologue(x, wr2, nk)
    assert torch.equal(logits2[0], logits[0]) and logits2[1].abs().max() == 0
    # batch-norm removes any per-feature affine map of x (exactly so but for eps = 1e-5 under the root)
    logits3, _ = orc.router_prologue(x * 3.0 + 11.0, wr, nk)
    assert (logits3 - logits).abs().max() < 1e-4


# ----------------------------------------------------------------------------------------------
# router top-k
# ----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("T,nk,K", [(64, 8, 8), (128, 32, 16), (32, 64, 8), (16, 128, 64), (5, 13, 13), (7, 9, 1)])
def test_router_topk_matches_bruteforce(T, nk, K):
    lp = orc.make_router_inputs(T, nk, seed=T + nk + K)
    scores, idx = orc.router_topk(lp, nk, K)
    b_scores, b_idx = bf.router_topk(lp.numpy(), nk, K)
    # scores are the K largest sums: identical whatever the tie order
    np.testing.assert_array_equal(scores.numpy(), b_scores)
    # index sets are identical unless the K-th and (K+1)-th sums tie (random fp32 normals: they do not)
    assert np.array_equal(np.sort(idx.numpy(), -1), np.sort(b_idx, -1))
    # and each returned index reproduces its score exactly
    i, j = idx // nk, idx % nk
    again = lp[0].gather(-1, i) + lp[1].gather(-1, j)
    assert torch.equal(again, scores)


def test_router_topk_numpy_argsort():
    # second independent check: numpy stable argsort of all nk*nk sums
    T, nk, K = 40, 16, 16
    lp = orc.make_router_inputs(T, nk, seed=11, log_probs=False)
    scores, idx = orc.router_topk(lp, nk, K)
    sums = (lp[0].numpy()[:, :, None] + lp[1].numpy()[:, None, :]).reshape(T, -1)
    order = np.argsort(-sums, axis=-1, kind="stable")[:, :K]
    np.testing.assert_array_equal(np.take_along_axis(sums, order, -1), scores.numpy())
    assert np.array_equal(np.sort(order, -1), np.sort(idx.numpy(), -1))


def test_router_topk_closed_forms():
    nk = 16
    lp = torch.full((2, 3, nk), -9.0)
    # one dominant key per half: the best pair is known, the next ones pair a dominant key with the rest
    lp[0, :, 5] = -0.1
    lp[1, :, 11] = -0.2
    lp[0, :, 2] = -1.0   # second best of half 0
    scores, idx = orc.router_topk(lp, nk, 2)
    assert idx[:, 0].tolist() == [5 * nk + 11] * 3
    assert idx[:, 1].tolist() == [2 * nk + 11] * 3
    assert torch.allclose(scores[:, 0], torch.tensor(-0.3)) and torch.allclose(scores[:, 1], torch.tensor(-1.2))
    # K = 1 is (argmax, argmax); transposing the halves transposes the index
    z = orc.make_router_inputs(50, nk, seed=5)
    s1, i1 = orc.router_topk(z, nk, 1)
    assert torch.equal(i1[:, 0], z[0].argmax(-1) * nk + z[1].argmax(-1))
    s2, i2 = orc.router_topk(z.flip(0), nk, 1)
    assert torch.equal(i2[:, 0], z[1].argmax(-1) * nk + z[0].argmax(-1)) and torch.equal(s1, s2)
    # K = nk: scores non-increasing, indices distinct and in range
    s, i = orc.router_topk(z, nk, nk)
    assert (s[:, 1:] <= s[:, :-1]).all()
    assert all(len(set(r.tolist())) == nk for r in i) and i.min() >= 0 and i.max() < nk * nk


def test_routing_weights():
    z = orc.make_router_inputs(20, 8, seed=9)
    s, i = orc.router_topk(z, 8, 4)
    w = orc.routing_weights(s, False)
    px, py = z[0].exp().gather(-1, i // 8), z[1].exp().gather(-1, i % 8)
    assert torch.allclose(w, px * py, rtol=1e-6)           # exp(lp_x + lp_y) = p_x * p_y
    assert (w.sum(-1) <= 1 + 1e-6).all()
    wn = orc.routing_weights(s, True)
    assert torch.allclose(wn.sum(-1), torch.ones(20), atol=1e-6)
    assert torch.allclose(wn * w.sum(-1, keepdim=True), w, rtol=1e-6)


# ----------------------------------------------------------------------------------------------
# routed experts
# ----------------------------------------------------------------------------------------------
def _expert_case(T, H, E, K, seed, std=0.3):
    x, wd, wu, idx, g = orc.make_expert_inputs(T, H, E, K, seed=seed, std=std)
    return tuple(t.double() if t.is_floating_point() else t for t in (x, wd, wu, idx, g))


@pytest.mark.parametrize("T,H,E,K", [(50, 24, 64, 8), (17, 40, 9, 9), (8, 16, 256, 32)])
def test_expert_matches_bruteforce(T, H, E, K):
    x, wd, wu, idx, g = _expert_case(T, H, E, K, seed=T)
    out = orc.expert_forward(x, wd, wu, idx, g, token_chunk=7)   # chunk that does not divide T
    ref = bf.expert(x.numpy(), wd.numpy(), wu.numpy(), idx.numpy(), g.numpy())
    np.testing.assert_allclose(out.numpy(), ref, rtol=1e-11, atol=1e-13)


def test_expert_special_cases():
    x, wd, wu, idx, g = _expert_case(12, 16, 32, 4, seed=4)
    out = orc.expert_forward(x, wd, wu, idx, g)
    # zero gates give exact zeros
    assert orc.expert_forward(x, wd, wu, idx, torch.zeros_like(g)).abs().max() == 0
    # linear in the gates
    assert torch.allclose(orc.expert_forward(x, wd, wu, idx, 2.5 * g), 2.5 * out, rtol=1e-12)
    # invariant under a permutation of the K slots
    perm = torch.tensor([2, 0, 3, 1])
    assert torch.allclose(orc.expert_forward(x, wd, wu, idx[:, perm], g[:, perm]), out, rtol=1e-12)
    # a repeated expert adds: K copies of expert e with gate 1/K  ==  one copy with gate 1
    e = torch.full((12, 4), 7, dtype=torch.int64)
    one = orc.expert_forward(x, wd, wu, e[:, :1], torch.ones(12, 1, dtype=torch.float64))
    rep = orc.expert_forward(x, wd, wu, e, torch.full((12, 4), 0.25, dtype=torch.float64))
    assert torch.allclose(rep, one, rtol=1e-12)
    # and that single-expert output is silu(<x, wd_e>) * wu_e: a scalar multiple of row e of the up table
    s = x @ wd[7]
    assert torch.allclose(one, (s / (1 + torch.exp(-s))).unsqueeze(-1) * wu[7], rtol=1e-12)
    # swapping the two tables changes the result (guards against a transposed table argument)
    assert not torch.allclose(orc.expert_forward(x, wu, wd, idx, g), out, rtol=1e-3)


# ----------------------------------------------------------------------------------------------
# shared MLP and the block
# ----------------------------------------------------------------------------------------------
def test_mlp_matches_bruteforce():
    g = torch.Generator().manual_seed(8)
    T, H, I = 21, 24, 56
    x = torch.randn(T, H, generator=g, dtype=torch.float64)
    wg, wu = (torch.randn(I, H, generator=g, dtype=torch.float64) * 0.4 for _ in range(2))
    wd = torch.randn(H, I, generator=g, dtype=torch.float64) * 0.4
    out = orc.mlp_forward(x, wg, wu, wd)
    np.testing.assert_allclose(out.numpy(), bf.mlp(x.numpy(), wg.numpy(), wu.numpy(), wd.numpy()), rtol=1e-11, atol=1e-13)
    # silu is applied to the gate branch, not the up branch
    assert not torch.allclose(orc.mlp_forward(x, wu, wg, wd), out, rtol=1e-3)


def test_block_is_the_composition_of_its_stages():
    H, I, E, K = 32, 64, 64, 4
    w = orc.make_block_weights(H, I, E, seed=3, std=0.3)
    x = torch.randn(2, 24, H, generator=torch.Generator().manual_seed(4))
    for norm in (False, True):
        w.running_mean.zero_(); w.running_var.fill_(1.0)
        r = orc.block_forward(x, w, K, norm_topk_prob=norm, training=True)
        hid = x.reshape(-1, H)
        logits, lp = orc.router_prologue(hid, w.router_gate, w.num_keys)
        s, i = orc.router_topk(lp, w.num_keys, K)
        g = orc.routing_weights(s, norm)
        y = orc.mlp_forward(hid, w.gate_proj, w.up_proj, w.down_proj) + orc.expert_forward(hid, w.down_embed, w.up_embed, i, g)
        assert torch.equal(r["indices"], i) and torch.allclose(r["y"].reshape(-1, H), y, rtol=1e-6, atol=1e-7)
        assert r["router_logits"].shape == (2, 48, w.num_keys) and torch.allclose(r["router_logits"], logits)
        # routing in fp32 is the same thing when the inputs are fp32
        w.running_mean.zero_(); w.running_var.fill_(1.0)
        r32 = orc.block_forward(x, w, K, norm_topk_prob=norm, training=True, routing_fp32=True)
        assert torch.equal(r32["indices"], r["indices"]) and torch.allclose(r32["y"], r["y"], rtol=1e-6, atol=1e-7)
    # eval mode uses the running statistics accumulated above
    r_eval = orc.block_forward(x, w, K, training=False)
    assert not torch.allclose(r_eval["router_logits"], r["router_logits"])


def test_block_bruteforce_end_to_end():
    # the whole block against the C brute force, stage by stage in float64
    H, I, E, K = 16, 24, 36, 5
    w = orc.make_block_weights(H, I, E, seed=6, std=0.5).to(torch.float64)
    x = torch.randn(1, 30, H, generator=torch.Generator().manual_seed(7), dtype=torch.float64)
    w.running_mean = None; w.running_var = None
    r = orc.block_forward(x, w, K, norm_topk_prob=True)
    nk = w.num_keys
    _, b_lp, _, _ = bf.prologue(x[0].numpy(), w.router_gate.numpy(), nk)
    sums = (b_lp[0][:, :, None] + b_lp[1][:, None, :]).reshape(30, -1)
    order = np.argsort(-sums, -1, kind="stable")[:, :K]
    assert np.array_equal(np.sort(order, -1), np.sort(r["indices"].numpy(), -1))
    gates = np.exp(np.take_along_axis(sums, order, -1))
    gates /= gates.sum(-1, keepdims=True)
    y = bf.mlp(x[0].numpy(), w.gate_proj.numpy(), w.up_proj.numpy(), w.down_proj.numpy()) + bf.expert(
        x[0].numpy(), w.down_embed.numpy(), w.up_embed.numpy(), order, gates)
    np.testing.assert_allclose(r["y"][0].numpy(), y, rtol=1e-9, atol=1e-11)


# ----------------------------------------------------------------------------------------------
# expert-centric bucketing (flash_expert.py:528-577)
# ----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("T,K,E,seed", [(40, 4, 16, 0), (7, 5, 100, 1), (64, 8, 8, 2), (1, 1, 3, 3), (33, 3, 1, 4)])
def test_bucketing_matches_exhaustive_scan(T, K, E, seed):
    g = torch.Generator().manual_seed(seed)
    idx = torch.randint(0, E, (T, K), generator=g)
    if T > 4:
        idx[1, 0] = -3          # ids outside [0, E) belong to no segment
        idx[2, K - 1] = E + 5
    tok, offsets, pairs, experts = orc.expert_bucketing(idx, E)
    b_offsets, b_pairs = bf.bucket(idx.numpy(), E)
    np.testing.assert_array_equal(offsets.numpy(), b_offsets)
    np.testing.assert_array_equal(pairs.numpy(), b_pairs)          # stable: ascending pair index inside a segment
    np.testing.assert_array_equal(tok.numpy(), b_pairs // K)
    np.testing.assert_array_equal(experts.numpy(), idx.reshape(-1).numpy()[b_pairs])
    assert offsets.dtype == torch.int32 and pairs.dtype == torch.int32 and tok.dtype == torch.int32


def test_bucketing_invariants_and_numpy_argsort():
    g = torch.Generator().manual_seed(9)
    T, K, E = 500, 16, 300
    idx = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)])
    tok, offsets, pairs, experts = orc.expert_bucketing(idx, E)
    flat = idx.reshape(-1).numpy()
    P = T * K
    assert int(offsets[0]) == 0 and int(offsets[-1]) == P and (offsets[1:] >= offsets[:-1]).all()
    assert sorted(pairs.tolist()) == list(range(P))                 # a permutation: the multiset of pairs is preserved
    for e in (0, 1, E // 2, E - 1):                                 # each segment holds one expert, in ascending pair index
        seg = pairs[int(offsets[e]):int(offsets[e + 1])].numpy()
        assert (flat[seg] == e).all() and (np.diff(seg) > 0).all()
    np.testing.assert_array_equal(pairs.numpy(), np.argsort(flat, kind="stable").astype(np.int32))
    np.testing.assert_array_equal(np.diff(offsets.numpy()), np.bincount(flat, minlength=E))
    # one expert selected by every token: a single segment listing the tokens in order
    one = torch.full((T, 1), 7)
    tok1, off1, pairs1, _ = orc.expert_bucketing(one, E)
    assert tok1.tolist() == list(range(T)) and int(off1[7]) == 0 and int(off1[8]) == T and int(off1[-1]) == T
    # no pairs at all
    tok0, off0, pairs0, _ = orc.expert_bucketing(torch.zeros(0, 4, dtype=torch.int64), 5)
    assert tok0.numel() == 0 and off0.tolist() == [0] * 6


# ----------------------------------------------------------------------------------------------
# PEER / PKM (tests/test_peer.py:9-24, tests/test_pkm.py:9-20)
# ----------------------------------------------------------------------------------------------
def test_peer_and_pkm_match_bruteforce():
    T, H, E, K = 24, 20, 50, 6
    x, wd, wu, idx, w = orc.make_expert_inputs(T, H, E, K, seed=12, std=0.7)
    x, wd, wu, w = (t.double() for t in (x, wd, wu, w))
    np.testing.assert_allclose(orc.peer_forward(x, wd, wu, w, idx).numpy(),
                               bf.peer(x.numpy(), wd.numpy(), wu.numpy(), idx.numpy(), w.numpy()), rtol=1e-11, atol=1e-12)
    np.testing.assert_allclose(orc.pkm_forward(wu, w, idx).numpy(), bf.pkm(wu.numpy(), idx.numpy(), w.numpy()),
                               rtol=1e-12, atol=1e-13)
    # the erf GELU is neither SiLU nor the tanh approximation
    silu = orc.expert_forward(x, wd, wu, idx, w)
    assert (orc.peer_forward(x, wd, wu, w, idx) - silu).abs().max() > 1e-3


def test_peer_and_pkm_closed_forms():
    g = torch.Generator().manual_seed(13)
    T, H, E = 9, 12, 30
    values = torch.randn(E, H, generator=g, dtype=torch.float64)
    idx = torch.randint(0, E, (T, 1), generator=g)
    # PKM: a unit weight copies the row; zero weights give zero; the same row twice doubles it
    assert torch.equal(orc.pkm_forward(values, torch.ones(T, 1, dtype=torch.float64), idx), values[idx[:, 0]])
    assert orc.pkm_forward(values, torch.zeros(T, 1, dtype=torch.float64), idx).abs().max() == 0
    twice = orc.pkm_forward(values, torch.ones(T, 2, dtype=torch.float64), idx.expand(T, 2))
    torch.testing.assert_close(twice, 2 * values[idx[:, 0]], rtol=1e-14, atol=0)
    # PEER: gelu(s) - gelu(-s) = s, so x and -x on the same expert differ by s * w * up[e]
    x = torch.randn(T, H, generator=g, dtype=torch.float64)
    wd = torch.randn(E, H, generator=g, dtype=torch.float64) * 0.5
    w = torch.rand(T, 1, generator=g, dtype=torch.float64) + 0.1
    s = (x * wd[idx[:, 0]]).sum(-1, keepdim=True)
    diff = orc.peer_forward(x, wd, values, w, idx) - orc.peer_forward(-x, wd, values, w, idx)
    torch.testing.assert_close(diff, s * w * values[idx[:, 0]], rtol=1e-12, atol=1e-13)
    # gelu(0) = 0: a zero input row gives a zero output row, whatever the weights
    assert orc.peer_forward(torch.zeros(T, H, dtype=torch.float64), wd, values, w, idx).abs().max() == 0
    # known values of the erf GELU: gelu(1) = 0.5 * (1 + erf(1/sqrt 2)) = 0.8413447460685429...
    one = orc.peer_forward(torch.ones(1, 1, dtype=torch.float64), torch.ones(1, 1, dtype=torch.float64),
                           torch.ones(1, 1, dtype=torch.float64), torch.ones(1, 1, dtype=torch.float64),
                           torch.zeros(1, 1, dtype=torch.int64))
    assert abs(float(one) - 0.8413447460685429) < 1e-15
