"""Golden fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py).

CPU: the oracle still reproduces them.  GPU: the HIP path reproduces them."""
import os
import sys

import numpy as np
import pytest
import torch

from helpers import assert_output_close, cuda
from oracle import flashmoe_oracle as orc

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
sys.path.insert(0, GOLD)
import make_golden  # noqa: E402


def load(name):
    return {k: v for k, v in np.load(os.path.join(GOLD, name)).items()}   # allow_pickle stays False


def small_weights(g):
    w = orc.BlockWeights(*(torch.from_numpy(g[f"w_{f}"]) for f in
                           ("gate_proj", "up_proj", "down_proj", "router_gate", "down_embed", "up_embed")))
    w.running_mean, w.running_var = torch.zeros(64), torch.ones(64)
    return w


def test_generator_inputs_are_reproducible():
    g = load("block_small_fp32.npz")
    x, w = make_golden.small_inputs()
    assert np.array_equal(x.numpy(), g["x"]) and np.array_equal(w.down_embed.numpy(), g["w_down_embed"])
    c1 = load("block_c1_fp32.npz")
    x, w = make_golden.c1_inputs()
    assert abs(x.double().sum().item() - float(c1["x_checksum"])) < 1e-9
    assert abs(w.down_embed.double().sum().item() - float(c1["table_checksum"])) < 1e-9


def test_oracle_reproduces_small_block():
    g = load("block_small_fp32.npz")
    x = torch.from_numpy(g["x"])
    for norm, tag in ((False, "raw"), (True, "norm")):
        w = small_weights(g)
        r = orc.block_forward(x, w, 8, norm_topk_prob=norm, training=True)
        assert np.array_equal(np.sort(r["indices"].numpy(), -1), np.sort(g[f"{tag}_indices"], -1))
        for k in ("y", "router_logits", "scores", "gates", "experts", "mlp"):
            np.testing.assert_allclose(r[k].numpy(), g[f"{tag}_{k}"], rtol=1e-5, atol=1e-6, err_msg=k)
    # the fixture's running statistics are those after one training pass from (0, 1)
    w = small_weights(g)
    orc.block_forward(x, w, 8, training=True)
    np.testing.assert_allclose(w.running_mean.numpy(), g["running_mean_after"], rtol=1e-5, atol=1e-7)
    np.testing.assert_allclose(w.running_var.numpy(), g["running_var_after"], rtol=1e-5)
    r = orc.block_forward(x, w, 8, training=False)
    np.testing.assert_allclose(r["y"].numpy(), g["eval_y"], rtol=1e-5, atol=1e-6)


def test_oracle_reproduces_c1():
    g = load("block_c1_fp32.npz")
    x, w = make_golden.c1_inputs()
    r = orc.block_forward(x, w, 16)
    assert np.array_equal(np.sort(r["indices"].numpy(), -1), np.sort(g["indices"].astype(np.int64), -1))
    np.testing.assert_allclose(r["scores"].numpy(), g["scores"], rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(r["y"][0, ::8].numpy(), g["y_rows"], rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(r["experts"][::8].numpy(), g["experts_rows"], rtol=1e-5, atol=1e-8)


def test_oracle_reproduces_router_cases():
    g = load("router_cases.npz")
    for name in "abcd":
        T, nk, K = (int(v) for v in g[f"{name}_shape"])
        s, i = orc.router_topk(torch.from_numpy(g[f"{name}_lp"]), nk, K)
        assert np.array_equal(s.numpy(), g[f"{name}_scores"])
        if name != "c":   # case c is all ties: index sets are not unique
            assert np.array_equal(np.sort(i.numpy(), -1), np.sort(g[f"{name}_indices"].astype(np.int64), -1))


# ------------------------------------------------------------------------------------------------
@pytest.mark.gpu
def test_hip_router_reproduces_router_cases():
    from flash_moe.ops import flash_router_func

    g = load("router_cases.npz")
    for name in "abcd":
        T, nk, K = (int(v) for v in g[f"{name}_shape"])
        lp = torch.from_numpy(g[f"{name}_lp"])
        s, i = flash_router_func(cuda(lp), nk, K)
        assert np.array_equal(s.cpu().numpy(), g[f"{name}_scores"]), name
        i = i.cpu()
        assert torch.equal(lp[0].gather(-1, i // nk) + lp[1].gather(-1, i % nk), s.cpu())
        if name != "c":
            assert np.array_equal(np.sort(i.numpy(), -1), np.sort(g[f"{name}_indices"].astype(np.int64), -1)), name


def _hip_block(H, I, E, K, norm, w, dtype=torch.float32):
    from flash_moe.modules.flash_moe import FlashMoE, FlashMoEConfig

    m = FlashMoE(FlashMoEConfig(H, I, "silu", E, K, norm))
    sd = {"gate_proj.weight": w.gate_proj, "up_proj.weight": w.up_proj, "down_proj.weight": w.down_proj,
          "router_gate.weight": w.router_gate, "down_embed.weight": w.down_embed, "up_embed.weight": w.up_embed}
    missing = m.load_state_dict(sd, strict=False)
    assert set(missing.missing_keys) <= {"router_norm.running_mean", "router_norm.running_var", "router_norm.num_batches_tracked"}
    return m.to(device="cuda", dtype=dtype)


@pytest.fixture
def fused_forward_path():
    """The module takes its fused forward when no gradient is being recorded."""
    with torch.no_grad():
        yield


@pytest.mark.gpu
def test_hip_block_reproduces_small_block(fused_forward_path):
    g = load("block_small_fp32.npz")
    x = torch.from_numpy(g["x"])
    w = small_weights(g)
    for norm, tag in ((False, "raw"), (True, "norm")):
        m = _hip_block(64, 128, 256, 8, norm, w)
        y, logits = m(x.cuda())
        assert y.shape == (2, 24, 64) and logits.shape == (2, 48, 16)
        assert_output_close(logits, torch.from_numpy(g[f"{tag}_router_logits"]), torch.float32, "router_logits")
        assert_output_close(y, torch.from_numpy(g[f"{tag}_y"]), torch.float32, f"y ({tag})")
        # running statistics after one training pass from (0, 1)
        np.testing.assert_allclose(m.router_norm.running_mean.cpu().numpy(), g["running_mean_after"], rtol=1e-4, atol=1e-6)
        np.testing.assert_allclose(m.router_norm.running_var.cpu().numpy(), g["running_var_after"], rtol=1e-4)
        saved = m.router_norm.running_mean.clone(), m.router_norm.running_var.clone()
        _, scores, indices, gates = m.route(x.cuda().view(-1, 64))     # a second training pass: undo its update
        m.router_norm.running_mean.copy_(saved[0]); m.router_norm.running_var.copy_(saved[1])
        assert np.array_equal(np.sort(indices.cpu().numpy(), -1), np.sort(g[f"{tag}_indices"], -1))
        np.testing.assert_allclose(gates.cpu().numpy(), g[f"{tag}_gates"], rtol=2e-4, atol=1e-7)
    m.eval()
    m.norm_topk_prob = False      # the eval fixture was written with un-normalised gates
    y, _ = m(x.cuda())
    assert_output_close(y, torch.from_numpy(g["eval_y"]), torch.float32, "eval y")


@pytest.mark.gpu
def test_hip_block_reproduces_c1(fused_forward_path):
    g = load("block_c1_fp32.npz")
    x, w = make_golden.c1_inputs()
    m = _hip_block(256, 1024, 1024, 16, False, w)
    y, logits = m(x.cuda())
    assert_output_close(y[0, ::8], torch.from_numpy(g["y_rows"]), torch.float32, "C1 y")
    assert_output_close(logits[:, ::8], torch.from_numpy(g["logits_rows"]), torch.float32, "C1 router_logits")
    m.router_norm.reset_running_stats()
    _, scores, indices, _ = m.route(x.cuda().view(-1, 256))
    same = (np.sort(indices.cpu().numpy(), -1) == np.sort(g["indices"].astype(np.int64), -1)).all(-1)
    # fp32 logits from a different summation order can flip a pair whose sums are within ~1e-5
    assert same.mean() > 0.97, same.mean()
    np.testing.assert_allclose(scores.cpu().numpy(), g["scores"], rtol=1e-4, atol=1e-4)
