"""Writes the golden fixtures of this directory from the CPU oracle (oracle/flashmoe_oracle.py).

The reference holds no golden vectors for the forward path (its tests print, they do not assert), and
its package is not imported here; the oracle is pinned by tests/test_oracle_pins.py (plain-C brute
force, closed forms) and these files freeze its output so that a later change of the oracle, of torch,
or of the HIP kernels shows up as a diff against committed data.

    python tests/golden/make_golden.py        # rewrites the .npz files next to this script

block_small_fp32.npz   a tiny block with every input tensor stored: T=2x24, H=64, I=128, E=256, K=8
block_c1_fp32.npz      configuration C1 (fp32, 1x512 tokens, H=256, I=1024, E=1024, K=16, seed 0):
                       inputs are regenerated from the seed, stored are scores, indices and every
                       8th row of the outputs
router_cases.npz       router inputs / outputs for a few (T, nk, K), including exact-tie inputs
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import bruteforce as bf          # noqa: E402
from oracle import flashmoe_oracle as orc    # noqa: E402


def c1_inputs():
    """Configuration C1: x ~ N(0,1) [1,512,256], weights ~ N(0,0.02), seed 0."""
    w = orc.make_block_weights(256, 1024, 1024, seed=0, std=0.02)
    x = torch.randn(1, 512, 256, generator=torch.Generator().manual_seed(0))
    return x, w


def small_inputs():
    w = orc.make_block_weights(64, 128, 256, seed=21, std=0.25)
    x = torch.randn(2, 24, 64, generator=torch.Generator().manual_seed(22))
    return x, w


def main():
    torch.set_num_threads(1)   # one thread: summation order of the CPU kernels is then fixed
    x, w = small_inputs()
    out = {}
    for norm in (False, True):
        w.running_mean.zero_(); w.running_var.fill_(1.0)
        r = orc.block_forward(x, w, 8, norm_topk_prob=norm, training=True)
        tag = "norm" if norm else "raw"
        for k in ("y", "router_logits", "scores", "indices", "gates", "experts", "mlp"):
            out[f"{tag}_{k}"] = r[k].contiguous().numpy()
    out["running_mean_after"] = w.running_mean.numpy().copy()
    out["running_var_after"] = w.running_var.numpy().copy()
    r = orc.block_forward(x, w, 8, norm_topk_prob=False, training=False)
    out["eval_y"] = r["y"].numpy()
    out["eval_indices"] = r["indices"].numpy()
    out["x"] = x.numpy()
    for f in ("gate_proj", "up_proj", "down_proj", "router_gate", "down_embed", "up_embed"):
        out[f"w_{f}"] = getattr(w, f).numpy()
    np.savez_compressed(os.path.join(HERE, "block_small_fp32.npz"), **out)

    x, w = c1_inputs()
    r = orc.block_forward(x, w, 16, norm_topk_prob=False, training=True)
    np.savez_compressed(
        os.path.join(HERE, "block_c1_fp32.npz"),
        scores=r["scores"].numpy(), indices=r["indices"].numpy().astype(np.int32),
        y_rows=r["y"][0, ::8].numpy(), experts_rows=r["experts"][::8].numpy(), mlp_rows=r["mlp"][::8].numpy(),
        logits_rows=r["router_logits"][:, ::8].contiguous().numpy(),
        x_checksum=np.float64(x.double().sum().item()), table_checksum=np.float64(w.down_embed.double().sum().item()),
    )

    cases = {}
    for name, (T, nk, K, quant) in {"a": (64, 32, 16, False), "b": (48, 128, 64, False), "c": (40, 16, 16, True),
                                    "d": (16, 100, 37, False)}.items():
        lp = orc.make_router_inputs(T, nk, seed=len(name) + T)
        if quant:
            lp = (lp * 2).round() / 2           # exact ties everywhere
        s, i = bf.router_topk(lp.numpy(), nk, K)    # exhaustive scan, ties to the lowest index
        so, io = orc.router_topk(lp, nk, K)
        assert np.array_equal(so.numpy(), s)
        cases[f"{name}_lp"] = lp.numpy(); cases[f"{name}_scores"] = s; cases[f"{name}_indices"] = i.astype(np.int32)
        cases[f"{name}_shape"] = np.array([T, nk, K])
    np.savez_compressed(os.path.join(HERE, "router_cases.npz"), **cases)
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")


if __name__ == "__main__":
    main()
