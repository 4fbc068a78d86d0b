"""Parity of the HIP SwiGLU MLP (MFMA GEMMs, fused activation) with the CPU oracle, through the op."""
import pytest
import torch

from helpers import assert_output_close, cuda, rel_fro
from oracle import flashmoe_oracle as orc

pytestmark = pytest.mark.gpu


def make(T, H, I, dtype, seed, x_std=1.0, w_std=0.02):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(T, H, generator=g) * x_std).to(dtype)
    wg = (torch.randn(I, H, generator=g) * w_std).to(dtype)
    wu = (torch.randn(I, H, generator=g) * w_std).to(dtype)
    wd = (torch.randn(H, I, generator=g) * w_std).to(dtype)
    return x, wg, wu, wd


def truth64(x, wg, wu, wd):
    return orc.mlp_forward(x.double(), wg.double(), wu.double(), wd.double())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("T,H,I", [
    (512, 256, 1024),      # C1
    (1024, 1024, 4096),    # C4 weights, fewer tokens (small-tile path)
    (4096, 1024, 4096),    # C4 (large-tile path for gate/up)
    (192, 128, 256),       # 64-row tiles (T a multiple of 64 only)
    (100, 128, 256),       # ragged T on the tiled path: the last tile row reads clamped rows, stores are bounds-checked
    (1000, 256, 512),
    (200, 72, 136),        # ragged in every dimension
    (1, 64, 64),
])
def test_mlp_matches_oracle(dtype, T, H, I):
    from flash_moe.ops import flash_mlp_func

    x, wg, wu, wd = make(T, H, I, dtype, seed=T + I)
    got = flash_mlp_func(*cuda(x, wg, wu, wd)).cpu()
    assert got.dtype == dtype and got.shape == (T, H)
    ref64 = truth64(x, wg, wu, wd)
    assert_output_close(got, ref64.to(dtype), dtype, "mlp vs float64 oracle")
    assert rel_fro(got, ref64) < {torch.float32: 2e-6, torch.bfloat16: 6e-3, torch.float16: 8e-4}[dtype]
    if T <= 1024:
        assert_output_close(got, orc.mlp_forward(x, wg, wu, wd), dtype, "mlp vs same-dtype oracle")


def test_mlp_fp32_tensors_off_the_16_byte_grid():
    # fp32 callers need not align their tensors: the tiled kernel moves 16-byte pieces, so these take the bounds-checked
    # kernel, and the result is the aligned one's up to summation order
    from flash_moe.ops import flash_mlp_func

    x, wg, wu, wd = cuda(*make(256, 256, 512, torch.float32, seed=9))

    def shifted(t):
        buf = torch.empty(t.numel() + 1, device="cuda", dtype=t.dtype)
        buf[1:].copy_(t.reshape(-1))
        v = buf[1:].view(t.shape)
        assert v.data_ptr() % 16 == 4
        return v

    aligned = flash_mlp_func(x, wg, wu, wd)
    moved = flash_mlp_func(shifted(x), shifted(wg), shifted(wu), shifted(wd))
    ref64 = truth64(*(t.cpu() for t in (x, wg, wu, wd)))
    assert rel_fro(aligned, ref64) < 2e-6 and rel_fro(moved, ref64) < 2e-6


def test_mlp_reference_test_distribution():
    # tests/test_mlp.py:95-107: seed 42, x ~ N(0,0.5), weights ~ N(0,0.1); its shape scaled down
    from flash_moe.ops import flash_mlp_func

    x, wg, wu, wd = make(1024, 512, 2048, torch.bfloat16, seed=42, x_std=0.5, w_std=0.1)
    got = flash_mlp_func(*cuda(x, wg, wu, wd)).cpu()
    assert rel_fro(got, truth64(x, wg, wu, wd)) < 6e-3


def test_mlp_leading_dims_and_residual():
    from flash_moe.ops import flash_mlp_func
    from flash_moe.ops.hip.flash_mlp import mlp_forward

    x, wg, wu, wd = cuda(*make(192, 128, 256, torch.bfloat16, seed=3))
    y2 = flash_mlp_func(x, wg, wu, wd)
    y3 = flash_mlp_func(x.view(2, 96, 128), wg, wu, wd)
    assert y3.shape == (2, 96, 128) and torch.equal(y3.view(192, 128), y2)
    res = torch.randn(192, 128, device="cuda").bfloat16()
    yr = mlp_forward(x, wg, wu, wd, residual=res)
    ref = truth64(*(t.cpu() for t in (x, wg, wu, wd))) + res.cpu().double()
    assert rel_fro(yr.cpu(), ref) < 6e-3
    assert flash_mlp_func(x[:0], wg, wu, wd).shape == (0, 128)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("T,H,I", [(4096, 1024, 4096), (1024, 1024, 4096), (192, 128, 256), (200, 72, 136)])
def test_mlp_residual_is_added_in_every_tile_shape_and_dtype(dtype, T, H, I):
    # the block's "experts + mlp" is the down projection's epilogue: one case per kernel the dispatch can pick (256 x 256 and
    # 128 x 128 tiles, 64-row tiles, the bounds-checked kernel).  The residual is large against the product, so a lane that
    # reads a neighbour's residual shows at once; the sum is rounded once, from the fp32 accumulator.
    from flash_moe.ops.hip.flash_mlp import mlp_forward

    x, wg, wu, wd = make(T, H, I, dtype, seed=T + H)
    res = torch.randn(T, H, generator=torch.Generator().manual_seed(5)).to(dtype)
    got = mlp_forward(*cuda(x, wg, wu, wd), residual=res.cuda()).cpu()
    ref64 = truth64(x, wg, wu, wd) + res.double()
    assert got.dtype == dtype and got.shape == (T, H)
    assert rel_fro(got, ref64) < {torch.float32: 2e-6, torch.bfloat16: 6e-3, torch.float16: 8e-4}[dtype]
    assert (got.double() - ref64).abs().max() < {torch.float32: 1e-5, torch.bfloat16: 4e-2, torch.float16: 6e-3}[dtype]


def test_mlp_linearity_full_size():
    # C4 at full size: out is linear in the down projection and in the up projection
    from flash_moe.ops import flash_mlp_func

    x, wg, wu, wd = cuda(*make(4096, 1024, 4096, torch.bfloat16, seed=0))
    y = flash_mlp_func(x, wg, wu, wd)
    assert torch.equal(flash_mlp_func(x, wg, wu, wd * 2), y * 2)
    assert torch.equal(flash_mlp_func(x, wg, wu * 0.5, wd), y * 0.5)
    assert flash_mlp_func(x, wg, wu * 0, wd).abs().max() == 0
    assert torch.equal(flash_mlp_func(x, wg, wu, wd), y)
