"""PEER and PKM ops against the oracle's restatement of the eager formulas of the reference's tests
(tests/test_peer.py:9-24, tests/test_pkm.py:9-20), evaluated in float64 on the CPU; the oracle functions are pinned by the
plain-C brute force and closed forms in tests/test_oracle_pins.py."""
import pytest
import torch

from helpers import assert_output_close, rel_fro
from oracle import flashmoe_oracle as orc

pytestmark = pytest.mark.gpu
FRO = {torch.float32: 2e-6, torch.bfloat16: 4e-3, torch.float16: 1e-3}


def peer_reference(x, wd, wu, w, idx):
    return orc.peer_forward(x, wd, wu, w, idx)


def pkm_reference(values, w, idx):
    return orc.pkm_forward(values, w, idx)


CASES = [(64, 128, 256, 8),            # row schedule
         (1024, 256, 4096, 64),        # column-slice schedule (T*K >= 65536, slice fits L2)
         (33, 1024, 1000, 5),          # ragged
         (16, 2048, 512, 4),
         (20, 5120, 96, 6)]            # rows beyond one wavefront's registers: column slices whatever the size


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,H,E,K", CASES)
def test_peer_forward(dtype, T, H, E, K):
    from flash_moe.ops.triton.peer import triton_peer_func

    x, wd, wu, idx, w = orc.make_expert_inputs(T, H, E, K, seed=4, std=0.05)
    x, wd, wu, w = (t.to(dtype) for t in (x, wd, wu, w))
    out = triton_peer_func(x.cuda(), wd.cuda(), wu.cuda(), w.cuda(), idx.cuda())
    ref = peer_reference(x.double(), wd.double(), wu.double(), w.double(), idx)
    assert out.shape == (T, H) and out.dtype == dtype
    assert rel_fro(out, ref) < FRO[dtype]
    assert_output_close(out, ref.to(dtype), dtype, "peer")
    # GELU is not SiLU: the op must differ from the routed-expert op on the same inputs
    from flash_moe.ops import flash_expert_func

    assert rel_fro(flash_expert_func(x.cuda(), wd.cuda(), wu.cuda(), idx.cuda(), w.cuda()), ref) > 10 * FRO[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,H,E,K", CASES + [(300, 128, 64, 16)])          # more tokens than table rows
def test_pkm_forward(dtype, T, H, E, K):
    from flash_moe.ops.triton.pkm import triton_pkm_func

    _, values, _, idx, w = orc.make_expert_inputs(T, H, E, K, seed=6, std=1.0)
    values, w = values.to(dtype), w.to(dtype)
    out = triton_pkm_func(values.cuda(), w.cuda(), idx.cuda())
    ref = pkm_reference(values.double(), w.double(), idx)
    assert out.shape == (T, H) and out.dtype == dtype
    assert rel_fro(out, ref) < FRO[dtype]
    assert_output_close(out, ref.to(dtype), dtype, "pkm")


def test_pkm_closed_forms():
    from flash_moe.ops import pkm_func

    values = torch.randn(512, 256, generator=torch.Generator().manual_seed(0)).cuda()
    idx = torch.randint(0, 512, (128, 8), generator=torch.Generator().manual_seed(1)).cuda()
    one_hot = torch.zeros(128, 8).cuda()
    one_hot[:, 3] = 1.0
    assert torch.equal(pkm_func(values, one_hot, idx), values[idx[:, 3]])                  # a single unit weight copies a row
    assert torch.equal(pkm_func(values, torch.zeros(128, 8).cuda(), idx), torch.zeros(128, 256).cuda())
    same = idx[:, :1].expand(-1, 8).contiguous()                                          # one row eight times, weights 1/8
    torch.testing.assert_close(pkm_func(values, torch.full((128, 8), 0.125).cuda(), same), values[idx[:, 0]], rtol=1e-6, atol=1e-6)
    with pytest.raises(NotImplementedError):
        pkm_func(values.requires_grad_(True), one_hot, idx).sum().backward()
