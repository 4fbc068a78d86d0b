"""Host-side mirror of the reference interface: names, signatures, parameters, error behaviour."""
import inspect

import pytest
import torch

from flash_moe.modules.flash_moe import FlashMoE, FlashMoEConfig
from flash_moe.ops.utils import ensure_contiguous, next_power_of_2


def test_config_signature_matches_reference():
    # flash_moe/modules/flash_moe.py:12-27
    params = list(inspect.signature(FlashMoEConfig.__init__).parameters)
    assert params == ["self", "hidden_size", "intermediate_size", "hidden_act", "num_experts",
                      "num_experts_per_tok", "norm_topk_prob"]
    c = FlashMoEConfig(64, 128, "silu", 100, 4)
    assert c.norm_topk_prob is False and c.num_experts == 100


def test_module_parameters_and_state_dict_names():
    m = FlashMoE(FlashMoEConfig(64, 128, "silu", 100, 4))
    assert m.num_keys == 10          # floor(sqrt(100)); flash_moe.py:38
    sd = m.state_dict()
    expect = {
        "gate_proj.weight": (128, 64), "up_proj.weight": (128, 64), "down_proj.weight": (64, 128),
        "router_gate.weight": (20, 64), "router_norm.running_mean": (64,), "router_norm.running_var": (64,),
        "router_norm.num_batches_tracked": (), "down_embed.weight": (100, 64), "up_embed.weight": (100, 64),
    }
    assert {k: tuple(v.shape) for k, v in sd.items()} == expect
    assert m.top_k == 4 and m.norm_topk_prob is False
    # non-square expert counts keep floor(sqrt(E)) keys: 120 experts -> 10 keys, ids >= 100 never routed
    assert FlashMoE(FlashMoEConfig(64, 128, "silu", 120, 4)).num_keys == 10


def test_module_rejects_other_activations():
    with pytest.raises(ValueError, match="silu"):
        FlashMoE(FlashMoEConfig(64, 128, "gelu", 100, 4))


def test_forward_signature():
    sig = inspect.signature(FlashMoE.forward)
    assert list(sig.parameters)[:2] == ["self", "hidden_states"]
    assert any(p.kind is inspect.Parameter.VAR_KEYWORD for p in sig.parameters.values())


def test_reference_import_paths_resolve_to_the_hip_ops():
    from flash_moe.ops import flash_expert_func, flash_mlp_func, flash_router_func
    from flash_moe.ops.flash_expert import triton_flash_expert_func as e2
    from flash_moe.ops.flash_router import triton_flash_router_func as r2
    from flash_moe.ops.triton.flash_expert import triton_flash_expert_func as e1
    from flash_moe.ops.triton.flash_mlp import triton_flash_mlp_func as m1
    from flash_moe.ops.triton.flash_router import triton_flash_router_func as r1

    assert r1 is flash_router_func and r2 is flash_router_func
    assert e1 is flash_expert_func and e2 is flash_expert_func
    assert m1 is flash_mlp_func
    assert list(inspect.signature(r1).parameters) == ["router_logits", "num_expert_keys", "num_experts_per_tok"]
    assert list(inspect.signature(e1).parameters) == ["hidden_states", "down_weights", "up_weights", "indices", "routing_weights"]
    assert list(inspect.signature(m1).parameters) == ["x", "gate_weight", "up_weight", "down_weight"]


def test_router_assertions_match_reference_wording():
    # flash_router.py:257-263: AssertionError for a non-3D input, a first dimension != 2, K outside [0, nk]
    from flash_moe.ops import flash_router_func

    with pytest.raises(AssertionError, match="3D tensor"):
        flash_router_func(torch.zeros(4, 8), 8, 2)
    with pytest.raises(AssertionError, match="first dimension"):
        flash_router_func(torch.zeros(3, 4, 8), 8, 2)
    with pytest.raises(AssertionError, match=r"should be in \[0, 8\], but got 9"):
        flash_router_func(torch.zeros(2, 4, 8), 8, 9)


def test_utils():
    assert [next_power_of_2(n) for n in (0, 1, 2, 3, 4, 5, 1023, 1024, 1025)] == [1, 1, 2, 4, 4, 8, 1024, 1024, 2048]
    seen = {}

    @ensure_contiguous
    def f(ctx, a, b, k=None):
        seen["ok"] = a.is_contiguous() and k.is_contiguous() and b == 3
        return a

    t = torch.arange(12.0).view(3, 4).t()
    f(None, t, 3, k=t)
    assert seen["ok"] and not t.is_contiguous()
