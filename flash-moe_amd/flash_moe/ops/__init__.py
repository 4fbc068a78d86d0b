"""Functional ops of the FlashMoE forward path (HIP, gfx950)."""
from flash_moe.ops.hip.flash_router import flash_router_func
from flash_moe.ops.hip.flash_expert import flash_expert_func
from flash_moe.ops.hip.flash_mlp import flash_mlp_func
from flash_moe.ops.hip.peer import peer_func
from flash_moe.ops.hip.pkm import pkm_func

__all__ = ["flash_router_func", "flash_expert_func", "flash_mlp_func", "peer_func", "pkm_func"]
