"""``flash_moe.ops.flash_expert`` is the path docs/flash_expert.md:18 of the reference imports from."""
from flash_moe.ops.hip.flash_expert import FlashExpertFunc, flash_expert_func

triton_flash_expert_func = flash_expert_func
__all__ = ["flash_expert_func", "triton_flash_expert_func", "FlashExpertFunc"]
