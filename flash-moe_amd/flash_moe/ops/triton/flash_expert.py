"""``triton_flash_expert_func`` under the reference's import path; it is the HIP op."""
from flash_moe.ops.hip.flash_expert import FlashExpertFunc, flash_expert_func

triton_flash_expert_func = flash_expert_func
__all__ = ["triton_flash_expert_func", "FlashExpertFunc"]
