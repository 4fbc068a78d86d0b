"""``triton_flash_mlp_func`` under the reference's import path; it is the HIP op."""
from flash_moe.ops.hip.flash_mlp import FlashMLPFunc, flash_mlp_func

triton_flash_mlp_func = flash_mlp_func
__all__ = ["triton_flash_mlp_func", "FlashMLPFunc"]
