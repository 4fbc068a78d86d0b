"""``triton_flash_router_func`` under the reference's import path; it is the HIP op."""
from flash_moe.ops.hip.flash_router import FlashRouterFunc, flash_router_func

triton_flash_router_func = flash_router_func
__all__ = ["triton_flash_router_func", "FlashRouterFunc"]
