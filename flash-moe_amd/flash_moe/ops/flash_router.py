"""``flash_moe.ops.flash_router`` is the path docs/flash_router.md:17 and tests/test_router.py:5 of the
reference import from."""
from flash_moe.ops.hip.flash_router import FlashRouterFunc, flash_router_func

triton_flash_router_func = flash_router_func
__all__ = ["flash_router_func", "triton_flash_router_func", "FlashRouterFunc"]
