"""FlashMoE forward path on AMD MI355X (gfx950): hand-written HIP kernels behind a C ABI.

The import paths, class names and call signatures are those of flash-algo/flash-moe
(``flash_moe.modules.flash_moe.FlashMoE``, ``flash_moe.ops.*``), so code written against the
reference runs on this package unchanged.
"""
__version__ = "0.1.0"
