"""Import-path compatibility with the reference only: it keeps its ops under ``flash_moe.ops.triton``.
Nothing here uses Triton; each module re-exports the HIP op under the reference's function name."""
