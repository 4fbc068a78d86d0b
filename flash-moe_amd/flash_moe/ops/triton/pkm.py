"""``triton_pkm_func`` under the reference's import path; it is the HIP op."""
from flash_moe.ops.hip.pkm import PKMFunc, pkm_func

triton_pkm_func = pkm_func
TritonPKMFunc = PKMFunc
__all__ = ["triton_pkm_func", "TritonPKMFunc"]
