"""``triton_peer_func`` under the reference's import path; it is the HIP op."""
from flash_moe.ops.hip.peer import PEERFunc, peer_func

triton_peer_func = peer_func
TritonPEERFunc = PEERFunc
__all__ = ["triton_peer_func", "TritonPEERFunc"]
