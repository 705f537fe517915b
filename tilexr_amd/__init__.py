"""tilexr_amd: MI355X-native MoE expert-parallel dispatch / combine behind the TileXR EP C ABI.

`tilexr_amd.ep` binds tilexr_amd/lib/libtilexr-ep.so (built by tilexr_amd/csrc/Makefile) with ctypes and offers
the same calls as the C header `include/tilexr_ep.h`, taking torch tensors for device memory.  There is no
fallback: if the library has not been built, importing `tilexr_amd.ep` raises.  `tilexr_amd.moonep` binds the
plan-driven Dispatch / Combine stages of the same library (`include/tilexr_moonep.h`).  `tilexr_amd.layer` wraps both
as torch-style methods (outputs allocated, stream hand-over done) for one rank per device.
"""

__all__ = ["ep", "moonep", "layer", "workloads"]
