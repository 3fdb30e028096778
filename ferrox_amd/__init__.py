"""ferrox_amd: MI355X (gfx950) backend for the Ferrox training hot path.

Product code lives in csrc/ (HIP kernels + C ABI, built into libferrox_hip.so) and the host-side mirror of
Ferrox's storage/operator interface.  `ferrox_amd.capi` is the ctypes binding of the C ABI.
"""
__all__ = ["capi"]
