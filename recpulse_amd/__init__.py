"""recpulse_amd — MI355X (gfx950) device layer for the RecPulse matmul path.

`recpulse_amd.capi` binds the C ABI of ``lib/librp_hip.so`` (declared in
``include/rp_hip.h``) with ctypes.  There is no CPU fallback: importing works
anywhere, but every compute call needs the built library and a GPU, and fails
loudly otherwise.
"""
__version__ = "0.1.0"
