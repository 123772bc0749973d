"""zdraw_amd: MI355X (gfx950) backend for zdraw's DiT joint self-attention.

The product is the C-ABI shared library `lib/libzdraw_hip.so` (declared in
`include/zdraw_hip.h`) and the C++ host layer `lib/libzdraw_host.so`. The
Python modules here are thin ctypes bindings used by the tests and the
benchmark: `zdraw_amd.hip` binds the C ABI, `zdraw_amd.host` binds the host
layer that mirrors the reference's `attention_fast.run` / `mattn.Context`.
There is no CPU implementation in this package: without the built libraries
and a gfx950 device every entry point raises.
"""
__version__ = "0.1.0"
