"""MI355X (gfx950) backend for the matrix-multiplication path of Sapphire.

The product is the C ABI library built from sapphire_amd/csrc (declared in
include/sapphire_hip.h) and the C++ operator layer in sapphire_amd/host.
The Python modules here are plumbing around them:

    build   compiles both libraries in-tree with hipcc
    capi    ctypes binding of the C ABI (device buffers, events, entry points)
    synth   seeded synthetic inputs of the benchmark configurations
"""
__all__ = ["build", "capi", "synth"]
