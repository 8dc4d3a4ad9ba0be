"""MI355X (gfx950) implementation of the NAtS-L token-level hybrid attention forward path.

Python operator API identical to the reference's mixed operators; the compute is hand-written
HIP kernels reached through a C ABI (include/natsl.h, csrc/libnatsl.so).
"""
__version__ = "0.1.0"
