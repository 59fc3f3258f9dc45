"""akg_amd: MI355X (gfx950) backend for AKG-MLIR fused operators - Python side.

The product is the C-ABI library `libakg_hip.so` (see include/akg_hip.h); this package holds its sources
(csrc/), the op descriptions it is measured on (fixtures/), and a ctypes mirror of the reference's driver.
"""
__version__ = "0.1"
