"""cortex_amd -- an MI355X (gfx950) backend for the cortex tensor-math driver.

The package holds the hand-written HIP kernels and their C ABI (``csrc/``,
``include/cortex_hip.h``), a ctypes binding (:mod:`cortex_amd.capi`) and a
Python mirror of the reference's driver / tensor interface for this path.
"""

__all__ = ["capi"]
