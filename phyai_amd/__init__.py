"""phyai_amd - MI355X (gfx950) native W8A8 fp8 quantized linear for PhyAI.

Hand-written HIP kernels behind a C ABI (``include/phyai_fp8.h``), with a Python
host side that mirrors the reference's ``Fp8Spec`` / ``LinearKernel`` plug-in
surface.  Importing the package does not touch the GPU; the native library is
loaded on first use and there is no fallback path without it.
"""

__version__ = "0.1.0"
