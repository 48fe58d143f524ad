"""gfx950 (MI355X) kernels for hipEngine's GGUF k-quant matmul path.

The host side is torch-free: NumPy for shapes and byte math, ``ctypes`` for the
HIP runtime and for ``libhipengine_gfx950.so``.  Importing the package loads
neither.  There is no CPU implementation in here; every kernel entry point
raises if the library has not been built.
"""

__version__ = "0.1.0"
