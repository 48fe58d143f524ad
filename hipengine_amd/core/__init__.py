"""Thin torch-free runtime layer: HIP ctypes binding, device buffers, library build."""
