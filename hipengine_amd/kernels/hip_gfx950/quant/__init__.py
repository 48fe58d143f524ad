"""Raw-pointer wrappers of the gfx950 GGUF k-quant kernels."""
