"""MoE routing index kernels of the gfx950 backend."""
