"""Kernel registry and the gfx950 backend package."""
