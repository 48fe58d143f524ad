"""GGUF file intake for the raw block layout the kernels consume."""
