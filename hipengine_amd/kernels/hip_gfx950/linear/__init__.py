"""Dense-layer helpers of the decode path that are not quantized matmuls."""
