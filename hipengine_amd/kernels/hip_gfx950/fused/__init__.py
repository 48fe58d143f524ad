"""Steps fused around the k-quant matmuls of an FFN block."""
