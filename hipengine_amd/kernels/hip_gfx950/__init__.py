"""Backend package ``hip_gfx950``: MI355X (CDNA4) kernels for the GGUF k-quant
matmul path.

hipEngine admits a backend through ``HIP_BACKEND_TARGET_ARCH`` plus a package
exposing ``register_backend_kernels(replace=False)``
(``hipengine/kernels/backends.py:35-38,129-148``); the constants below are the
source literals its consumer-surface reader looks for
(``loading/qwen35_gguf_consumer_surface.py:616-640``).
"""

from __future__ import annotations

BACKEND = "hip_gfx950"
TARGET_ARCH = "gfx950"
WAVEFRONT_SIZE = 64

GGUF_CONSUMER_LAYERS: frozenset[str] = frozenset({"linear", "moe_linear", "activation_quant", "embedding"})

_registered = False


def register_backend_kernels(replace: bool = False) -> None:
    """Register every gfx950 kernel wrapper under the ``hip_gfx950`` backend key."""
    global _registered
    if _registered and not replace:
        return
    from hipengine_amd.kernels.hip_gfx950.fused import paro_combine
    from hipengine_amd.kernels.hip_gfx950.linear import lm_head
    from hipengine_amd.kernels.hip_gfx950.moe import group_scatter, router
    from hipengine_amd.kernels.hip_gfx950.quant import (
        gguf_embedding,
        gguf_mmq_prefill,
        gguf_moe,
        gguf_q8_1_gemv,
        gguf_quantize,
    )

    gguf_quantize.register_kernels(BACKEND, replace=True)
    gguf_q8_1_gemv.register_kernels(BACKEND, replace=True)
    gguf_mmq_prefill.register_kernels(BACKEND, replace=True)
    gguf_moe.register_kernels(BACKEND, replace=True)
    group_scatter.register_kernels(BACKEND, replace=True)
    router.register_kernels(BACKEND, replace=True)
    gguf_embedding.register_kernels(BACKEND, replace=True)
    lm_head.register_kernels(BACKEND, replace=True)
    paro_combine.register_kernels(BACKEND, replace=True)
    _registered = True
