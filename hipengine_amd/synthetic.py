"""Synthetic raw GGUF block tensors for benchmarks and smoke runs.

Random block bytes with well-formed fields: quants and packed 6-bit scales are
uniform random bytes, the fp16 super-block scales are small finite positive
values.  No quantizer is involved; only shape, layout and byte count matter to
the kernels' speed, and parity checks compare against whatever bytes they are
given.
"""

from __future__ import annotations

import numpy as np

from hipengine_amd.quant.gguf import GGMLQuantizationType, quant_layout


def synthetic_blocks(qtype: int | GGMLQuantizationType, out_features: int, in_features: int, seed: int = 0,
                     tile_rows: int = 1024) -> np.ndarray:
    """uint8 ``[out_features, row_bytes]`` of random, finite blocks of ``qtype``.

    ``tile_rows`` distinct rows are generated and repeated down the tensor, which
    keeps generation of multi-hundred-megabyte tensors fast.
    """
    layout = quant_layout(qtype)
    if in_features % layout.block_size:
        raise ValueError(f"in_features must be a multiple of {layout.block_size}")
    nb = in_features // layout.block_size
    rows = min(tile_rows, out_features)
    rng = np.random.default_rng(seed)
    blk = rng.integers(0, 256, size=(rows, nb, layout.type_size), dtype=np.uint8)
    scale = (rng.random((rows, nb), dtype=np.float32) * 0.01 + 0.001).astype(np.float16).view(np.uint16)
    lo, hi = (scale & 0xFF).astype(np.uint8), (scale >> 8).astype(np.uint8)
    q = GGMLQuantizationType(int(qtype))
    if q == GGMLQuantizationType.Q6_K:
        blk[..., 208], blk[..., 209] = lo, hi
    else:                                    # Q4_K / Q5_K (d, dmin) and Q8_0 (d) keep their scale first
        blk[..., 0], blk[..., 1] = lo, hi
        if q in (GGMLQuantizationType.Q4_K, GGMLQuantizationType.Q5_K):
            blk[..., 2], blk[..., 3] = lo, hi
    tile = blk.reshape(rows, nb * layout.type_size)
    reps = -(-out_features // rows)
    return np.ascontiguousarray(np.tile(tile, (reps, 1))[:out_features])
