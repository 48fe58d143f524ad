"""The benchmark configurations as they are stated, through the C ABI, against the oracle.

  C1  one Q4_K GEMV, weight 17408 x 5120 float32 ~ N(0, 0.02) through the Q4_K quantizer (every row distinct),
      activation one float32 vector ~ N(0, 1); the full CPU reference (dequantize -> float32 matmul on the
      q8_1-dequantized activation) is the comparison, at batch 1 and batch 8.
  C3  the MMQ prefill GEMM at M = 512 and M = 8192 on the 17408 x 5120 Q4_K and 5120 x 17408 Q6_K shapes
      (M = 2048 is in test_gpu_fullsize.py), bf16 activations ~ N(0, 1): sampled rows against the MMQ formula
      and the reference CPU GEMV, every output feature of those rows.
  C5  the seven (type, K, N) matrices of one 27B-shaped layer (q, k, v, o, gate, up, down) at batch 1 and 8.
"""

from __future__ import annotations

import numpy as np
import pytest

from oracle import gguf_oracle as O
from hipengine_amd.kernels.hip_gfx950.quant import gguf_mmq_prefill as M
from hipengine_amd.kernels.hip_gfx950.quant import gguf_q8_1_gemv as G
from hipengine_amd.kernels.hip_gfx950.quant import gguf_quantize as Q

pytestmark = pytest.mark.gpu

REL_TOL = 1e-3
COS_MIN = 0.99999


def _close(got, ref):
    err, cos = O.max_rel_err(got, ref), O.cosine(got, ref)
    assert err <= REL_TOL, f"max rel err {err}"
    assert cos >= COS_MIN, f"cosine {cos}"


def _gemv(dev, short, qt, w, dw, x):
    rows, k = x.shape
    n = w.shape[0]
    dx = dev.put(x)
    dout = dev.empty(rows * n * 4, fill=0xFF)
    G.FUSED[(short, "f32", "f32")](dx.ptr, dw.ptr, dout.ptr, rows, k, n)
    got = dev.get(dout, np.float32, (rows, n)).copy()
    dev.free(dx, dout)
    return got


def test_c1_as_stated(dev):
    n, k = 17408, 5120
    w = O.random_weight(O.GGML_Q4_K, n, k, seed=20260101)          # N(0, 0.02) -> Q4_K, 17408 distinct rows
    assert w.shape == (n, k // 256 * 144)
    dw = dev.put(w)
    rng = np.random.default_rng(20260102)
    for rows in (1, 8):
        x = rng.standard_normal((rows, k)).astype(np.float32)     # N(0, 1)
        got = _gemv(dev, "q4_k", O.GGML_Q4_K, w, dw, x)
        xq = O.quantize_q8_1(x)
        ref = O.gguf_quant_gemv_chunked(O.dequantize_q8_1(xq), w, O.GGML_Q4_K)
        _close(got, ref)
        kl, top1 = O.softmax_kl_top1(O.gguf_quant_gemv_chunked(x, w, O.GGML_Q4_K), got)   # reported floor only
        assert kl <= 0.05 and top1 >= 0.75, (kl, top1)
    dev.free(dw)


C5_SHAPES = [   # (name, type, K, N) of one layer: hidden 5120, 40 query and 8 KV heads of 128, FFN 17408
    ("q", "q4_k", O.GGML_Q4_K, 5120, 5120), ("k", "q4_k", O.GGML_Q4_K, 5120, 1024), ("v", "q6_k", O.GGML_Q6_K, 5120, 1024),
    ("o", "q4_k", O.GGML_Q4_K, 5120, 5120), ("gate", "q4_k", O.GGML_Q4_K, 5120, 17408),
    ("up", "q4_k", O.GGML_Q4_K, 5120, 17408), ("down", "q6_k", O.GGML_Q6_K, 17408, 5120),
]


@pytest.mark.parametrize("name,short,qt,k,n", C5_SHAPES, ids=[s[0] for s in C5_SHAPES])
def test_c5_layer_shapes(dev, name, short, qt, k, n):
    w = O.random_weight(qt, n, k, seed=sum(map(ord, name)) + k)
    dw = dev.put(w)
    rng = np.random.default_rng(n + k)
    for rows in (1, 8):
        x = rng.standard_normal((rows, k)).astype(np.float32)
        got = _gemv(dev, short, qt, w, dw, x)
        _close(got, O.gguf_quant_gemv_chunked(O.dequantize_q8_1(O.quantize_q8_1(x)), w, qt))
    dev.free(dw)


SAMPLE = 10


@pytest.mark.parametrize("quant,k,n", [("q4_k", 5120, 17408), ("q6_k", 17408, 5120)])
@pytest.mark.parametrize("m", [512, 8192])
def test_c3_mmq_full_shape(dev, quant, k, n, m):
    qt = O.GGML_Q4_K if quant == "q4_k" else O.GGML_Q6_K
    w = O.random_weight(qt, n, k, seed=m + n)
    rng = np.random.default_rng(m + k)
    xb = O.f32_to_bf16_bits(rng.standard_normal((m, k)).astype(np.float32))     # bf16 ~ N(0, 1)
    dx, dw = dev.put(xb), dev.put(w)
    blk = 144 if quant == "q4_k" else 160
    dxq = dev.empty(m * (k // 128) * blk)
    dout = dev.empty(m * n * 4, fill=0xFF)
    if quant == "q4_k":
        Q.gguf_q8_1_mmq_ds4_pack_bf16(dx.ptr, dxq.ptr, m, k)
        M.gguf_q4_k_q8_1_mmq32_vdr_dense_bf16_f32_out(dxq.ptr, dw.ptr, dout.ptr, m, k, n)
    else:
        Q.gguf_q8_1_d4s4_f32_quantize_bf16(dx.ptr, dxq.ptr, m, k)
        M.gguf_q6_k_mmq32_q8_1_d4s4_f32_bf16_f32_out(dxq.ptr, dw.ptr, dout.ptr, m, k, n)
    got = dev.get(dout, np.float32, (m, n))
    packed = dev.get(dxq, np.uint8, (m, k // 128, blk))
    dev.free(dx, dw, dxq, dout)
    assert not np.isnan(got).any()                                   # every element written (the poison is NaN)
    rows = np.unique(np.concatenate([[0, 1, 31, 32, 127, 128, m - 1], rng.integers(0, m, size=SAMPLE)]))
    if quant == "q4_k":
        want_pack = O.pack_q8_1_ds4(xb[rows])
        ref = O.mmq_q4_k_ds4(want_pack, w)
        xd, _, q8 = O.ds4_fields(want_pack)
    else:
        want_pack = O.pack_q8_1_d4s4(xb[rows])
        ref = O.mmq_q6_k_d4s4(want_pack, w)
        xd, _, q8 = O.d4s4_fields(want_pack)
    assert np.array_equal(packed[rows], want_pack)
    _close(got[rows], ref)
    x_deq = (q8.astype(np.float32) * xd[..., None]).reshape(len(rows), k)
    cpu = O.gguf_quant_gemv_chunked(x_deq, w, qt)
    if quant == "q4_k":   # the MMQ's min term uses the fp16 sum of the raw activations, the CPU GEMV the quantized ones
        np.testing.assert_allclose(got[rows], cpu, rtol=2e-2, atol=1e-2 * (np.abs(cpu).max() + 1))
        assert O.cosine(got[rows], cpu) >= 0.9995
    else:
        _close(got[rows], cpu)
