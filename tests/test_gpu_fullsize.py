"""GPU parity at the full sizes of the headline workloads, through the C ABI.

The weight tensors are ``synthetic_blocks``: ``TILE`` distinct random block rows
repeated down the tensor.  That gives two checks whose cost does not grow with
the tensor:

  * the first ``TILE`` output features are compared with the reference CPU GEMV
    (dequantize -> float32 matmul) applied to the dequantized q8 activations, to
    max relative error <= 1e-3 and cosine >= 0.99999;
  * every later output feature repeats feature ``n % TILE``.  The MMQ GEMM sums a
    feature's K blocks in an order that does not depend on where the feature sits,
    so there the repeats must be equal bit for bit.  The decode GEMV's stream form
    assigns the K blocks of a row to lanes by the row's offset in its wave's run, so
    its float32 summation order varies with position: there every repeat is held to
    the same tolerance against the reference of feature ``n % TILE``.

Shapes: Qwen3.6-27B FFN gate/up (17408x5120 Q4_K), FFN down (5120x17408 Q6_K),
attention output (5120x5120 Q8_0), lm_head (151936x5120 Q6_K) for the decode GEMV
at batch 1..8, and the Q4_K / Q6_K MMQ prefill GEMM at M = 2048.
"""

from __future__ import annotations

import numpy as np
import pytest

from oracle import gguf_oracle as O
from hipengine_amd.kernels.hip_gfx950.quant import gguf_mmq_prefill as M
from hipengine_amd.kernels.hip_gfx950.quant import gguf_q8_1_gemv as G
from hipengine_amd.synthetic import synthetic_blocks

pytestmark = pytest.mark.gpu

REL_TOL = 1e-3
COS_MIN = 0.99999
TILE = 1024


def _assert_periodic(got: np.ndarray):
    """Column n of ``got`` equals column n % TILE bit for bit."""
    bits = got.view(np.uint32 if got.dtype == np.float32 else np.uint16)
    n = bits.shape[1]
    first = bits[:, :TILE]
    for c0 in range(TILE, n, TILE):
        part = bits[:, c0:c0 + TILE]
        assert np.array_equal(part, first[:, :part.shape[1]]), f"features {c0}.. differ from features 0.."


def _assert_close(got, ref):
    err, cos = O.max_rel_err(got, ref), O.cosine(got, ref)
    assert err <= REL_TOL, f"max rel err {err}"
    assert cos >= COS_MIN, f"cosine {cos}"


GEMV_SHAPES = [
    ("q4_k", O.GGML_Q4_K, 17408, 5120),
    ("q6_k", O.GGML_Q6_K, 5120, 17408),
    ("q8_0", O.GGML_Q8_0, 5120, 5120),
    ("q6_k", O.GGML_Q6_K, 151936, 5120),
]


@pytest.mark.parametrize("short,qt,n,k", GEMV_SHAPES, ids=lambda v: str(v))
def test_decode_gemv_full_size(dev, short, qt, n, k):
    w = synthetic_blocks(qt, n, k, seed=n + k, tile_rows=TILE)
    dw = dev.put(w)
    rng = np.random.default_rng(k)
    dout = dev.empty(8 * n * 4)
    for batch in (1, 2, 4, 8):
        # fresh activations and a freshly poisoned output for every batch: the batches take different kernel
        # forms, and an element one of them failed to write must not pass on what the previous one left there
        x = (rng.standard_normal((batch, k)) * 0.5).astype(np.float32)
        dx = dev.put(x)
        dev.runtime.memset(dout.ptr, 0xFF, 8 * n * 4)         # all-ones bits: NaN as float32
        G.FUSED[(short, "f32", "f32")](dx.ptr, dw.ptr, dout.ptr, batch, k, n)
        got = dev.get(dout, np.float32, (8, n))
        dev.free(dx)
        assert np.all(got[batch:].view(np.uint32) == 0xFFFFFFFF)   # rows past the batch are not touched
        ref = O.gguf_quant_gemv(O.dequantize_q8_1(O.quantize_q8_1(x)), w[:TILE], qt)
        _assert_close(got[:batch], np.tile(ref, (1, -(-n // TILE)))[:, :n])
    dev.free(dw, dout)


def test_decode_gemv_full_size_bf16_in_bf16_out(dev):
    n, k = 17408, 5120
    w = synthetic_blocks(O.GGML_Q4_K, n, k, seed=3, tile_rows=TILE)
    x = (np.random.default_rng(4).standard_normal((1, k)) * 0.5).astype(np.float32)
    xb = O.f32_to_bf16_bits(x)
    dw, dx, dxb = dev.put(w), dev.put(O.bf16_bits_to_f32(xb)), dev.put(xb)
    d32, d16 = dev.empty(n * 4), dev.empty(n * 2)
    G.FUSED[("q4_k", "f32", "f32")](dx.ptr, dw.ptr, d32.ptr, 1, k, n)
    G.FUSED[("q4_k", "bf16", "bf16")](dxb.ptr, dw.ptr, d16.ptr, 1, k, n)
    f32 = dev.get(d32, np.float32, (1, n))
    b16 = dev.get(d16, np.uint16, (1, n))
    dev.free(dw, dx, dxb, d32, d16)
    assert np.array_equal(b16, O.f32_to_bf16_bits(f32))


def _bf16_rows(seed, rows, k):
    rng = np.random.default_rng(seed)
    return O.f32_to_bf16_bits((rng.standard_normal((rows, k)) * 0.1 + 0.002).astype(np.float32))


SAMPLE_ROWS = np.array([0, 1, 31, 32, 127, 128, 1000, 1023, 1024, 2047])


def test_q4_k_mmq_full_size(dev):
    rows, k, n = 2048, 5120, 17408
    w = synthetic_blocks(O.GGML_Q4_K, n, k, seed=5, tile_rows=TILE)
    ds4 = O.pack_q8_1_ds4(_bf16_rows(6, rows, k))
    dxq, dw = dev.put(ds4), dev.put(w)
    dout = dev.empty(rows * n * 4)
    M.gguf_q4_k_q8_1_mmq32_vdr_dense_bf16_f32_out(dxq.ptr, dw.ptr, dout.ptr, rows, k, n)
    got = dev.get(dout, np.float32, (rows, n))
    dev.free(dxq, dw, dout)
    _assert_periodic(got)
    _assert_close(got[SAMPLE_ROWS, :TILE], O.mmq_q4_k_ds4(ds4[SAMPLE_ROWS], w[:TILE]))
    # the reference CPU backend on the dequantized activations (min-term convention differs: rtol 2e-2)
    xd, _, q8 = O.ds4_fields(ds4[SAMPLE_ROWS])
    x_deq = (q8.astype(np.float32) * xd[..., None]).reshape(len(SAMPLE_ROWS), k)
    cpu = O.gguf_quant_gemv(x_deq, w[:TILE], O.GGML_Q4_K)
    np.testing.assert_allclose(got[SAMPLE_ROWS, :TILE], cpu, rtol=2e-2, atol=1e-2 * (np.abs(cpu).max() + 1))
    assert O.cosine(got[SAMPLE_ROWS, :TILE], cpu) >= 0.9999


def test_q6_k_mmq_full_size(dev):
    rows, k, n = 2048, 17408, 5120
    w = synthetic_blocks(O.GGML_Q6_K, n, k, seed=7, tile_rows=TILE)
    d4s4 = O.pack_q8_1_d4s4(_bf16_rows(8, rows, k))
    dxq, dw = dev.put(d4s4), dev.put(w)
    dout = dev.empty(rows * n * 4)
    M.gguf_q6_k_mmq32_q8_1_d4s4_f32_bf16_f32_out(dxq.ptr, dw.ptr, dout.ptr, rows, k, n)
    got = dev.get(dout, np.float32, (rows, n))
    dev.free(dxq, dw, dout)
    _assert_periodic(got)
    _assert_close(got[SAMPLE_ROWS, :TILE], O.mmq_q6_k_d4s4(d4s4[SAMPLE_ROWS], w[:TILE]))
    xd, _, q8 = O.d4s4_fields(d4s4[SAMPLE_ROWS])
    x_deq = (q8.astype(np.float32) * xd[..., None]).reshape(len(SAMPLE_ROWS), k)
    _assert_close(got[SAMPLE_ROWS, :TILE], O.gguf_quant_gemv(x_deq, w[:TILE], O.GGML_Q6_K))
