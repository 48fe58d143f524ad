"""GPU parity of the direct slab form of the decode GEMV (weights streamed straight into LDS, 16x16 int8 MFMA,
K optionally split over workgroups) through the C ABI.

Gates, as for the other forms: int32 sub-block dots of the production kernel body bit-exact against the
oracle's; float32 outputs max relative error <= 1e-3 and cosine >= 0.99999 against the reference CPU GEMV on the
q8_1-dequantized activations; results identical from launch to launch (the K parts are added in a fixed order
whichever workgroup arrives last).
"""

from __future__ import annotations

import numpy as np
import pytest

from oracle import gguf_oracle as O
from hipengine_amd.kernels.hip_gfx950.quant import gguf_q8_1_gemv as G
from hipengine_amd.kernels.hip_gfx950.quant import gguf_verify as V

pytestmark = pytest.mark.gpu

REL_TOL = 1e-3
COS_MIN = 0.99999
QT = {"gguf_q4_k": O.GGML_Q4_K, "gguf_q6_k": O.GGML_Q6_K, "gguf_q8_0": O.GGML_Q8_0}


def _close(got, ref):
    err, cos = O.max_rel_err(got, ref), O.cosine(got, ref)
    assert err <= REL_TOL, f"max rel err {err}"
    assert cos >= COS_MIN, f"cosine {cos}"


def _want_dots(quant, xq, w):
    qs = O.q8_1_fields(xq)[2]
    if quant == "gguf_q4_k":
        return O.block_dots_q4_k(qs, w)[0].astype(np.int32)
    if quant == "gguf_q6_k":
        return O.block_dots_q6_k(qs, w).astype(np.int32)
    return O.block_dots_q8_0(qs, w).astype(np.int32)


# (rows, K, N): one and two blocks per wave, ragged steps, several groups of steps per workgroup, K in 2 and 4 parts
SHAPES = [(8, 512, 16), (3, 1024, 100), (8, 5120, 544), (5, 4096, 1000), (1, 2048, 256 * 3 + 7), (6, 2048, 256 * 130 + 77),
          (8, 17408, 640), (3, 8192, 777), (2, 12288, 64)]


@pytest.mark.parametrize("quant", ["gguf_q4_k", "gguf_q6_k", "gguf_q8_0"])
@pytest.mark.parametrize("rows,k,n", SHAPES)
def test_dslab_dots_bit_exact_and_output(dev, quant, rows, k, n):
    rng = np.random.default_rng(rows + k + n)
    x = rng.standard_normal((rows, k)).astype(np.float32)
    xq = O.quantize_q8_1(x)
    w = O.random_weight(QT[quant], n, k, seed=n)
    per = k // 16 if quant == "gguf_q6_k" else k // 32
    dx, dxq, dw = dev.put(x), dev.put(xq), dev.put(w)
    ddots, dout, dout2 = dev.empty(rows * n * per * 4, fill=0x5A), dev.empty(rows * n * 4), dev.empty(rows * n * 4)
    V.gguf_gemv_mfma_dots_i32(quant, V.FORM_DSLAB, dxq.ptr, dw.ptr, ddots.ptr, dout.ptr, rows, k, n)
    G.gguf_q8_1_fused_gemv_dslab_tuned(quant, dx.ptr, "f32", dw.ptr, dout2.ptr, "f32", rows, k, n)
    dots = dev.get(ddots, np.int32, (rows, n, per)).copy()
    out_q = dev.get(dout, np.float32, (rows, n)).copy()
    out_f = dev.get(dout2, np.float32, (rows, n)).copy()
    dev.free(dx, dxq, dw, ddots, dout, dout2)
    assert np.array_equal(dots, _want_dots(quant, xq, w))
    ref = O.gguf_quant_gemv(O.dequantize_q8_1(xq), w, QT[quant])
    _close(out_q, ref)
    _close(out_f, ref)
    # float32 activations quantized in the kernel and pre-quantized q8_1 blocks give the same bits
    assert np.array_equal(out_q.view(np.uint32), out_f.view(np.uint32))


@pytest.mark.parametrize("quant,k,n,parts", [("gguf_q6_k", 17408, 5120, 4), ("gguf_q4_k", 5120, 3000, 2), ("gguf_q8_0", 4096, 1999, 4)])
def test_dslab_split_k_is_deterministic_and_rotates_regions(dev, quant, k, n, parts):
    """Twenty launches back to back (more than the library has scratch regions), no synchronization in between:
    every launch leaves the same bits, and they pass the gate."""
    rows = 8
    rng = np.random.default_rng(k + n)
    x = rng.standard_normal((rows, k)).astype(np.float32)
    w = O.random_weight(QT[quant], n, k, seed=3)
    dx, dw = dev.put(x), dev.put(w)
    outs = [dev.empty(rows * n * 4) for _ in range(20)]
    for o in outs:
        G.gguf_q8_1_fused_gemv_dslab_tuned(quant, dx.ptr, "f32", dw.ptr, o.ptr, "f32", rows, k, n, k_parts=parts)
    got = [dev.get(o, np.float32, (rows, n)).copy() for o in outs]
    dev.free(dx, dw, *outs)
    for g in got[1:]:
        assert np.array_equal(g.view(np.uint32), got[0].view(np.uint32))
    _close(got[0], O.gguf_quant_gemv(O.dequantize_q8_1(O.quantize_q8_1(x)), w, QT[quant]))


@pytest.mark.parametrize("quant,k,n", [("gguf_q6_k", 17408, 5120), ("gguf_q4_k", 8192, 2048)])
@pytest.mark.parametrize("rows", [3, 8])
def test_default_dispatch_takes_dslab_for_long_rows(dev, quant, k, n, rows):
    """Batch 3..8 of rows too long for one K part: the dense entry points and the residual epilogue run the
    direct slab form; bf16 in and out as hipEngine's dispatcher calls them."""
    assert G.gguf_gemv_default_form(quant, rows, k, n)[0] == "direct_slab"
    rng = np.random.default_rng(rows + k)
    x = (rng.standard_normal((rows, k)) * 0.5).astype(np.float32)
    xb = O.f32_to_bf16_bits(x)
    res = O.f32_to_bf16_bits(rng.standard_normal((rows, n)).astype(np.float32))
    w = O.random_weight(QT[quant], n, k, seed=5)
    short = quant.replace("gguf_", "")
    dx, dw, dres = dev.put(xb), dev.put(w), dev.put(res)
    dout, dout2 = dev.empty(rows * n * 2), dev.empty(rows * n * 2)
    G.FUSED[(short, "bf16", "bf16")](dx.ptr, dw.ptr, dout.ptr, rows, k, n)
    G.gguf_gemv_residual(quant, dx.ptr, "bf16", dw.ptr, dres.ptr, dout2.ptr, "bf16", rows, k, n)
    got = O.bf16_bits_to_f32(dev.get(dout, np.uint16, (rows, n)).copy())
    got_res = O.bf16_bits_to_f32(dev.get(dout2, np.uint16, (rows, n)).copy())
    dev.free(dx, dw, dres, dout, dout2)
    ref = O.gguf_quant_gemv(O.dequantize_q8_1(O.quantize_q8_1(O.bf16_bits_to_f32(xb))), w, QT[quant])
    # bf16 outputs: the float32 result rounded once (half an ulp of bf16 = 2^-9 relative)
    assert np.allclose(got, ref, rtol=2.0 ** -8, atol=1e-3 * np.abs(ref).max())
    want_res = O.bf16_bits_to_f32(O.f32_to_bf16_bits(ref)) + O.bf16_bits_to_f32(res)
    assert np.allclose(got_res, want_res, rtol=2.0 ** -7, atol=2e-3 * np.abs(want_res).max())
