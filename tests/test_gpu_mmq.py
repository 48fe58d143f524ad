"""GPU parity of the activation packers (DS4, D4S4) and of the MMQ prefill GEMM
(int8 MFMA) through the C ABI.

Gates: packed activation bytes identical to the oracle's; float32 outputs within
max relative error 1e-3 / cosine 0.99999 of (a) the MMQ formula evaluated in
float64 and (b) the reference CPU GEMV (dequantize -> float32 matmul) applied to
the dequantized q8 activations (the pattern of
tests/test_gpu_gguf_k_mmq_prefill.py:528-541 in the hipEngine tree); bf16 output
equals bf16_round(float32 output); ctl and vdr entry points bit-identical;
repeated runs bit-identical.
"""

from __future__ import annotations

import numpy as np
import pytest

from oracle import c_oracle as C
from oracle import gguf_oracle as O
from hipengine_amd.kernels.hip_gfx950.quant import gguf_mmq_prefill as M
from hipengine_amd.kernels.hip_gfx950.quant import gguf_quantize as Q

pytestmark = pytest.mark.gpu


def _bf16_rows(seed, rows, k, scale=1.0, offset=0.0):
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal((rows, k)) * scale + offset).astype(np.float32)
    x[0, :32] = 0.0
    if rows > 2:
        x[2, 32:64] = np.arange(-16, 16) / 8.0
        x[2, 63] = 127.0 / 8.0          # exact .5 ties: DS4 rounds to even, D4S4 away from zero
    return O.f32_to_bf16_bits(x)


@pytest.mark.parametrize("rows,k", [(1, 128), (5, 1024), (33, 5120)])
def test_ds4_and_d4s4_pack_bytes(dev, rows, k):
    xb = _bf16_rows(rows + k, rows, k)
    dx = dev.put(xb)
    for fn, nbytes, want in ((Q.gguf_q8_1_mmq_ds4_pack_bf16, 144, O.pack_q8_1_ds4(xb)),
                             (Q.gguf_q8_1_d4s4_f32_quantize_bf16, 160, O.pack_q8_1_d4s4(xb))):
        dq = dev.empty(rows * (k // 128) * nbytes)
        fn(dx.ptr, dq.ptr, rows, k)
        got = dev.get(dq, np.uint8, want.shape)
        dev.free(dq)
        assert np.array_equal(got, want)
    assert np.array_equal(O.pack_q8_1_ds4(xb), C.pack_ds4(xb))
    dev.free(dx)


@pytest.mark.parametrize("tokens,top_k,k", [(1, 8, 2048), (7, 4, 512), (40, 2, 1280)])
def test_gather_ds4_pack_bytes(dev, tokens, top_k, k):
    """gguf_q8_1_mmq_gather_ds4_pack_bf16: the bytes of a row gather through sorted_lanes followed by the plain DS4
    pack; lanes that are negative or name a token outside the input pack as rows of zeros (scale 0, sum 0)."""
    xb = _bf16_rows(tokens + k, tokens, k)
    lanes = tokens * top_k
    rng = np.random.default_rng(lanes)
    sorted_lanes = rng.permutation(lanes).astype(np.int64)
    if lanes > 4:
        sorted_lanes[1] = -1
        sorted_lanes[3] = lanes + 5
    src = sorted_lanes // top_k
    gathered = np.zeros((lanes, k), dtype=np.uint16)
    ok = (sorted_lanes >= 0) & (src < tokens)
    gathered[ok] = xb[src[ok]]
    want = O.pack_q8_1_ds4(gathered)
    dx, dl = dev.put(xb), dev.put(sorted_lanes)
    dq = dev.empty(lanes * (k // 128) * 144)
    Q.gguf_q8_1_mmq_gather_ds4_pack_bf16(dx.ptr, dl.ptr, dq.ptr, lanes, k, tokens, top_k)
    got = dev.get(dq, np.uint8, want.shape)
    dev.free(dx, dl, dq)
    assert np.array_equal(got, want)
    with pytest.raises(ValueError):
        Q.gguf_q8_1_mmq_gather_ds4_pack_bf16(1, 1, 1, lanes, k + 64, tokens, top_k)


def _run_q4(dev, fn, ds4, w, rows, k, n, out_dtype=np.float32):
    dxq, dw = dev.put(ds4), dev.put(w)
    dout = dev.empty(rows * n * np.dtype(out_dtype).itemsize)
    fn(dxq.ptr, dw.ptr, dout.ptr, rows, k, n)
    got = dev.get(dout, out_dtype, (rows, n))
    dev.free(dxq, dw, dout)
    return got


@pytest.mark.parametrize("rows,k,n", [(1, 256, 32), (7, 512, 64), (128, 1024, 128), (130, 768, 160), (300, 5120, 416)])
def test_q4_k_mmq_matches_formula_and_cpu_reference(dev, rows, k, n):
    xb = _bf16_rows(7 * rows + k + n, rows, k, scale=0.1, offset=0.002)
    ds4 = O.pack_q8_1_ds4(xb)
    w = O.random_weight(O.GGML_Q4_K, n, k, seed=k + n)
    got = _run_q4(dev, M.gguf_q4_k_q8_1_mmq32_vdr_dense_bf16_f32_out, ds4, w, rows, k, n)
    want = O.mmq_q4_k_ds4(ds4, w)                     # float64 evaluation of the MMQ formula
    assert O.max_rel_err(got, want) <= 1e-3 and O.cosine(got, want) >= 0.99999
    assert O.max_rel_err(got, C.mmq_q4_k_ds4(ds4, w)) <= 1e-3
    # the reference CPU backend on the dequantized activations: equal up to the min-term
    # convention (fp16 raw sum vs xd*sum(q8)), which the reference test bounds at rtol 2e-2
    xd, _, qs = O.ds4_fields(ds4)
    xdeq = (xd[..., None] * qs.astype(np.float32)).reshape(rows, k)
    ref = O.gguf_quant_gemv(xdeq, w, O.GGML_Q4_K)
    np.testing.assert_allclose(got, ref, rtol=2e-2, atol=1e-2 * (np.abs(ref).max() + 1))
    assert O.cosine(got, ref) >= 0.9999


def test_q4_k_mmq_closed_form_weights(dev):
    rows, k, n = 40, 512, 96
    xb = _bf16_rows(3, rows, k, scale=0.125)
    ds4 = O.pack_q8_1_ds4(xb)
    w = O.closed_form_q4_k(n, k)
    got = _run_q4(dev, M.gguf_q4_k_q8_1_mmq32_vdr_dense_bf16_f32_out, ds4, w, rows, k, n)
    want = O.mmq_q4_k_ds4(ds4, w)
    assert O.max_rel_err(got, want) <= 1e-3 and O.cosine(got, want) >= 0.99999


def test_q4_k_mmq_siblings_bf16_and_determinism(dev):
    rows, k, n = 70, 1024, 96
    xb = _bf16_rows(11, rows, k)
    ds4 = O.pack_q8_1_ds4(xb)
    w = O.random_weight(O.GGML_Q4_K, n, k, seed=5)
    vdr = _run_q4(dev, M.gguf_q4_k_q8_1_mmq32_vdr_dense_bf16_f32_out, ds4, w, rows, k, n)
    ctl = _run_q4(dev, M.gguf_q4_k_q8_1_mmq32_ctl_dense_bf16_f32_out, ds4, w, rows, k, n)
    again = _run_q4(dev, M.gguf_q4_k_q8_1_mmq32_vdr_dense_bf16_f32_out, ds4, w, rows, k, n)
    assert np.array_equal(vdr.view(np.uint32), ctl.view(np.uint32))
    assert np.array_equal(vdr.view(np.uint32), again.view(np.uint32))
    b16 = _run_q4(dev, M.gguf_q4_k_q8_1_mmq32_vdr_dense_bf16_bf16_out, ds4, w, rows, k, n, out_dtype=np.uint16)
    assert np.array_equal(b16, O.f32_to_bf16_bits(vdr))


def test_q4_k_mmq_kernel_forms_agree(dev):
    rows, k, n = 150, 1536, 160
    xb = _bf16_rows(21, rows, k)
    ds4 = O.pack_q8_1_ds4(xb)
    w = O.random_weight(O.GGML_Q4_K, n, k, seed=9)
    import functools
    a = _run_q4(dev, functools.partial(M.gguf_q4_k_q8_1_mmq_tuned, variant=0), ds4, w, rows, k, n)
    b = _run_q4(dev, functools.partial(M.gguf_q4_k_q8_1_mmq_tuned, variant=1), ds4, w, rows, k, n)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    assert O.max_rel_err(a, O.mmq_q4_k_ds4(ds4, w)) <= 1e-3


@pytest.mark.parametrize("rows,k,n", [(1, 256, 1), (7, 512, 33), (128, 1024, 128), (130, 768, 160), (300, 5120, 200)])
def test_q6_k_mmq_matches_formula_and_cpu_reference(dev, rows, k, n):
    xb = _bf16_rows(5 * rows + k + n, rows, k, scale=0.1, offset=0.002)
    d4 = O.pack_q8_1_d4s4(xb)
    w = O.random_weight(O.GGML_Q6_K, n, k, seed=k + n + 1)
    got = _run_q4(dev, M.gguf_q6_k_mmq32_q8_1_d4s4_f32_bf16_f32_out, d4, w, rows, k, n)
    want = O.mmq_q6_k_d4s4(d4, w)                     # float64 evaluation of the MMQ formula
    assert O.max_rel_err(got, want) <= 1e-3 and O.cosine(got, want) >= 0.99999
    assert O.max_rel_err(got, C.mmq_q6_k_d4s4(d4, w)) <= 1e-3
    # the reference CPU backend (dequantize -> float32 matmul) on the dequantized activations
    xd, _, qs = O.d4s4_fields(d4)
    xdeq = (xd[..., None] * qs.astype(np.float32)).reshape(rows, k)
    ref = O.gguf_quant_gemv(xdeq, w, O.GGML_Q6_K)
    assert O.max_rel_err(got, ref) <= 1e-3 and O.cosine(got, ref) >= 0.99999


def test_q6_k_mmq_narrow_tiles(dev):
    """A shape whose 128-wide tiles would leave the last round of resident workgroups a quarter full takes 64-wide
    tiles (20 x 32 = 640 tiles against 1280): sampled rows against the formula, every row against the wide-tile
    result of the same columns computed as two half-width problems is not needed - the sums of an element do not
    depend on the tile, so a second shape that takes wide tiles on the same data must give the same bits."""
    rows, k, n = 2560, 256, 4096
    xb = _bf16_rows(21, rows, k, scale=0.1, offset=0.002)
    d4 = O.pack_q8_1_d4s4(xb)
    w = O.random_weight(O.GGML_Q6_K, n, k, seed=31)
    got = _run_q4(dev, M.gguf_q6_k_mmq32_q8_1_d4s4_f32_bf16_f32_out, d4, w, rows, k, n)
    pick = np.array([0, 1, 31, 32, 127, 128, 1000, 2047, 2048, 2559])
    want = O.mmq_q6_k_d4s4(d4[pick], w)
    assert O.max_rel_err(got[pick], want) <= 1e-3 and O.cosine(got[pick], want) >= 0.99999
    # the first 128 rows alone are one row of tiles: 32 wide tiles, filled 6 %, so the wide kernel runs them
    wide = _run_q4(dev, M.gguf_q6_k_mmq32_q8_1_d4s4_f32_bf16_f32_out, d4[:128], w, 128, k, n)
    assert np.array_equal(got[:128].view(np.uint32), wide.view(np.uint32))


def test_q6_k_mmq_closed_form_bf16_and_determinism(dev):
    rows, k, n = 70, 512, 96
    xb = _bf16_rows(13, rows, k, scale=0.125)
    d4 = O.pack_q8_1_d4s4(xb)
    w = O.closed_form_q6_k(n, k)
    f32 = _run_q4(dev, M.gguf_q6_k_mmq32_q8_1_d4s4_f32_bf16_f32_out, d4, w, rows, k, n)
    again = _run_q4(dev, M.gguf_q6_k_mmq32_q8_1_d4s4_f32_bf16_f32_out, d4, w, rows, k, n)
    want = O.mmq_q6_k_d4s4(d4, w)
    assert O.max_rel_err(f32, want) <= 1e-3 and O.cosine(f32, want) >= 0.99999
    assert np.array_equal(f32.view(np.uint32), again.view(np.uint32))
    b16 = _run_q4(dev, M.gguf_q6_k_mmq32_q8_1_d4s4_f32_bf16_bf16_out, d4, w, rows, k, n, out_dtype=np.uint16)
    assert np.array_equal(b16, O.f32_to_bf16_bits(f32))


@pytest.mark.parametrize("rows,k,n", [(1, 128, 1), (7, 384, 33), (128, 1024, 128), (130, 640, 160), (300, 5120, 200),
                                      (2560, 256, 4096)])
def test_q8_0_mmq_matches_formula_and_cpu_reference(dev, rows, k, n):
    """Q8_0 x D4S4 on the int8 MFMA (K a multiple of 128, any N; the last shape takes 64-wide tiles): the formula in
    float64, the reference CPU GEMV on the dequantized activations, bf16 output = bf16(float32 output), repeatable."""
    xb = _bf16_rows(3 * rows + k + n, rows, k, scale=0.1, offset=0.002)
    d4 = O.pack_q8_1_d4s4(xb)
    w = O.random_weight(O.GGML_Q8_0, n, k, seed=k + n + 2)
    got = _run_q4(dev, M.gguf_q8_0_mmq32_q8_1_d4s4_f32_bf16_f32_out, d4, w, rows, k, n)
    pick = np.arange(rows) if rows <= 300 else np.array([0, 1, 31, 32, 127, 128, 1000, 2047, 2048, 2559])
    want = O.mmq_q8_0_d4s4(d4[pick], w)
    assert O.max_rel_err(got[pick], want) <= 1e-3 and O.cosine(got[pick], want) >= 0.99999
    xd, _, qs = O.d4s4_fields(d4[pick])
    xdeq = (xd[..., None] * qs.astype(np.float32)).reshape(len(pick), k)
    ref = O.gguf_quant_gemv(xdeq, w, O.GGML_Q8_0)
    assert O.max_rel_err(got[pick], ref) <= 1e-3 and O.cosine(got[pick], ref) >= 0.99999
    again = _run_q4(dev, M.gguf_q8_0_mmq32_q8_1_d4s4_f32_bf16_f32_out, d4, w, rows, k, n)
    assert np.array_equal(got.view(np.uint32), again.view(np.uint32))
    b16 = _run_q4(dev, M.gguf_q8_0_mmq32_q8_1_d4s4_f32_bf16_bf16_out, d4, w, rows, k, n, out_dtype=np.uint16)
    assert np.array_equal(b16, O.f32_to_bf16_bits(got))
    if rows > 300:      # the first 128 rows alone take wide tiles: the same bits
        wide = _run_q4(dev, M.gguf_q8_0_mmq32_q8_1_d4s4_f32_bf16_f32_out, d4[:128], w, 128, k, n)
        assert np.array_equal(got[:128].view(np.uint32), wide.view(np.uint32))


def _random_q5_k(n, k, seed):
    """Random valid Q5_K blocks (the oracle has no fp32 -> Q5_K quantizer): every field drawn uniformly."""
    rng = np.random.default_rng(seed)
    nblk = n * (k // 256)
    blk = O.pack_q5_k_blocks(rng.integers(0, 32, size=(nblk, 8, 32), dtype=np.uint8),
                             rng.integers(0, 64, size=(nblk, 8), dtype=np.uint8),
                             rng.integers(0, 64, size=(nblk, 8), dtype=np.uint8),
                             (rng.random(nblk) * 0.05).astype(np.float32), (rng.random(nblk) * 0.02).astype(np.float32))
    return blk.reshape(n, -1)


@pytest.mark.parametrize("rows,k,n", [(1, 256, 32), (7, 512, 64), (128, 1024, 128), (130, 768, 160), (300, 5120, 224)])
def test_q5_k_mmq_matches_formula_and_cpu_reference(dev, rows, k, n):
    """Q5_K x D4S4 (gguf_k_mmq_prefill.hip:655-664) on the tile engine of the Q4_K GEMM: the formula in float64,
    and the reference CPU GEMV on the dequantized activations (which differs in the min term only: xd * sum(q8)
    against the raw float32 sum, so the gate there is the looser one hipEngine's own q8_1 tests use)."""
    xb = _bf16_rows(3 * rows + k + n, rows, k, scale=0.1, offset=0.002)
    d4 = O.pack_q8_1_d4s4(xb)
    w = _random_q5_k(n, k, seed=k + n + 2)
    got = _run_q4(dev, M.gguf_q5_k_mmq32_q8_1_d4s4_f32_bf16_f32_out, d4, w, rows, k, n)
    want = O.mmq_q5_k_d4s4(d4, w)
    assert O.max_rel_err(got, want) <= 1e-3 and O.cosine(got, want) >= 0.99999
    xd, _, qs = O.d4s4_fields(d4)
    xdeq = (xd[..., None] * qs.astype(np.float32)).reshape(rows, k)
    ref = O.gguf_quant_gemv(xdeq, w, O.GGML_Q5_K)
    assert O.cosine(got, ref) >= 0.9995
    np.testing.assert_allclose(got, ref, rtol=2e-2, atol=1e-2 * (np.abs(ref).max() + 1))


def test_q5_k_mmq_bf16_and_determinism(dev):
    rows, k, n = 70, 512, 96
    xb = _bf16_rows(17, rows, k, scale=0.125)
    d4 = O.pack_q8_1_d4s4(xb)
    w = O.closed_form_q5_k(n, k)
    f32 = _run_q4(dev, M.gguf_q5_k_mmq32_q8_1_d4s4_f32_bf16_f32_out, d4, w, rows, k, n)
    again = _run_q4(dev, M.gguf_q5_k_mmq32_q8_1_d4s4_f32_bf16_f32_out, d4, w, rows, k, n)
    want = O.mmq_q5_k_d4s4(d4, w)
    assert O.max_rel_err(f32, want) <= 1e-3 and O.cosine(f32, want) >= 0.99999
    assert np.array_equal(f32.view(np.uint32), again.view(np.uint32))
    b16 = _run_q4(dev, M.gguf_q5_k_mmq32_q8_1_d4s4_f32_bf16_bf16_out, d4, w, rows, k, n, out_dtype=np.uint16)
    assert np.array_equal(b16, O.f32_to_bf16_bits(f32))


def test_mmq_wrapper_rejects_bad_shapes(dev):
    f = M.gguf_q4_k_q8_1_mmq32_vdr_dense_bf16_f32_out
    with pytest.raises(ValueError, match="divisible"):
        f(1, 1, 1, 4, 300, 32)
    with pytest.raises(ValueError, match="divisible by 32"):
        f(1, 1, 1, 4, 256, 40)
    with pytest.raises(ValueError, match="rows"):
        f(1, 1, 1, 0, 256, 32)


def _mmq_sweep_cases():
    """32 seeded (quant, M, K, N) draws with ragged tiles in both dimensions and K from one step to 20."""
    rng = np.random.default_rng(77001)
    cases = []
    for i in range(32):
        quant = ("q4_k", "q5_k", "q6_k", "q8_0")[i % 4]
        m = int(rng.choice([1, 5, 31, 33, 64, 127, 129, 200, 257, 385]))
        k = (128 if quant == "q8_0" else 256) * int(rng.choice([1, 2, 3, 5, 8, 10]))
        n = int(rng.choice([1, 33, 63, 65, 127, 129, 200, 320, 513]))
        if quant in ("q4_k", "q5_k"):
            n = (n + 31) // 32 * 32          # these two take out_features in multiples of 32
        cases.append((quant, m, k, n))
    return cases


@pytest.mark.parametrize("quant,rows,k,n", _mmq_sweep_cases())
def test_mmq_seeded_shape_sweep(dev, quant, rows, k, n):
    xb = _bf16_rows(rows + 3 * k + 7 * n, rows, k, scale=0.2, offset=0.001)
    if quant == "q4_k":
        xq, w = O.pack_q8_1_ds4(xb), O.random_weight(O.GGML_Q4_K, n, k, seed=n + k)
        fn, want = M.gguf_q4_k_q8_1_mmq32_vdr_dense_bf16_f32_out, O.mmq_q4_k_ds4(xq, w)
    elif quant == "q5_k":
        xq, w = O.pack_q8_1_d4s4(xb), _random_q5_k(n, k, seed=n + k)
        fn, want = M.gguf_q5_k_mmq32_q8_1_d4s4_f32_bf16_f32_out, O.mmq_q5_k_d4s4(xq, w)
    elif quant == "q6_k":
        xq, w = O.pack_q8_1_d4s4(xb), O.random_weight(O.GGML_Q6_K, n, k, seed=n + k)
        fn, want = M.gguf_q6_k_mmq32_q8_1_d4s4_f32_bf16_f32_out, O.mmq_q6_k_d4s4(xq, w)
    else:
        xq, w = O.pack_q8_1_d4s4(xb), O.random_weight(O.GGML_Q8_0, n, k, seed=n + k)
        fn, want = M.gguf_q8_0_mmq32_q8_1_d4s4_f32_bf16_f32_out, O.mmq_q8_0_d4s4(xq, w)
    dxq, dw, dout = dev.put(xq), dev.put(w), dev.empty((rows * n + 4) * 4, fill=0x6B)
    fn(dxq.ptr, dw.ptr, dout.ptr, rows, k, n)
    got = dev.get(dout, np.float32, (rows * n + 4,)).copy()
    dev.free(dxq, dw, dout)
    assert np.all(got[rows * n:].view(np.uint32) == 0x6B6B6B6B)          # nothing past the output
    got = got[:rows * n].reshape(rows, n)
    assert O.max_rel_err(got, want) <= 1e-3 and O.cosine(got, want) >= 0.99999


def test_q5_k_and_q6_k_mmq_variant_names_are_the_same_gemm(dev):
    """hipEngine's pipe / mb4 / direct_dp4a names: the bits of the plain entries."""
    rows, k, n = 70, 512, 96
    xb = _bf16_rows(3, rows, k, scale=0.2)
    d4 = O.pack_q8_1_d4s4(xb)
    w5 = _random_q5_k(n, k, seed=4)
    base16 = _run_q4(dev, M.gguf_q5_k_mmq32_q8_1_d4s4_f32_bf16_bf16_out, d4, w5, rows, k, n, out_dtype=np.uint16)
    base32 = _run_q4(dev, M.gguf_q5_k_mmq32_q8_1_d4s4_f32_bf16_f32_out, d4, w5, rows, k, n)
    for fn in (M.gguf_q5_k_mmq32_pipe_q8_1_d4s4_f32_bf16_bf16_out, M.gguf_q5_k_mmq32_mb4_q8_1_d4s4_f32_bf16_bf16_out,
               M.gguf_q5_k_mmq32_direct_dp4a_q8_1_d4s4_f32_bf16_bf16_out):
        assert np.array_equal(_run_q4(dev, fn, d4, w5, rows, k, n, out_dtype=np.uint16), base16)
    got = _run_q4(dev, M.gguf_q5_k_mmq32_direct_dp4a_q8_1_d4s4_f32_bf16_f32_out, d4, w5, rows, k, n)
    assert np.array_equal(got.view(np.uint32), base32.view(np.uint32))
    from hipengine_amd.kernels.hip_gfx950._launch import I64, VOID, check_launch, entry
    w6 = O.random_weight(O.GGML_Q6_K, n, k, seed=6)
    base6 = _run_q4(dev, M.gguf_q6_k_mmq32_q8_1_d4s4_f32_bf16_bf16_out, d4, w6, rows, k, n, out_dtype=np.uint16)
    for name in ("pipe", "mb4"):
        sym = entry(f"hipengine_gguf_q6_k_mmq32_{name}_q8_1_d4s4_f32_bf16_bf16_out", [VOID, VOID, VOID, I64, I64, I64, VOID])
        fn = lambda xq, w, out, r, kk, nn, sym=sym: check_launch(sym(xq, w, out, r, kk, nn, 0), None)
        assert np.array_equal(_run_q4(dev, fn, d4, w6, rows, k, n, out_dtype=np.uint16), base6)
