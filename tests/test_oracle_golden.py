"""Pins the CPU oracle (oracle/gguf_oracle.py and oracle/gguf_oracle.c) before it
is trusted as the checker of the HIP kernels.  CPU only.

Sources of truth used here, none of which is the oracle's own formula retyped:
  * the reference's known-answer vectors (one-block Q8_0 / Q4_K dequant,
    tests/test_unit_gguf_quant_layout.py:41-80 in the hipEngine tree);
  * the reference's committed golden for the MoE FFN (tests/golden/);
  * inverse functions (pack <-> unpack round trips over boundary values);
  * float64 / int64 brute force over independently unpacked integers;
  * the two restatements (NumPy, C) against each other, bit for bit;
  * invariants of the quantizers and of the routing index.
"""

from __future__ import annotations

import json
from pathlib import Path

import numpy as np
import pytest

from oracle import c_oracle as C
from oracle import gguf_oracle as O

GOLDEN = Path(__file__).parent / "golden"


def f16_bytes(v: float) -> np.ndarray:
    return np.asarray([v], dtype=np.float16).view(np.uint8)


# ---------------------------------------------------------------- block unpack

def test_q8_0_one_block_known_answer():
    block = np.concatenate([f16_bytes(2.0), np.arange(-16, 16, dtype=np.int8).view(np.uint8)]).reshape(1, 34)
    want = np.arange(-16, 16, dtype=np.float32) * 2.0
    for deq in (O.dequantize, C.dequantize):
        out = deq(block, O.GGML_Q8_0)
        assert out.dtype == np.float32 and out.shape == (1, 32)
        np.testing.assert_array_equal(out[0], want)


def test_q4_k_one_superblock_known_answer():
    scales = np.zeros(12, dtype=np.uint8)
    scales[0] = 1                                   # first sub-block: scale 1, min 0
    qs = np.zeros(128, dtype=np.uint8)
    qs[:32] = np.arange(32, dtype=np.uint8) & 0x0F
    block = np.concatenate([f16_bytes(2.0), f16_bytes(0.0), scales, qs]).reshape(1, 144)
    want = (np.arange(32) & 0x0F).astype(np.float32) * 2.0
    for deq in (O.dequantize, C.dequantize):
        out = deq(block, O.GGML_Q4_K)
        assert out.shape == (1, 256)
        np.testing.assert_array_equal(out[0, :32], want)
        np.testing.assert_array_equal(out[0, 32:], 0.0)


def test_q4_k_high_nibble_and_min_known_answer():
    """Second sub-block lives in the high nibbles of the first 32 bytes; mins subtract."""
    scales = np.zeros(12, dtype=np.uint8)
    scales[1] = 3       # sc[1] = 3
    scales[5] = 2       # mn[1] = 2
    qs = np.zeros(128, dtype=np.uint8)
    qs[:32] = (np.arange(32, dtype=np.uint8) % 16) << 4
    block = np.concatenate([f16_bytes(0.5), f16_bytes(0.25), scales, qs]).reshape(1, 144)
    for deq in (O.dequantize, C.dequantize):
        out = deq(block, O.GGML_Q4_K)[0]
        np.testing.assert_array_equal(out[32:64], 0.5 * 3 * (np.arange(32) % 16) - 0.25 * 2)
        np.testing.assert_array_equal(out[:32], 0.0)
        np.testing.assert_array_equal(out[64:], 0.0)


def test_q4_k_scale_min_round_trip_over_boundaries():
    edge = np.array([0, 1, 15, 16, 31, 32, 47, 48, 63], dtype=np.uint8)
    rng = np.random.default_rng(1)
    sc = np.concatenate([np.stack(np.meshgrid(edge, edge), -1).reshape(-1, 2).repeat(4, axis=1),
                         rng.integers(0, 64, size=(4096, 8), dtype=np.uint8)])
    mn = np.roll(sc, 3, axis=1)[::-1].copy()
    packed = O.pack_q4_k_scale_min(sc, mn)
    for unpack in (O.q4_k_scale_min, C.q4_k_scale_min):
        got_sc, got_mn = unpack(packed)
        np.testing.assert_array_equal(got_sc, sc)
        np.testing.assert_array_equal(got_mn, mn)
    # scalar per-sub-block statement of the unpack, independent of the vectorised one
    s = packed[7]
    for j in range(8):
        want_sc = (s[j] & 63) if j < 4 else ((s[j + 4] & 0x0F) | ((s[j - 4] >> 6) << 4))
        want_mn = (s[j + 4] & 63) if j < 4 else ((s[j + 4] >> 4) | ((s[j] >> 6) << 4))
        assert (want_sc, want_mn) == (sc[7, j], mn[7, j])


def test_q6_k_unpack_is_inverse_of_the_block_builder():
    rng = np.random.default_rng(2)
    n = 64
    q = rng.integers(-32, 32, size=(n, 256)).astype(np.int8)
    sc = rng.integers(-128, 128, size=(n, 16)).astype(np.int8)
    d = (rng.random(n).astype(np.float32) * 0.01).astype(np.float16).astype(np.float32)
    blocks = O.pack_q6_k_blocks(q, sc, d)
    np.testing.assert_array_equal(O.q6_k_quants(blocks).reshape(n, 256), q)
    np.testing.assert_array_equal(C.unpack_int(blocks, O.GGML_Q6_K), q)
    want = (d[:, None].astype(np.float64) * np.repeat(sc, 16, axis=1) * q).astype(np.float32)   # exact products
    np.testing.assert_array_equal(O.dequantize(blocks, O.GGML_Q6_K), want)
    np.testing.assert_array_equal(C.dequantize(blocks, O.GGML_Q6_K), want)
    # element map spelled out for single elements (builder side, independent loop)
    b = np.zeros((1, 210), dtype=np.uint8)
    k = 5 * 32 + 7                     # group 5: second half, second 32-byte group, low nibble; qh shift 2
    u = 0b101101
    b[0, 64 + 32 + 7] |= u & 0x0F
    b[0, 128 + 32 + 7] |= (u >> 4) << 2
    assert int(O.q6_k_quants(b)[0].reshape(256)[k]) == u - 32
    assert int(C.unpack_int(b, O.GGML_Q6_K)[0, k]) == u - 32


def test_closed_form_weights_match_their_formulas_and_both_dequantizers_agree():
    for qt, gen in ((O.GGML_Q4_K, O.closed_form_q4_k), (O.GGML_Q6_K, O.closed_form_q6_k), (O.GGML_Q8_0, O.closed_form_q8_0)):
        w = gen(37, 768)
        a, b = O.dequantize(w, qt), C.dequantize(w, qt)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    # Q4_K closed form evaluated straight from its definition at (o=9, b=2, k=77)
    w = O.closed_form_q4_k(12, 768)
    o, b, k = 9, 2, 77
    j = k >> 5
    want = 0.015625 * (1 + o % 5) * ((3 * j + o + b) % 63 + 1) * ((k + 7 * o + 11 * b) % 16) - 0.0078125 * (1 + b % 3) * ((5 * j + 2 * o + b) % 17)
    assert O.dequantize(w, O.GGML_Q4_K)[o, b * 256 + k] == np.float32(want)
    w = O.closed_form_q6_k(12, 768)
    want = 0.0078125 * (1 + o % 7) * (((3 * (k >> 4) + o + b) % 33) - 16) * (((k + 11 * o + 19 * b) % 64) - 32)
    assert O.dequantize(w, O.GGML_Q6_K)[o, b * 256 + k] == np.float32(want)
    w = O.closed_form_q8_0(12, 768)
    kk, bb = 13, 5
    want = 0.03125 * (1 + o % 5) * (((kk + 7 * o + 3 * bb) % 31) - 15)
    assert O.dequantize(w, O.GGML_Q8_0)[o, bb * 32 + kk] == np.float32(want)


def test_random_weights_dequantize_identically_in_both_restatements():
    for qt in (O.GGML_Q4_K, O.GGML_Q6_K, O.GGML_Q8_0):
        w = O.random_weight(qt, 96, 1024, seed=qt)
        a, b = O.dequantize(w, qt), C.dequantize(w, qt)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
        src = np.random.default_rng(qt).standard_normal((96, 1024), dtype=np.float32) * np.float32(0.02)
        rel = float(np.sqrt(np.mean((a - src) ** 2)) / src.std())
        assert rel < {O.GGML_Q4_K: 0.12, O.GGML_Q6_K: 0.04, O.GGML_Q8_0: 0.01}[qt]   # the quantizers do quantize


# ---------------------------------------------------------------- reference CPU GEMV

@pytest.mark.parametrize("qt,gen,n", [(O.GGML_Q4_K, O.closed_form_q4_k, 5), (O.GGML_Q6_K, O.closed_form_q6_k, 7),
                                      (O.GGML_Q8_0, O.closed_form_q8_0, 6)])
def test_cpu_gemv_is_dequantize_then_matmul(qt, gen, n):
    x = ((np.arange(2 * 512, dtype=np.float32).reshape(2, 512) % 13) - 6) / 8.0
    w = gen(n, 512)
    out = O.gguf_quant_gemv(x, w, qt)
    assert out.dtype == np.float32 and out.shape == (2, n)
    want = x.astype(np.float64) @ O.dequantize(w, qt).astype(np.float64).T
    np.testing.assert_allclose(out, want, rtol=0.0, atol=1e-6 * np.abs(want).max())
    np.testing.assert_allclose(C.gemv_dequant(x, w, qt), want, rtol=0.0, atol=1e-6 * np.abs(want).max())
    np.testing.assert_allclose(O.gguf_quant_gemv_chunked(x, w, qt, chunk_rows=3), out, rtol=1e-6, atol=1e-6)
    with pytest.raises(ValueError):
        O.gguf_quant_gemv(x[:, :256], w, qt)


# ---------------------------------------------------------------- MoE golden

def moe_fixture_inputs() -> dict:
    """Inputs of the reference's MoE golden, from the recipe its test states."""
    rng = np.random.default_rng(20260609)
    tokens, hidden, ffn, experts = 4, 256, 256, 4
    x = rng.standard_normal((tokens, hidden)).astype(np.float32) * np.float32(1.0e-3)
    residual = rng.standard_normal((tokens, hidden)).astype(np.float32) * np.float32(0.25)
    selected = np.array([[0, 1], [1, 2], [2, 3], [3, 0]], dtype=np.int64)
    logits = rng.standard_normal((tokens, 2)).astype(np.float32)
    e = np.exp(logits - logits.max(axis=1, keepdims=True))
    routing = (e / e.sum(axis=1, keepdims=True)).astype(np.float32)
    q8 = O.closed_form_q8_0(ffn, hidden)
    return {
        "x": x, "residual": residual, "selected": selected, "routing": routing,
        "gate": O.stack_experts(O.closed_form_q4_k(ffn, hidden), experts, seed=1),
        "up": O.stack_experts(O.closed_form_q4_k(ffn, hidden), experts, seed=5),
        "down": O.stack_experts(O.closed_form_q4_k(hidden, ffn), experts, seed=9),
        "shared_gate": q8, "shared_up": np.roll(q8, 3, axis=0), "shared_down": O.closed_form_q8_0(hidden, ffn),
        "shared_gate_logit_w": rng.standard_normal((hidden,)).astype(np.float32) * np.float32(0.05),
    }


def test_moe_selected_ffn_matches_the_reference_golden():
    golden = json.loads((GOLDEN / "moe_ffn_selected_gguf_q4_k.json").read_text())
    f = moe_fixture_inputs()
    got = O.moe_selected_ffn(f["x"], f["selected"], f["routing"], f["gate"], f["up"], f["down"])
    np.testing.assert_allclose(got, np.asarray(golden["expected_selected"], dtype=np.float32), rtol=1e-6, atol=1e-6)
    block = O.moe_ffn_block(f["x"], f["residual"], f["selected"], f["routing"], f["gate"], f["up"], f["down"],
                            f["shared_gate_logit_w"], f["shared_gate"], f["shared_up"], f["shared_down"])
    np.testing.assert_allclose(block, np.asarray(golden["expected_block"], dtype=np.float32), rtol=1e-6, atol=1e-6)


def test_moe_selected_ffn_row_invariance_and_cache_equivalence():
    f = moe_fixture_inputs()
    full = O.moe_selected_ffn(f["x"], f["selected"], f["routing"], f["gate"], f["up"], f["down"])
    nocache = O.moe_selected_ffn(f["x"], f["selected"], f["routing"], f["gate"], f["up"], f["down"], cache=False)
    np.testing.assert_array_equal(full, nocache)
    for t in range(4):
        one = O.moe_selected_ffn(f["x"][t:t + 1], f["selected"][t:t + 1], f["routing"][t:t + 1], f["gate"], f["up"], f["down"])
        np.testing.assert_array_equal(one[0], full[t])
    with pytest.raises(ValueError):
        O.moe_selected_ffn(f["x"], f["selected"] + 9, f["routing"], f["gate"], f["up"], f["down"])


# ---------------------------------------------------------------- q8_1 quantizers

def _rng_rows(seed, rows=6, k=512):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((rows, k)).astype(np.float32)
    x[0, 64:96] = 0.0
    x[1] *= 1e-4
    x[2] *= 1e3
    return x


def test_q8_1_quantizer_against_float64_and_invariants():
    x = _rng_rows(3)
    blocks = O.quantize_q8_1(x)
    assert np.array_equal(blocks, C.quantize_q8_1(x))
    d, s, qs = O.q8_1_fields(blocks)
    g = x.reshape(6, -1, 32).astype(np.float64)
    amax = np.abs(g).max(axis=-1)
    assert np.all(qs[amax == 0] == 0) and np.all(d[amax == 0] == 0)
    assert np.all(np.abs(qs.astype(int)) <= 127)
    top = np.take_along_axis(qs, np.abs(g).argmax(axis=-1)[..., None], axis=-1)[..., 0]
    assert np.all(np.abs(top[amax > 0].astype(int)) == 127)
    # float64 evaluation of round-half-away(x / (amax/127)); the float32 quotient can differ from
    # it only at exact ties, which the next test covers
    scale32 = (amax.astype(np.float32) / np.float32(127.0)).astype(np.float64)
    ratio = np.divide(g, scale32[..., None], out=np.zeros_like(g), where=scale32[..., None] > 0)
    want = np.sign(ratio) * np.floor(np.abs(ratio) + 0.5)
    near_tie = np.abs(np.abs(ratio) % 1.0 - 0.5) < 1e-4
    assert np.array_equal(qs[~near_tie], want[~near_tie].astype(np.int8))
    np.testing.assert_array_equal(d, scale32.astype(np.float16).astype(np.float32))
    np.testing.assert_allclose(s, g.sum(axis=-1), rtol=2e-3, atol=2e-3)
    deq = O.dequantize_q8_1(blocks).reshape(6, -1, 32)
    # half a step of rounding plus the fp16 rounding of d on |q| <= 127: 2^-11 relative for a
    # normal half, half the subnormal spacing 2^-24 below 2^-14
    d_err = np.maximum(scale32 * 2.0 ** -11, 2.0 ** -25)
    assert np.all(np.abs(deq - g) <= (0.5 * scale32 + 127 * d_err)[..., None] * (1 + 1e-6) + 1e-12)


def test_q8_1_ties_round_away_ds4_ties_round_to_even():
    """amax = 127/8 makes d = 1/8 exactly, so x = (n + 0.5)/8 are exact .5 ties."""
    x = np.zeros((1, 128), dtype=np.float32)
    x[0, 0] = 127.0 / 8.0
    x[0, 1:9] = (np.array([0, 1, 2, 3, -1, -2, -3, -4]) + 0.5) / 8.0
    for blocks in (O.quantize_q8_1(x), C.quantize_q8_1(x)):
        qs = O.q8_1_fields(blocks)[2][0, 0]
        assert qs[0] == 127 and list(qs[1:9]) == [1, 2, 3, 4, -1, -2, -3, -4]          # away from zero
    xb = O.f32_to_bf16_bits(x)
    assert np.array_equal(O.bf16_bits_to_f32(xb), x)                                   # exactly representable
    for blocks in (O.pack_q8_1_ds4(xb), C.pack_ds4(xb)):
        qs = O.ds4_fields(blocks)[2][0, 0]
        assert qs[0] == 127 and list(qs[1:9]) == [0, 2, 2, 4, 0, -2, -2, -4]           # to even
    for blocks in (O.pack_q8_1_d4s4(xb), C.pack_d4s4(xb)):
        qs = O.d4s4_fields(blocks)[2][0, 0]
        assert list(qs[1:9]) == [1, 2, 3, 4, -1, -2, -3, -4]


def test_ds4_and_d4s4_packs_against_float64_and_each_other():
    x = _rng_rows(4)
    x[3, :32] = 3.0e38            # scale above the fp16 range is clamped to 65504 (DS4 only)
    xb = O.f32_to_bf16_bits(x)
    xf = O.bf16_bits_to_f32(xb).astype(np.float64).reshape(6, -1, 32)
    ds4 = O.pack_q8_1_ds4(xb)
    assert np.array_equal(ds4, C.pack_ds4(xb))
    scale, ssum, qs = O.ds4_fields(ds4)
    amax = np.abs(xf).max(axis=-1)
    want_scale = np.minimum(65504.0, (amax.astype(np.float32) / np.float32(127.0)))
    np.testing.assert_array_equal(scale, want_scale.astype(np.float16).astype(np.float32))
    assert np.all(np.abs(qs.astype(int)) <= 127)
    ratio = np.divide(xf, want_scale.astype(np.float64)[..., None], out=np.zeros_like(xf), where=want_scale[..., None] > 0)
    near_tie = np.abs(np.abs(ratio) % 1.0 - 0.5) < 1e-4
    assert np.array_equal(qs[~near_tie], np.clip(np.rint(ratio), -127, 127)[~near_tie].astype(np.int8))
    fin = np.isfinite(xf.sum(axis=-1)) & (np.abs(xf.sum(axis=-1)) < 6e4)
    np.testing.assert_allclose(ssum[fin], xf.sum(axis=-1)[fin], rtol=2e-3, atol=2e-3)
    assert np.all(np.isfinite(ssum)) and np.all(np.isfinite(scale))
    d4 = O.pack_q8_1_d4s4(xb)
    assert np.array_equal(d4, C.pack_d4s4(xb))
    d, s, q = O.d4s4_fields(d4)
    np.testing.assert_array_equal(d, np.where(amax > 0, amax.astype(np.float32) / np.float32(127.0), 0).astype(np.float32))
    ok = np.abs(xf).sum(axis=-1) < 3.0e38          # the float32 sum of the huge block overflows, as on the device
    np.testing.assert_allclose(s[ok], xf.sum(axis=-1)[ok], rtol=1e-5, atol=1e-4 * np.abs(xf[ok]).max())


# ---------------------------------------------------------------- integer dots and combines

def test_block_dots_against_int64_brute_force():
    rng = np.random.default_rng(6)
    rows, k, n = 3, 512, 9
    xq = O.quantize_q8_1(rng.standard_normal((rows, k)).astype(np.float32))
    q8 = O.q8_1_fields(xq)[2].astype(np.int64)                                    # [rows, 16, 32]
    w4 = O.random_weight(O.GGML_Q4_K, n, k, seed=1)
    ints = C.unpack_int(w4, O.GGML_Q4_K).reshape(n, k // 32, 32).astype(np.int64)   # C unpack, NumPy dot
    want = np.einsum("rjk,njk->rnj", q8, ints)
    dots, qsum = O.block_dots_q4_k(O.q8_1_fields(xq)[2], w4)
    cd, cq = C.block_dots(xq, w4, O.GGML_Q4_K)
    assert np.array_equal(dots, want) and np.array_equal(cd, want)
    assert np.array_equal(qsum, q8.sum(axis=-1)) and np.array_equal(cq, q8.sum(axis=-1))
    w6 = O.random_weight(O.GGML_Q6_K, n, k, seed=2)
    ints = C.unpack_int(w6, O.GGML_Q6_K).reshape(n, k // 16, 16).astype(np.int64)
    want = np.einsum("rjk,njk->rnj", q8.reshape(rows, k // 16, 16), ints)
    assert np.array_equal(O.block_dots_q6_k(O.q8_1_fields(xq)[2], w6), want)
    assert np.array_equal(C.block_dots(xq, w6, O.GGML_Q6_K), want)
    w8 = O.random_weight(O.GGML_Q8_0, n, k, seed=3)
    ints = w8.reshape(n, k // 32, 34)[..., 2:].view(np.int8).astype(np.int64)
    want = np.einsum("rjk,njk->rnj", q8, ints)
    assert np.array_equal(O.block_dots_q8_0(O.q8_1_fields(xq)[2], w8), want)
    assert np.array_equal(C.block_dots(xq, w8, O.GGML_Q8_0), want)


def test_q8_1_gemv_formulas_equal_the_cpu_gemv_on_dequantized_activations():
    """sum xd*(d*sc*dot - dmin*mn*qsum) is algebraically W_deq . (xd*q8): the q8_1 route and the
    reference CPU GEMV fed the dequantized activations must agree to float rounding."""
    rng = np.random.default_rng(8)
    rows, k, n = 2, 1024, 24
    x = rng.standard_normal((rows, k)).astype(np.float32)
    xq = O.quantize_q8_1(x)
    xdeq = O.dequantize_q8_1(xq).astype(np.float64)
    for qt, f in ((O.GGML_Q4_K, O.gemv_q8_1_q4_k), (O.GGML_Q6_K, O.gemv_q8_1_q6_k), (O.GGML_Q8_0, O.gemv_q8_1_q8_0)):
        w = O.random_weight(qt, n, k, seed=qt)
        exact = xdeq @ O.dequantize(w, qt).astype(np.float64).T
        np.testing.assert_allclose(f(xq, w), exact, rtol=1e-9, atol=1e-9 * np.abs(exact).max())
        assert O.max_rel_err(C.gemv_q8_1(xq, w, qt), exact) < 2e-4
        assert O.max_rel_err(O.gguf_quant_gemv(xdeq.astype(np.float32), w, qt), exact) < 2e-4


def test_mmq_formulas_against_float64():
    rng = np.random.default_rng(9)
    rows, k, n = 5, 1024, 32
    xb = O.f32_to_bf16_bits((rng.standard_normal((rows, k)) * 0.1 + 0.002).astype(np.float32))
    w4 = O.random_weight(O.GGML_Q4_K, n, k, seed=4)
    ds4 = O.pack_q8_1_ds4(xb)
    xd, xs, qs = O.ds4_fields(ds4)
    wd = O.dequantize(w4, O.GGML_Q4_K).astype(np.float64)
    # W_deq . (xd*q8) differs from the MMQ formula only in the min term (fp16 raw sum vs xd*qsum)
    blocks = w4.reshape(-1, 144)
    sc, mn = O.q4_k_scale_min(blocks[:, 4:16])
    dmin = blocks[:, 2:4].copy().view(np.float16).astype(np.float64)
    dm = (dmin * mn).reshape(n, -1)
    dsc = (blocks[:, 0:2].copy().view(np.float16).astype(np.float64) * sc).reshape(n, -1)
    q4 = C.unpack_int(w4, O.GGML_Q4_K).reshape(n, -1, 32).astype(np.float64)
    main = np.einsum("rj,nj,rjk,njk->rn", xd.astype(np.float64), dsc, qs.astype(np.float64), q4)
    want = main - xs.astype(np.float64) @ dm.T
    np.testing.assert_allclose(O.mmq_q4_k_ds4(ds4, w4), want, rtol=1e-9, atol=1e-9 * np.abs(want).max())
    assert O.max_rel_err(C.mmq_q4_k_ds4(ds4, w4), want) < 2e-4
    w6 = O.random_weight(O.GGML_Q6_K, n, k, seed=5)
    d4 = O.pack_q8_1_d4s4(xb)
    d, _, q = O.d4s4_fields(d4)
    want = (d[..., None].astype(np.float64) * q).reshape(rows, k) @ O.dequantize(w6, O.GGML_Q6_K).astype(np.float64).T
    np.testing.assert_allclose(O.mmq_q6_k_d4s4(d4, w6), want, rtol=1e-9, atol=1e-9 * np.abs(want).max())
    assert O.max_rel_err(C.mmq_q6_k_d4s4(d4, w6), want) < 2e-4
    # Q8_0 x D4S4: exactly the product of the dequantized weight with the dequantized activations (no min term)
    w8 = O.random_weight(O.GGML_Q8_0, n, k, seed=8)
    want = (d[..., None].astype(np.float64) * q).reshape(rows, k) @ O.dequantize(w8, O.GGML_Q8_0).astype(np.float64).T
    np.testing.assert_allclose(O.mmq_q8_0_d4s4(d4, w8), want, rtol=1e-9, atol=1e-9 * np.abs(want).max())
    # Q5_K x D4S4: the Q4_K structure with 5-bit values and the float32 raw sum; an independent float64 evaluation
    # from the unpacked fields, and the dequantize-matmul identity it must stay close to (they differ in the min
    # term only: raw sum of the activations against xd * sum(q8))
    from hipengine_amd.synthetic import synthetic_blocks
    w5 = synthetic_blocks(O.GGML_Q5_K, n, k, seed=6, tile_rows=n)
    b5 = w5.reshape(-1, 176)
    sc5, mn5 = O.q4_k_scale_min(b5[:, 4:16])
    dsc5 = (b5[:, 0:2].copy().view(np.float16).astype(np.float64) * sc5).reshape(n, -1)
    dm5 = (b5[:, 2:4].copy().view(np.float16).astype(np.float64) * mn5).reshape(n, -1)
    q5 = O.q5_k_quants(b5).reshape(n, -1, 32).astype(np.float64)
    d, s4, q = O.d4s4_fields(d4)
    want = np.einsum("rj,nj,rjk,njk->rn", d.astype(np.float64), dsc5, q.astype(np.float64), q5) - s4.astype(np.float64) @ dm5.T
    got5 = O.mmq_q5_k_d4s4(d4, w5)
    np.testing.assert_allclose(got5, want, rtol=1e-9, atol=1e-9 * np.abs(want).max())
    deq = (d[..., None].astype(np.float64) * q).reshape(rows, k) @ O.dequantize(w5, O.GGML_Q5_K).astype(np.float64).T
    assert O.cosine(got5, deq) > 0.9999


# ---------------------------------------------------------------- fp16 / bf16 helpers of the C restatement

def test_c_fp16_conversions_match_numpy():
    lib = C.load()
    halves = np.arange(65536, dtype=np.uint16)
    want = halves.view(np.float16).astype(np.float32)
    got = np.array([lib.oracle_f16_to_f32(int(h)) for h in halves[::7]], dtype=np.float32)
    ok = ~np.isnan(want[::7])
    assert np.array_equal(got[ok].view(np.uint32), want[::7][ok].view(np.uint32))
    rng = np.random.default_rng(10)
    vals = np.concatenate([rng.standard_normal(4000).astype(np.float32) * s for s in (1e-8, 1e-6, 1e-4, 1.0, 300.0, 7e4)])
    with np.errstate(over="ignore"):
        want16 = vals.astype(np.float16).view(np.uint16)
    got16 = np.array([lib.oracle_f32_to_f16(float(v)) for v in vals], dtype=np.uint16)
    assert np.array_equal(got16, want16)
    bits = np.array([lib.oracle_f32_to_bf16(float(v)) for v in vals[:2000]], dtype=np.uint16)
    assert np.array_equal(bits, O.f32_to_bf16_bits(vals[:2000]))
    assert np.array_equal(O.bf16_bits_to_f32(np.array([0x3F80, 0xC020, 0x3F00], dtype=np.uint16)),
                          np.array([1.0, -2.5, 0.5], dtype=np.float32))


# ---------------------------------------------------------------- routing

def test_router_topk_softmax_brute_force_and_ties():
    rng = np.random.default_rng(11)
    lg = rng.standard_normal((16, 64)).astype(np.float32)
    lg[0, 5] = lg[0, 9] = lg[0].max() + 1.0          # a tie for first place: lowest index first
    sel, w = O.router_topk_softmax(lg, 8)
    assert sel[0, 0] == 5 and sel[0, 1] == 9
    for t in range(16):
        order = sorted(range(64), key=lambda e: (-float(lg[t, e]), e))[:8]
        assert list(sel[t]) == order
        e = np.exp(lg[t, order].astype(np.float64) - float(lg[t, order[0]]))
        np.testing.assert_allclose(w[t], e / e.sum(), rtol=1e-6)
    sel2, w2 = O.mtp_moe_routing(lg, 8)
    np.testing.assert_allclose(w2.sum(axis=-1), 1.0, rtol=1e-6)
    assert np.array_equal(np.sort(sel2, axis=-1), np.sort(sel, axis=-1))          # same expert sets, softmax is monotone
    np.testing.assert_allclose(w2, w, rtol=1e-5)                                  # and, renormalised, the same weights


def test_routing_index_invariants():
    rng = np.random.default_rng(12)
    t, k, e = 37, 8, 64
    sel = np.stack([rng.permutation(e)[:k] for _ in range(t)]).astype(np.int64)
    sel[3, 2] = -1                                    # dropped, as the device kernels drop it
    wts = rng.random((t, k)).astype(np.float32)
    idx = O.build_routing_index(sel, wts, e)
    flat = sel.reshape(-1)
    valid = np.nonzero((flat >= 0) & (flat < e))[0]
    assert idx["total"] == valid.size and idx["expert_start"][-1] == valid.size
    assert np.array_equal(np.diff(idx["expert_start"]), np.bincount(flat[valid], minlength=e))
    assert sorted(idx["sorted_lanes"]) == sorted(valid)                           # a permutation of the valid lanes
    for ex in range(e):
        seg = idx["sorted_lanes"][idx["expert_start"][ex]:idx["expert_start"][ex + 1]]
        assert np.all(flat[seg] == ex) and np.all(np.diff(seg) > 0)              # right expert, ascending lanes
    assert np.array_equal(idx["compact_to_source"], idx["sorted_lanes"] // k)
    assert np.array_equal(idx["sorted_weights"], wts.reshape(-1)[idx["sorted_lanes"]])
    assert idx["active_count"] == int((np.bincount(flat[valid], minlength=e) > 0).sum())
    padded = O.build_routing_index(sel, wts, e, pad_multiple=16)
    assert np.all(np.diff(padded["expert_start"]) % 16 == 0)
    assert np.array_equal(padded["sorted_lanes"][padded["sorted_lanes"] >= 0], idx["sorted_lanes"])
    tm = O.tile_map(idx["expert_start"], e, 32)
    counts = np.diff(idx["expert_start"])
    assert tm["total"] == int(((counts + 31) // 32 * 32).sum())
    for tile, ex in enumerate(tm["tile_expert"]):
        assert tm["tile_expert_start"][ex] <= tile * 32 < tm["tile_expert_start"][ex + 1]


def test_q5_k_dequant_against_the_block_builder_a_scalar_loop_and_q4_k():
    """Q5_K: (i) values packed by the reference's block builder come back exactly, and the closed-form
    generator equals its element formula d*sc*q - dmin*mn; (ii) a per-element scalar loop that follows
    the device lookup formula (qs nibble | bit sb of qh[lane] << 4) agrees; (iii) with qh = 0 a Q5_K block
    dequantizes like the Q4_K block with the same header and nibbles."""
    rng = np.random.default_rng(55)
    n = 6
    q5 = rng.integers(0, 32, size=(n, 8, 32), dtype=np.uint8)
    sc = rng.integers(0, 64, size=(n, 8), dtype=np.uint8)
    mn = rng.integers(0, 64, size=(n, 8), dtype=np.uint8)
    d = rng.random(n).astype(np.float16).astype(np.float32) * 0.05
    dmin = rng.random(n).astype(np.float16).astype(np.float32) * 0.02
    blk = O.pack_q5_k_blocks(q5, sc, mn, d, dmin)
    assert blk.shape == (n, 176)
    assert np.array_equal(O.q5_k_quants(blk), q5)
    d16, m16 = d.astype(np.float16).astype(np.float32), dmin.astype(np.float16).astype(np.float32)
    want = ((d16[:, None] * sc.astype(np.float32))[:, :, None] * q5.astype(np.float32)
            - (m16[:, None] * mn.astype(np.float32))[:, :, None]).reshape(n, 256)
    got = O.dequant_q5_k(blk)
    assert np.array_equal(got.view(np.uint32), want.astype(np.float32).view(np.uint32))
    # (ii) scalar loop over one block
    b0 = blk[0]
    scales = b0[4:16]
    def sc_of(s):
        return (scales[s] & 63) if s < 4 else ((scales[8 + s - 4] & 0x0F) | ((scales[s - 4] >> 2) & 0x30))
    def mn_of(s):
        return (scales[4 + s] & 63) if s < 4 else ((scales[8 + s - 4] >> 4) | ((scales[4 + s - 4] >> 2) & 0x30))
    for k in range(256):
        s, lane = k >> 5, k & 31
        packed = b0[48 + (s >> 1) * 32 + lane]
        ql = (packed >> 4) if (s & 1) else (packed & 0x0F)
        q = int(ql) | (((int(b0[16 + lane]) >> s) & 1) << 4)
        v = np.float32(d16[0]) * np.float32(sc_of(s)) * np.float32(q) - np.float32(m16[0]) * np.float32(mn_of(s))
        assert np.float32(v) == got[0, k]
    # (iii) qh = 0 -> Q4_K
    blk0 = blk.copy()
    blk0[:, 16:48] = 0
    q4 = np.concatenate([blk0[:, :16], blk0[:, 48:]], axis=1)
    assert np.array_equal(O.dequant_q5_k(blk0), O.dequant_q4_k(q4))
    # closed-form generator of the reference tests
    w = O.closed_form_q5_k(3, 512)
    deq = O.dequantize(w, O.GGML_Q5_K)
    for o in range(3):
        for b in range(2):
            dd, mm = np.float32(0.015625 * (1 + o % 5)), np.float32(0.0078125 * (1 + b % 3))
            for k in (0, 31, 32, 100, 255):
                j = k >> 5
                q = (k + 13 * o + 17 * b) % 32
                want1 = dd * np.float32((3 * j + o + b) % 63 + 1) * np.float32(q) - mm * np.float32((5 * j + 2 * o + b) % 17)
                assert deq[o, b * 256 + k] == np.float32(want1)


def test_embedding_lookup_definition_and_errors():
    w = O.closed_form_q4_k(9, 512)
    ids = np.array([3, 0, 8, 3], dtype=np.int64)
    assert np.array_equal(O.embedding_lookup(ids, w, O.GGML_Q4_K), O.dequantize(w, O.GGML_Q4_K)[ids])
    with pytest.raises(ValueError, match="out-of-range"):
        O.embedding_lookup(np.array([9]), w, O.GGML_Q4_K)
    with pytest.raises(ValueError, match="shape"):
        O.embedding_lookup(np.array([[1]]), w, O.GGML_Q4_K)


def test_argmax_rows_brute_force_with_ties():
    rng = np.random.default_rng(8)
    lg = rng.standard_normal((5, 97)).astype(np.float32)
    lg[1, [7, 40, 90]] = 9.0
    lg[2, :] = -1.5
    idx, val = O.argmax_rows(lg)
    for r in range(5):
        bv, bi = np.float32(-3.4028234663852886e38), 2**31 - 1
        for i in range(97):
            if lg[r, i] > bv or (lg[r, i] == bv and i < bi):
                bv, bi = lg[r, i], i
        assert idx[r] == bi and val[r] == bv
    assert idx[1] == 7 and idx[2] == 0


def test_q5_k_block_dots_against_int64_brute_force():
    rng = np.random.default_rng(77)
    n, k, rows = 3, 512, 2
    nblk = n * (k // 256)
    w = O.pack_q5_k_blocks(rng.integers(0, 32, size=(nblk, 8, 32), dtype=np.uint8), rng.integers(0, 64, size=(nblk, 8), dtype=np.uint8),
                           rng.integers(0, 64, size=(nblk, 8), dtype=np.uint8), np.full(nblk, 0.01, np.float32),
                           np.full(nblk, 0.005, np.float32)).reshape(n, -1)
    qs = rng.integers(-128, 128, size=(rows, k // 32, 32), dtype=np.int8)
    dots, qsum = O.block_dots_q5_k(qs, w)
    deq = O.q5_k_quants(w.reshape(-1, 176)).reshape(n, k).astype(np.int64)
    for r in range(rows):
        for row in range(n):
            for j in range(k // 32):
                assert dots[r, row, j] == int(np.dot(qs[r, j].astype(np.int64), deq[row, j * 32:(j + 1) * 32]))
        assert np.array_equal(qsum[r], qs[r].astype(np.int64).sum(axis=-1))


def test_moe_tail_next_rmsnorm_reference_known_answer_and_scalar_loop():
    """The reference's own known answer (tests/test_gpu_moe_tail_next_rmsnorm.py:98-119: both rounding boundaries,
    gate taken from column 0), a float64 scalar loop within one bf16 step, and the three input forms agreeing."""
    selected = np.asarray([[[0.5, -1.0], [0.5, -1.0]]], dtype=np.float32)
    rounded, normed = O.moe_tail_next_rmsnorm(selected, np.asarray([[2.0, 4.0]], np.float32),
                                              np.asarray([[0.0, 99.0]], np.float32), np.asarray([[3.0, -1.0]], np.float32),
                                              np.ones(2, np.float32), routing_weights=np.asarray([[1.0, 1.0]], np.float32))
    assert np.array_equal(rounded, np.asarray([[5.0, -1.0]], np.float32))
    scale = np.float32(1.0 / np.sqrt(np.mean(rounded * rounded, axis=-1, keepdims=True) + 1e-6))
    assert np.array_equal(normed, O.bf16_bits_to_f32(O.f32_to_bf16_bits(rounded * scale)))

    rng = np.random.default_rng(31)
    tokens, top_k, hidden = 3, 4, 24
    bf = lambda a: O.bf16_bits_to_f32(O.f32_to_bf16_bits(a.astype(np.float32)))
    slots = bf(rng.standard_normal((tokens, top_k, hidden)) * 0.3)
    shared, residual = bf(rng.standard_normal((tokens, hidden)) * 0.3), bf(rng.standard_normal((tokens, hidden)))
    routing = rng.uniform(-0.5, 0.75, (tokens, top_k)).astype(np.float32)
    gate = rng.uniform(-4, 4, (tokens, 3)).astype(np.float32)
    weight = rng.uniform(0.5, 1.5, hidden).astype(np.float32)
    got_r, got_n = O.moe_tail_next_rmsnorm(slots, shared, gate, residual, weight, routing_weights=routing, eps=1e-5)
    for t in range(tokens):
        row, routed = np.empty(hidden), np.empty(hidden)
        for h in range(hidden):
            routed[h] = sum(float(slots[t, s, h]) * float(routing[t, s]) for s in range(top_k))
            row[h] = float(residual[t, h]) + routed[h] + float(shared[t, h]) / (1.0 + np.exp(-float(gate[t, 0])))
        # two bf16 roundings on the way: half a step of the routed sum, then half a step of the result
        assert np.all(np.abs(got_r[t] - row) <= (np.abs(routed) + np.abs(row)) * 2.0 ** -8 + 1e-6)
        norm = got_r[t].astype(np.float64) / np.sqrt(np.mean(got_r[t].astype(np.float64) ** 2) + 1e-5) * weight
        assert np.all(np.abs(got_n[t] - norm) <= np.abs(norm) * 2.0 ** -8 + 1e-6)
    # the aggregate form on the separately formed sum, and the gathered form on a permutation of the rows
    agg = np.zeros((tokens, hidden), np.float32)
    for s in range(top_k):
        agg = (agg + (slots[:, s] * routing[:, s, None]).astype(np.float32)).astype(np.float32)
    r2, n2 = O.moe_tail_next_rmsnorm(bf(agg), shared, gate, residual, weight, eps=1e-5)
    assert np.array_equal(r2, got_r) and np.array_equal(n2, got_n)
    perm = rng.permutation(tokens * top_k)
    compact = np.empty((tokens * top_k, hidden), np.float32)
    compact[perm] = slots.reshape(-1, hidden)
    r3, n3 = O.moe_tail_next_rmsnorm(compact, shared, gate, residual, weight, routing_weights=routing,
                                     lane_to_compact=perm, eps=1e-5)
    assert np.array_equal(r3, got_r) and np.array_equal(n3, got_n)
    dropped = perm.copy().reshape(tokens, top_k)
    dropped[1, 2] = -1
    r4, _ = O.moe_tail_next_rmsnorm(compact, shared, gate, residual, weight, routing_weights=routing,
                                    lane_to_compact=dropped, eps=1e-5)
    routing0 = routing.copy()
    routing0[1, 2] = 0.0
    r5, _ = O.moe_tail_next_rmsnorm(slots, shared, gate, residual, weight, routing_weights=routing0, eps=1e-5)
    assert np.array_equal(r4, r5)


def test_quantize_q8_1x2_planes():
    """Plane 0 is the plain quantizer; plane 1 quantizes what plane 0 leaves, so the two planes together are within
    half a step of the second scale (|residual| <= d0/2 + fp16 rounding of d0, so d1 <= amax/127 * 0.52 / 127); a block
    that plane 0 represents exactly leaves a zero plane."""
    rng = np.random.default_rng(12)
    x = O.bf16_bits_to_f32(O.f32_to_bf16_bits((rng.standard_normal((5, 256)) * 3.0).astype(np.float32)))
    x[1, 32:64] = np.arange(-16, 16) * 0.25
    x[1, 63] = 127 * 0.25                       # d = 0.25 exactly: q = x / 0.25, nothing left
    planes = O.quantize_q8_1x2(x)
    assert planes.shape == (2, 5, 8, 36) and np.array_equal(planes[0], O.quantize_q8_1(x))
    d0, _, q0 = O.q8_1_fields(planes[0])
    d1, s1, q1 = O.q8_1_fields(planes[1])
    recon = d0[..., None].astype(np.float64) * q0 + d1[..., None].astype(np.float64) * q1
    amax = np.abs(x.reshape(5, 8, 32)).max(axis=-1, keepdims=True)
    assert np.all(np.abs(recon - x.reshape(5, 8, 32)) <= amax * 2.0 ** -13 + 1e-12)
    assert np.all(q1[1, 1] == 0) and d1[1, 1] == 0 and s1[1, 1] == 0
