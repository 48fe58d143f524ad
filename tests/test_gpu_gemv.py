"""GPU parity of the q8_1 decode GEMV (Q4_K / Q6_K / Q8_0) through the C ABI.

Parity definition (the reference CPU backend has no q8_1 path, so it is
extended the way the reference's own q8_1 tests do,
tests/test_gpu_gguf_k_mmq_prefill.py:534-540):
  1. q8_1 activation bytes: identical to the oracle's;
  2. unpacked weights / dequantized float32: identical bit patterns;
  3. int32 sub-block dots: identical;
  4. float32 outputs: max relative error <= 1e-3 (floor 1e-3*max|ref|) and
     cosine >= 0.99999 against the reference CPU GEMV (dequantize -> float32
     matmul) applied to the q8_1-dequantized activations;
  5. bf16 output == bf16_round(float32 output) bit for bit;
  6. reported, with a loose floor as in the reference: KL / top-1 of
     softmax(out) against the unquantized-activation reference.
"""

from __future__ import annotations

import numpy as np
import pytest

from oracle import c_oracle as C
from oracle import gguf_oracle as O
from hipengine_amd.kernels.hip_gfx950.quant import gguf_q8_1_gemv as G
from hipengine_amd.kernels.hip_gfx950.quant import gguf_quantize as Q
from hipengine_amd.kernels.hip_gfx950.quant import gguf_verify as V

pytestmark = pytest.mark.gpu

REL_TOL = 1e-3
COS_MIN = 0.99999
QT = {"gguf_q4_k": O.GGML_Q4_K, "gguf_q6_k": O.GGML_Q6_K, "gguf_q8_0": O.GGML_Q8_0}
SHORT = {"gguf_q4_k": "q4_k", "gguf_q6_k": "q6_k", "gguf_q8_0": "q8_0"}
CLOSED = {"gguf_q4_k": O.closed_form_q4_k, "gguf_q6_k": O.closed_form_q6_k, "gguf_q8_0": O.closed_form_q8_0}


def _check_f32(got, xq, w, qt, x_unq=None):
    ref = O.gguf_quant_gemv(O.dequantize_q8_1(xq), w, qt)
    err, cos = O.max_rel_err(got, ref), O.cosine(got, ref)
    assert err <= REL_TOL, f"max rel err {err}"
    assert cos >= COS_MIN, f"cosine {cos}"
    if x_unq is not None and got.shape[1] >= 16:
        kl, top1 = O.softmax_kl_top1(O.gguf_quant_gemv(x_unq, w, qt), got)
        assert kl <= 0.05 and top1 >= 0.75, (kl, top1)   # outer floor only; parity is the gate above


def _run_fused(dev, quant, x, w, act="f32", out="f32"):
    rows, k = x.shape
    n = w.shape[0]
    xin = x if act == "f32" else O.f32_to_bf16_bits(x)
    dx, dw = dev.put(xin), dev.put(w)
    dout = dev.empty(rows * n * (4 if out == "f32" else 2))
    G.FUSED[(SHORT[quant], act, out)](dx.ptr, dw.ptr, dout.ptr, rows, k, n)
    res = dev.get(dout, np.float32 if out == "f32" else np.uint16, (rows, n))
    dev.free(dx, dw, dout)
    return res


def _random_q5_k(n, k, seed):
    rng = np.random.default_rng(seed)
    nblk = n * (k // 256)
    blk = O.pack_q5_k_blocks(rng.integers(0, 32, size=(nblk, 8, 32), dtype=np.uint8),
                             rng.integers(0, 64, size=(nblk, 8), dtype=np.uint8),
                             rng.integers(0, 64, size=(nblk, 8), dtype=np.uint8),
                             (rng.random(nblk) * 0.05).astype(np.float32), (rng.random(nblk) * 0.02).astype(np.float32))
    return blk.reshape(n, -1)


@pytest.mark.parametrize("quant", ["gguf_q4_k", "gguf_q5_k", "gguf_q6_k", "gguf_q8_0"])
def test_dequantize_bit_exact(dev, quant):
    qt = {"gguf_q5_k": O.GGML_Q5_K, **QT}[quant]
    cases = ((O.closed_form_q5_k(37, 768), _random_q5_k(64, 1024, 11)) if quant == "gguf_q5_k"
             else (CLOSED[quant](37, 768), O.random_weight(qt, 64, 1024, seed=11)))
    for w in cases:
        block, nbytes = {8: (32, 34), 12: (256, 144), 13: (256, 176), 14: (256, 210)}[qt]
        n_blocks = w.size // nbytes
        dw = dev.put(w)
        dout = dev.empty(n_blocks * block * 4)
        V.gguf_dequantize_f32(quant, dw.ptr, dout.ptr, n_blocks)
        got = dev.get(dout, np.float32, (w.shape[0], w.shape[1] // nbytes * block))
        dev.free(dw, dout)
        want = O.dequantize(w, qt)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("quant", ["gguf_q4_k", "gguf_q5_k", "gguf_q6_k", "gguf_q8_0"])
def test_embedding_lookup_bit_exact(dev, quant):
    """bf16(dequantize(row token)) bit for bit; rows with an out-of-range token id stay untouched."""
    from hipengine_amd.kernels.hip_gfx950.quant import gguf_embedding as E
    qt = {"gguf_q5_k": O.GGML_Q5_K, **QT}[quant]
    vocab, hidden = 301, 1280
    w = _random_q5_k(vocab, hidden, 3) if quant == "gguf_q5_k" else O.random_weight(qt, vocab, hidden, seed=4)
    ids = np.array([0, 300, 17, 17, -1, 301, 128, 5], dtype=np.int64)
    did, dw = dev.put(ids), dev.put(w)
    dout = dev.empty(ids.size * hidden * 2, fill=0xAB)
    E.EMBEDDING[quant](did.ptr, dw.ptr, dout.ptr, ids.size, hidden, vocab)
    got = dev.get(dout, np.uint16, (ids.size, hidden))
    dev.free(did, dw, dout)
    ok = (ids >= 0) & (ids < vocab)
    want = O.f32_to_bf16_bits(O.embedding_lookup(ids[ok], w, qt))
    assert np.array_equal(got[ok], want)
    assert np.all(got[~ok] == 0xABAB)


@pytest.mark.parametrize("kind", ["f32", "bf16"])
def test_quantize_q8_1_bytes(dev, kind):
    rng = np.random.default_rng(5)
    x = rng.standard_normal((5, 1024)).astype(np.float32)
    x[1, 32:64] = 0.0                       # a zero block
    x[2, :32] = np.arange(-16, 16) / 8.0    # exact binary fractions
    x[2, 31] = 127.0 / 8.0                  # amax such that x/d hits .5 ties
    x[3] *= 1e-6
    x[4] *= 3e4
    xin = x if kind == "f32" else O.f32_to_bf16_bits(x)
    xf = x if kind == "f32" else O.bf16_bits_to_f32(xin)
    want = O.quantize_q8_1(xf)
    dx = dev.put(xin)
    dq = dev.empty(want.size)
    (Q.gguf_q4_k_quantize_f32_q8_1 if kind == "f32" else Q.gguf_q4_k_quantize_bf16_q8_1)(dx.ptr, dq.ptr, 5, 1024)
    got = dev.get(dq, np.uint8, want.shape)
    dev.free(dx, dq)
    assert np.array_equal(got, want)
    assert np.array_equal(got, C.quantize_q8_1(xin, bf16=(kind == "bf16")))


@pytest.mark.parametrize("quant", ["gguf_q4_k", "gguf_q6_k", "gguf_q8_0"])
def test_block_dots_bit_exact(dev, quant):
    qt = QT[quant]
    rng = np.random.default_rng(7)
    rows, k, n = 3, 1024, 40
    x = rng.standard_normal((rows, k)).astype(np.float32)
    xq = O.quantize_q8_1(x)
    w = O.random_weight(qt, n, k, seed=3)
    per = 16 if qt == O.GGML_Q6_K else 32
    dxq, dw = dev.put(xq), dev.put(w)
    ddots = dev.empty(rows * n * (k // per) * 4)
    dqs = dev.empty(rows * (k // 32) * 4)
    V.gguf_q8_1_block_dots_i32(quant, dxq.ptr, dw.ptr, ddots.ptr, dqs.ptr, rows, k, n)
    dots = dev.get(ddots, np.int32, (rows, n, k // per))
    qs = dev.get(dqs, np.int32, (rows, k // 32))
    dev.free(dxq, dw, ddots, dqs)
    ref = C.block_dots(xq, w, qt)
    if qt == O.GGML_Q4_K:
        assert np.array_equal(dots, ref[0]) and np.array_equal(qs, ref[1])
    else:
        assert np.array_equal(dots, ref)
    assert np.array_equal(qs, O.q8_1_fields(xq)[2].astype(np.int32).sum(axis=-1))


@pytest.mark.parametrize("quant", ["gguf_q4_k", "gguf_q6_k", "gguf_q8_0"])
@pytest.mark.parametrize("rows", [1, 2, 3, 4, 8])
def test_fused_gemv_closed_form_weights(dev, quant, rows):
    """The reference's closed-form weights and its `(arange % 13 - 6) / 8` activations
    (tests/test_gpu_gguf_q4_k_gemv.py:102-112)."""
    k, n = 512, 37
    x = ((np.arange(rows * k, dtype=np.float32).reshape(rows, k) % 13) - 6) / 8.0
    w = CLOSED[quant](n, k)
    got = _run_fused(dev, quant, x, w)
    _check_f32(got, O.quantize_q8_1(x), w, QT[quant])


@pytest.mark.parametrize("quant,k,n", [
    ("gguf_q4_k", 5120, 1024), ("gguf_q4_k", 2048, 512), ("gguf_q4_k", 512, 2048), ("gguf_q4_k", 256, 16),
    ("gguf_q4_k", 1536, 50), ("gguf_q4_k", 6144, 30), ("gguf_q4_k", 4096, 70),
    ("gguf_q6_k", 5120, 1000), ("gguf_q6_k", 17408, 160), ("gguf_q6_k", 2048, 45), ("gguf_q6_k", 512, 77),
    ("gguf_q8_0", 5120, 640), ("gguf_q8_0", 768, 33), ("gguf_q8_0", 2048, 100), ("gguf_q8_0", 512, 41),
])
@pytest.mark.parametrize("rows", [1, 2, 5, 8])
def test_fused_gemv_random_weights(dev, quant, k, n, rows):
    rng = np.random.default_rng(1000 + k + n + rows)
    x = rng.standard_normal((rows, k)).astype(np.float32)
    w = O.random_weight(QT[quant], n, k, seed=k + n)
    got = _run_fused(dev, quant, x, w)
    _check_f32(got, O.quantize_q8_1(x), w, QT[quant], x_unq=x)


@pytest.mark.parametrize("quant", ["gguf_q4_k", "gguf_q6_k", "gguf_q8_0"])
def test_fused_gemv_bf16_in_out(dev, quant):
    rng = np.random.default_rng(21)
    rows, k, n = 2, 1024, 96
    x = rng.standard_normal((rows, k)).astype(np.float32)
    xb = O.f32_to_bf16_bits(x)
    w = O.random_weight(QT[quant], n, k, seed=9)
    f32 = _run_fused(dev, quant, x, w, act="bf16", out="f32")
    _check_f32(f32, O.quantize_q8_1(O.bf16_bits_to_f32(xb)), w, QT[quant])
    b16 = _run_fused(dev, quant, x, w, act="bf16", out="bf16")
    assert np.array_equal(b16, O.f32_to_bf16_bits(f32))


@pytest.mark.parametrize("quant,fn", [
    ("gguf_q4_k", "gguf_q4_k_q8_1_dp4a_vdr_bf16_f32_out"),
    ("gguf_q6_k", "gguf_q6_k_q8_1_dp4a_gemv_bf16_f32_out"),
    ("gguf_q8_0", "gguf_q8_0_dp4a_gemv_f32_f32_out"),
])
def test_prequantized_gemv_matches_fused_bit_for_bit(dev, quant, fn):
    """Sibling variants must agree exactly: same integer dots, same float32 order."""
    rng = np.random.default_rng(33)
    rows, k, n = 4, 2048, 80
    x = rng.standard_normal((rows, k)).astype(np.float32)
    x[1, 64:96] *= np.float32(1e-36)         # scale in the denormal range
    x[2, :32] = np.arange(-16, 16) / 8.0     # exact .5 ties
    x[2, 31] = 127.0 / 8.0
    x[3, 128:160] *= np.float32(3e4)
    w = O.random_weight(QT[quant], n, k, seed=4)
    fused = _run_fused(dev, quant, x, w)
    xq = O.quantize_q8_1(x)
    dxq, dw = dev.put(xq), dev.put(w)
    dout = dev.empty(rows * n * 4)
    getattr(G, fn)(dxq.ptr, dw.ptr, dout.ptr, rows, k, n)
    pre = dev.get(dout, np.float32, (rows, n))
    dev.free(dxq, dw, dout)
    assert np.array_equal(pre.view(np.uint32), fused.view(np.uint32))
    _check_f32(pre, xq, w, QT[quant])


@pytest.mark.parametrize("rows,k,sizes,suffix", [
    (1, 5120, (1024, 256, 512), "f32_f32_out"),      # one launch shared among the matrices
    (2, 4096, (768, 130), "bf16_bf16_out"),          # ragged second matrix
    (1, 1024, (48, 80, 16), "bf16_bf16_out"),        # too small to share a launch: one launch per matrix
    (6, 2048, (96, 40, 72), "f32_f32_out"),          # more than two activation rows
    (11, 1024, (64, 33), "f32_f32_out"),             # more than eight
])
def test_q8_0_dp4a_family_takes_hipengine_argument_lists(dev, rows, k, sizes, suffix):
    """gguf_q8_0_dp4a_{,rowtile4_,dual_split_rowtile4_,triple_split_rowtile4_}gemv_*: the argument lists of
    hipEngine's exports (a `threads` slot before the stream; one output buffer and row count per matrix).  Every
    output equals the single-matrix call's bit for bit and the oracle's q8_1 x Q8_0 GEMV within float32 noise."""
    rng = np.random.default_rng(1234 + rows)
    x = rng.standard_normal((rows, k)).astype(np.float32)
    xq = O.quantize_q8_1(x)
    ws = [O.random_weight(O.GGML_Q8_0, n, k, seed=50 + i) for i, n in enumerate(sizes)]
    bf16 = suffix.startswith("bf16")
    width, dtype = (2, np.uint16) if bf16 else (4, np.float32)
    dxq = dev.put(xq)
    dws = [dev.put(w) for w in ws]

    def run(name, weights, ns):
        outs = [dev.empty(rows * n * width) for n in ns]
        getattr(G, name)(dxq.ptr, *[w.ptr for w in weights], *[o.ptr for o in outs], rows, k, *ns)
        got = [dev.get(o, dtype, (rows, n)) for o, n in zip(outs, ns)]
        dev.free(*outs)
        return got

    single = [run(f"gguf_q8_0_dp4a_gemv_{suffix}", [dw], [n])[0] for dw, n in zip(dws, sizes)]
    tiled = [run(f"gguf_q8_0_dp4a_rowtile4_gemv_{suffix}", [dw], [n])[0] for dw, n in zip(dws, sizes)]
    shape = {2: "dual", 3: "triple"}[len(sizes)]
    split = run(f"gguf_q8_0_dp4a_{shape}_split_rowtile4_gemv_{suffix}", dws, list(sizes))
    dev.free(dxq, *dws)
    for one, four, many, w in zip(single, tiled, split, ws):
        assert np.array_equal(one, four)
        assert np.array_equal(one, many)
        ref = O.gemv_q8_1_q8_0(xq, w).astype(np.float32)
        if bf16:      # the bf16 output is the float32 result rounded to nearest even
            assert O.max_rel_err(O.bf16_bits_to_f32(one), ref) <= 2.0 ** -8
        else:
            assert O.max_rel_err(one, ref) <= REL_TOL
            assert O.cosine(one, ref) >= COS_MIN


def test_more_than_eight_rows_and_determinism(dev):
    rng = np.random.default_rng(44)
    rows, k, n = 19, 1024, 48
    x = rng.standard_normal((rows, k)).astype(np.float32)
    w = O.random_weight(O.GGML_Q4_K, n, k, seed=2)
    a = _run_fused(dev, "gguf_q4_k", x, w)
    b = _run_fused(dev, "gguf_q4_k", x, w)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    _check_f32(a, O.quantize_q8_1(x), w, O.GGML_Q4_K)
    # row invariance inside one kernel family: a row computed alone equals the same
    # row of a 2-row batch bit for bit (both take the whole-row "run" kernel) ...
    one = _run_fused(dev, "gguf_q4_k", x[7:8], w)
    two = _run_fused(dev, "gguf_q4_k", x[6:8], w)
    assert np.array_equal(one.view(np.uint32), two[1:2].view(np.uint32))
    # ... and within float32 summation-order noise of the 8-row kernel's result
    assert O.max_rel_err(one, a[7:8]) <= 1e-4


@pytest.mark.parametrize("rows,k,n,rpw,kind", [(1, 5120, 300, 0, "f32"), (8, 5120, 1000, 68, "f32"),
                                               (4, 2048, 257, 33, "bf16"), (2, 4096, 96, 96, "fp16"),
                                               (5, 4352, 64, 7, "f32"), (8, 1024, 40, 0, "bf16"),
                                               (3, 6144, 130, 65, "f32")])
def test_slab_form_q4_k(dev, rows, k, n, rpw, kind):
    """The slab form of the fused Q4_K GEMV: K split over the waves of a workgroup (one or two blocks per wave,
    odd block counts included), slabs of up to three 32-row steps with ragged last steps and a ragged last slab."""
    rng = np.random.default_rng(91 + rows + k)
    x = rng.standard_normal((rows, k)).astype(np.float32)
    x[0, :32] = 0.0
    if kind != "f32":
        x = O.bf16_bits_to_f32(O.f32_to_bf16_bits(x)) if kind == "bf16" else x.astype(np.float16).astype(np.float32)
    w = O.random_weight(O.GGML_Q4_K, n, k, seed=k + n)
    xin = x if kind == "f32" else (O.f32_to_bf16_bits(x) if kind == "bf16" else x.astype(np.float16))
    dx, dw = dev.put(xin), dev.put(w)
    dout = dev.empty(rows * n * 4)
    G.gguf_q4_k_q8_1_fused_gemv_slab_tuned(dx.ptr, kind, dw.ptr, dout.ptr, "f32", rows, k, n, rows_per_workgroup=rpw)
    got = dev.get(dout, np.float32, (rows, n))
    dev.free(dx, dw, dout)
    _check_f32(got, O.quantize_q8_1(x), w, O.GGML_Q4_K)


@pytest.mark.parametrize("quant,rows,k,n,waves,bpw,wgs,kind", [
    ("gguf_q6_k", 8, 5120, 300, 0, 0, 0, "f32"),      # planner: one phase, 10 waves x 2 blocks, 1-2 rows per workgroup
    ("gguf_q6_k", 8, 17408, 200, 0, 0, 0, "f32"),     # planner: phased (activations re-quantized per phase)
    ("gguf_q6_k", 4, 2048, 257, 8, 1, 3, "bf16"),     # three 32-row steps with a ragged last one
    ("gguf_q6_k", 5, 4096, 700, 6, 1, 8, "f32"),      # three phases, 87-88 rows per workgroup
    ("gguf_q6_k", 3, 3072, 130, 6, 2, 1, "fp16"),     # one workgroup, two row groups (96 + 34)
    ("gguf_q6_k", 8, 8192, 64, 8, 4, 2, "f32"),       # four blocks per wave
    ("gguf_q6_k", 8, 10240, 100, 10, 2, 0, "q8_1"),   # two phases of two blocks per wave, pre-quantized activations
    ("gguf_q6_k", 4, 5632, 50, 8, 1, 0, "f32"),       # last phase: two waves without a block
    ("gguf_q4_k", 8, 17408, 200, 0, 0, 0, "f32"),     # Q4_K rows too long for the slab form: phased
    ("gguf_q4_k", 4, 5120, 131, 0, 0, 2, "bf16"),     # one phase, 65-66 rows per workgroup
    ("gguf_q4_k", 5, 8192, 97, 8, 2, 0, "q8_1"),      # two phases of two blocks
    ("gguf_q8_0", 8, 5120, 300, 0, 0, 0, "f32"),
    ("gguf_q8_0", 4, 4096, 100, 0, 0, 0, "bf16"),
    ("gguf_q8_0", 6, 17408, 97, 0, 0, 0, "f32"),
    ("gguf_q8_0", 3, 2048, 200, 8, 1, 2, "q8_1"),
])
def test_pslab_form(dev, quant, rows, k, n, waves, bpw, wgs, kind):
    """The phased slab form (Q6_K / Q8_0 on the int8 MFMA): planner layouts and explicit ones - one and several
    phases, 1/2/4 blocks per wave, several row groups per workgroup, ragged steps, the last row of the tensor."""
    rng = np.random.default_rng(17 + rows + k + n)
    x = rng.standard_normal((rows, k)).astype(np.float32)
    x[0, :32] = 0.0
    if kind == "bf16":
        x = O.bf16_bits_to_f32(O.f32_to_bf16_bits(x))
    elif kind == "fp16":
        x = x.astype(np.float16).astype(np.float32)
    w = O.random_weight(QT[quant], n, k, seed=k + n)
    xq = O.quantize_q8_1(x)
    xin = {"f32": x, "bf16": O.f32_to_bf16_bits(x), "fp16": x.astype(np.float16), "q8_1": xq}[kind]
    dx, dw = dev.put(xin), dev.put(w)
    dout = dev.empty(rows * n * 4)
    G.gguf_q8_1_fused_gemv_pslab_tuned(quant, dx.ptr, kind, dw.ptr, dout.ptr, "f32", rows, k, n, waves=waves,
                                       blocks_per_wave=bpw, workgroups=wgs)
    got = dev.get(dout, np.float32, (rows, n))
    dev.free(dx, dw, dout)
    _check_f32(got, xq, w, QT[quant])
    # against the float64 evaluation of the kernel's own formula, which isolates float32 summation order
    exact = {"gguf_q4_k": O.gemv_q8_1_q4_k, "gguf_q6_k": O.gemv_q8_1_q6_k, "gguf_q8_0": O.gemv_q8_1_q8_0}[quant](xq, w)
    assert O.max_rel_err(got, exact) <= 1e-4


@pytest.mark.parametrize("rows,k,n,waves,bpw,wgs", [(8, 5120, 300, 0, 0, 0), (4, 17408, 100, 0, 0, 0), (5, 2048, 130, 8, 1, 1)])
def test_pslab_form_q5_k(dev, rows, k, n, waves, bpw, wgs):
    """Q5_K in the phased slab form (one phase, several phases, two row groups); the default dispatch takes the same
    form from batch 3 and must give the same bits."""
    rng = np.random.default_rng(23 + rows + k)
    x = rng.standard_normal((rows, k)).astype(np.float32)
    w = _random_q5_k(n, k, seed=k + n)
    xq = O.quantize_q8_1(x)
    dx, dw = dev.put(x), dev.put(w)
    dout, ddef = dev.empty(rows * n * 4), dev.empty(rows * n * 4)
    G.gguf_q8_1_fused_gemv_pslab_tuned("gguf_q5_k", dx.ptr, "f32", dw.ptr, dout.ptr, "f32", rows, k, n, waves=waves,
                                       blocks_per_wave=bpw, workgroups=wgs)
    G.FUSED[("q5_k", "f32", "f32")](dx.ptr, dw.ptr, ddef.ptr, rows, k, n)
    got = dev.get(dout, np.float32, (rows, n))
    default = dev.get(ddef, np.float32, (rows, n))
    dev.free(dx, dw, dout, ddef)
    _check_f32(got, xq, w, O.GGML_Q5_K)
    if waves == 0:
        assert np.array_equal(got.view(np.uint32), default.view(np.uint32))
    else:
        _check_f32(default, xq, w, O.GGML_Q5_K)


@pytest.mark.parametrize("quant,d,waves,waves_total,n", [("gguf_q4_k", 2, 4, 64, 256), ("gguf_q4_k", 2, 10, 120, 256),
                                                        ("gguf_q6_k", 2, 12, 96, 256), ("gguf_q8_0", 2, 8, 64, 256),
                                                        ("gguf_q4_k", 2, 12, 96, 1021), ("gguf_q5_k", 2, 5, 35, 333),
                                                        ("gguf_q6_k", 2, 7, 7 * 64, 255)])
def test_stream_form_explicit_layouts(dev, quant, d, waves, waves_total, n):
    """Stream form with explicit wave and workgroup counts (up to 12 waves per workgroup at batch 1, ring depth 2),
    also with row counts that leave the last chunk of 4 rows partial and the workgroups with unequal chunk counts.
    With 4 waves the two activation groups per thread fetched up front do not cover K = 5120, so the launch takes
    the kernel that loops over the rest; with 10 or 12 they do and it takes the one without that loop."""
    rng = np.random.default_rng(5 + waves_total)
    rows, k = 1, 5120
    x = rng.standard_normal((rows, k)).astype(np.float32)
    qt = O.GGML_Q5_K if quant == "gguf_q5_k" else QT[quant]
    w = _random_q5_k(n, k, seed=3) if quant == "gguf_q5_k" else O.random_weight(qt, n, k, seed=3)
    dx, dw = dev.put(x), dev.put(w)
    dout = dev.empty(rows * n * 4)
    G.gguf_q8_1_fused_gemv_stream_tuned(quant, dx.ptr, "f32", dw.ptr, dout.ptr, "f32", rows, k, n, loads_in_flight=d,
                                        waves=waves, waves_total=waves_total)
    got = dev.get(dout, np.float32, (rows, n))
    dev.free(dx, dw, dout)
    _check_f32(got, O.quantize_q8_1(x), w, qt)


def test_output_canaries_untouched(dev):
    rng = np.random.default_rng(55)
    rows, k, n = 3, 512, 21
    x = rng.standard_normal((rows, k)).astype(np.float32)
    w = O.random_weight(O.GGML_Q4_K, n, k, seed=6)
    dx, dw = dev.put(x), dev.put(w)
    pad = 64
    dout = dev.empty((rows * n + 2 * pad) * 4, fill=0x5A)
    G.FUSED[("q4_k", "f32", "f32")](dx.ptr, dw.ptr, dout.ptr + pad * 4, rows, k, n)
    raw = dev.get(dout, np.uint32, (rows * n + 2 * pad,))
    dev.free(dx, dw, dout)
    assert np.all(raw[:pad] == 0x5A5A5A5A) and np.all(raw[-pad:] == 0x5A5A5A5A)


def test_c_abi_rejects_bad_arguments(dev):
    import ctypes
    lib = dev.library
    f = lib.hipengine_gguf_q4_k_q8_1_fused_gemv_f32_f32_out
    f.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p] + [ctypes.c_int64] * 4 + [ctypes.c_void_p]
    f.restype = ctypes.c_int
    buf = dev.empty(4096)
    assert f(None, buf.ptr, buf.ptr, 1, 256, 1, 128, None) == 1
    assert f(buf.ptr, buf.ptr, buf.ptr, 1, 255, 1, 128, None) == 1
    assert f(buf.ptr, buf.ptr, buf.ptr, 0, 256, 1, 128, None) == 1
    dev.free(buf)
    with pytest.raises(ValueError, match="divisible"):
        G.FUSED[("q4_k", "f32", "f32")](1, 1, 1, 1, 100, 8)
    with pytest.raises(ValueError, match="threads"):
        G.FUSED[("q4_k", "f32", "f32")](1, 1, 1, 1, 256, 8, threads=96)


@pytest.mark.parametrize("rows,kind,round_mid", [(1, "bf16", True), (2, "bf16", True), (1, "f32", False)])
def test_pair_silu_gemv(dev, rows, kind, round_mid):
    """Gate/up pair with SiLU fused (stream form, both matrices in one pass) against the unfused composition of
    the oracle's GEMV and SiLU*up on the same q8_1 activations; bf16 intermediates rounded as the unfused
    sequence stores them."""
    k, n = 4096, 4096
    rng = np.random.default_rng(5 + rows)
    x = rng.standard_normal((rows, k)).astype(np.float32)
    if kind == "bf16":
        x = O.bf16_bits_to_f32(O.f32_to_bf16_bits(x))
    wg = O.random_weight(O.GGML_Q4_K, n, k, seed=11)
    wu = O.random_weight(O.GGML_Q4_K, n, k, seed=12)
    xin = x if kind == "f32" else O.f32_to_bf16_bits(x)
    dx, dg, du = dev.put(xin), dev.put(wg), dev.put(wu)
    esz = 4 if kind == "f32" else 2
    dout = dev.empty(rows * n * esz)
    G.gguf_pair_silu_gemv("gguf_q4_k", dx.ptr, kind, dg.ptr, du.ptr, dout.ptr, kind, rows, k, n, round_mid=round_mid)
    got = dev.get(dout, np.float32 if kind == "f32" else np.uint16, (rows, n))
    dev.free(dx, dg, du, dout)
    xdq = O.dequantize_q8_1(O.quantize_q8_1(x))
    gate = O.gguf_quant_gemv(xdq, wg, O.GGML_Q4_K)
    up = O.gguf_quant_gemv(xdq, wu, O.GGML_Q4_K)
    if round_mid and kind == "bf16":
        gate = O.bf16_bits_to_f32(O.f32_to_bf16_bits(gate))
        up = O.bf16_bits_to_f32(O.f32_to_bf16_bits(up))
    want = (O.silu(gate) * up).astype(np.float32)
    if kind == "bf16":
        got = O.bf16_bits_to_f32(got)
        # one bf16 ulp of slack on top of the float32 gate: a gate or up value within float32 noise of a bf16
        # rounding boundary may round the other way
        assert O.cosine(got, want) >= 0.9999
        assert np.max(np.abs(got - want)) <= 2.0 ** -6 * max(1.0, float(np.max(np.abs(want))))
    else:
        assert O.max_rel_err(got, want) <= 1e-3 and O.cosine(got, want) >= 0.99999


@pytest.mark.parametrize("quant,rows,k,n,kind,round_mid", [
    ("gguf_q4_k", 8, 5120, 600, "bf16", True),      # slab form, gate and up in one launch
    ("gguf_q4_k", 4, 5120, 300, "f32", False),
    ("gguf_q6_k", 5, 5120, 300, "bf16", True),      # phased slab, one phase
    ("gguf_q4_k", 8, 17408, 200, "f32", False),     # phased slab, several phases
])
def test_pair_silu_gemv_batch_3_to_8(dev, quant, rows, k, n, kind, round_mid):
    """Gate/up pair at batch 3..8 on the MFMA forms (one launch on the Q4_K slab form, gate launch then up launch
    elsewhere): out = silu(round(gate)) * round(up), against the unfused kernels' own gate and up outputs."""
    rng = np.random.default_rng(15 + rows + n)
    x = rng.standard_normal((rows, k)).astype(np.float32)
    if kind == "bf16":
        x = O.bf16_bits_to_f32(O.f32_to_bf16_bits(x))
    wg = O.random_weight(QT[quant], n, k, seed=21)
    wu = O.random_weight(QT[quant], n, k, seed=22)
    xin = x if kind == "f32" else O.f32_to_bf16_bits(x)
    dx, dg, du = dev.put(xin), dev.put(wg), dev.put(wu)
    esz = 4 if kind == "f32" else 2
    dout, dgate, dup = dev.empty(rows * n * esz), dev.empty(rows * n * esz), dev.empty(rows * n * esz)
    G.gguf_pair_silu_gemv(quant, dx.ptr, kind, dg.ptr, du.ptr, dout.ptr, kind, rows, k, n, round_mid=round_mid)
    G.FUSED[(quant[5:], kind, kind)](dx.ptr, dg.ptr, dgate.ptr, rows, k, n)
    G.FUSED[(quant[5:], kind, kind)](dx.ptr, du.ptr, dup.ptr, rows, k, n)
    dt = np.float32 if kind == "f32" else np.uint16
    got, gate, up = (dev.get(b, dt, (rows, n)) for b in (dout, dgate, dup))
    dev.free(dx, dg, du, dout, dgate, dup)
    if kind == "bf16":
        got, gate, up = (O.bf16_bits_to_f32(a) for a in (got, gate, up))
    want = (O.silu(gate) * up).astype(np.float32)
    # the device's expf and the final rounding to the output type are the only differences
    tol = 2.0 ** -7 if kind == "bf16" else 1e-5
    assert np.max(np.abs(got - want)) <= tol * max(1.0, float(np.max(np.abs(want))))
    assert O.cosine(got, want) >= 0.99999
    if kind != "f32":
        with pytest.raises(G.FusedFormUnavailable):
            G.gguf_pair_silu_gemv(quant, 16, kind, 16, 16, 16, kind, rows, k, n, round_mid=False)


@pytest.mark.parametrize("rows,k,n,kind", [
    (8, 5120, 17408, "f32"),      # 68 rows per workgroup and matrix: two full steps and an early 4-row step, twice
    (3, 2048, 10240, "bf16"),     # one block per wave; 40 rows: a full step and a step of 8
    (5, 5120, 8960, "f32"),       # 35 rows: one full step, an early step of 3
    (8, 4096, 18432, "bf16"),     # 72 rows: the most a pair launch takes
    (4, 5120, 18500, "f32"),      # 73 rows: past it, gate launch then up launch
    (6, 5120, 700, "bf16"),       # ragged last workgroup
])
def test_pair_silu_gemv_slab_one_launch(dev, rows, k, n, kind):
    """The Q4_K gate/up pair at batch 3..8 as ONE slab launch (a workgroup walks its rows of the gate matrix, then
    the same rows of the up matrix): out = silu(round(gate)) * round(up) against the single-matrix launches' own
    gate and up outputs, over the step shapes of the slab (full steps, early short steps, ragged ends)."""
    from hipengine_amd.synthetic import synthetic_blocks

    rng = np.random.default_rng(rows * 1000 + n)
    x = (rng.standard_normal((rows, k)) * 0.5).astype(np.float32)
    wg = synthetic_blocks(O.GGML_Q4_K, n, k, seed=31)
    wu = synthetic_blocks(O.GGML_Q4_K, n, k, seed=32)
    xin = x if kind == "f32" else O.f32_to_bf16_bits(x)
    dx, dg, du = dev.put(xin), dev.put(wg), dev.put(wu)
    esz = 4 if kind == "f32" else 2
    dout, dgate, dup = dev.empty(rows * n * esz, fill=0x7B), dev.empty(rows * n * esz), dev.empty(rows * n * esz)
    G.gguf_pair_silu_gemv("gguf_q4_k", dx.ptr, kind, dg.ptr, du.ptr, dout.ptr, kind, rows, k, n, round_mid=True)
    G.FUSED[("q4_k", kind, kind)](dx.ptr, dg.ptr, dgate.ptr, rows, k, n)
    G.FUSED[("q4_k", kind, kind)](dx.ptr, du.ptr, dup.ptr, rows, k, n)
    dt = np.float32 if kind == "f32" else np.uint16
    got, gate, up = (dev.get(b, dt, (rows, n)) for b in (dout, dgate, dup))
    dev.free(dx, dg, du, dout, dgate, dup)
    if kind == "bf16":
        got, gate, up = (O.bf16_bits_to_f32(a) for a in (got, gate, up))
    want = (O.silu(gate) * up).astype(np.float32)
    assert np.all(np.isfinite(got))
    # the device's expf and the final rounding to the output type are the only differences
    tol = 2.0 ** -7 if kind == "bf16" else 1e-5
    assert np.max(np.abs(got - want)) <= tol * max(1.0, float(np.max(np.abs(want))))
    assert O.cosine(got, want) >= 0.99999


@pytest.mark.parametrize("quant,rows,k,n,kind", [("gguf_q6_k", 1, 17408, 5120, "bf16"), ("gguf_q4_k", 2, 4096, 4096, "bf16"),
                                                 ("gguf_q4_k", 5, 5120, 1000, "bf16"), ("gguf_q4_k", 1, 5120, 17408, "f32"),
                                                 ("gguf_q6_k", 8, 17408, 700, "bf16"), ("gguf_q6_k", 3, 5120, 300, "f32")])
def test_gemv_residual(dev, quant, rows, k, n, kind):
    """Projection + residual fused (stream, slab and phased slab forms): out = round(W x) + residual in the output type,
    bit for bit from the unfused kernel's own output."""
    rng = np.random.default_rng(31 + rows + n)
    x = rng.standard_normal((rows, k)).astype(np.float32)
    res = rng.standard_normal((rows, n)).astype(np.float32)
    w = O.random_weight(QT[quant], n, k, seed=n)
    if kind == "bf16":
        xin, rin, esz = O.f32_to_bf16_bits(x), O.f32_to_bf16_bits(res), 2
    else:
        xin, rin, esz = x, res, 4
    dx, dw, dr = dev.put(xin), dev.put(w), dev.put(rin)
    dplain, dout = dev.empty(rows * n * esz), dev.empty(rows * n * esz)
    G.FUSED[(quant[5:], kind, kind)](dx.ptr, dw.ptr, dplain.ptr, rows, k, n)
    G.gguf_gemv_residual(quant, dx.ptr, kind, dw.ptr, dr.ptr, dout.ptr, kind, rows, k, n)
    if kind == "bf16":
        plain = O.bf16_bits_to_f32(dev.get(dplain, np.uint16, (rows, n)))
        got = dev.get(dout, np.uint16, (rows, n))
        want = O.f32_to_bf16_bits(plain + O.bf16_bits_to_f32(rin))
        assert np.array_equal(got, want)
    else:
        plain = dev.get(dplain, np.float32, (rows, n))
        got = dev.get(dout, np.float32, (rows, n))
        assert np.array_equal(got.view(np.uint32), (plain + res).astype(np.float32).view(np.uint32))
    dev.free(dx, dw, dr, dplain, dout)


@pytest.mark.parametrize("rows,vocab,threads", [(1, 151936, 256), (8, 151936, 512), (3, 1000, 128), (5, 129, 256)])
def test_argmax_rows(dev, rows, vocab, threads):
    """Row-wise arg-max over the caller-owned two-stage scratch; equal values go to the lowest index."""
    from hipengine_amd.kernels.hip_gfx950.linear import lm_head as L
    rng = np.random.default_rng(rows + vocab)
    lg = rng.standard_normal((rows, vocab)).astype(np.float32)
    lg[0, [vocab - 1, vocab // 2, 5]] = 7.5
    if rows > 1:
        lg[1, :] = 0.25
    n = L.argmax_scratch_entries(rows, vocab, threads)
    dl = dev.put(lg)
    dbv, dbi = dev.empty(n * 4, fill=0xFF), dev.empty(n * 4, fill=0xFF)
    doi, dov = dev.empty(rows * 4, fill=0xFF), dev.empty(rows * 4, fill=0xFF)
    L.argmax_f32_rows_i32(dl.ptr, dbv.ptr, dbi.ptr, doi.ptr, dov.ptr, rows, vocab, threads=threads)
    idx, val = dev.get(doi, np.int32, (rows,)), dev.get(dov, np.float32, (rows,))
    L.argmax_f32_rows_i32(dl.ptr, dbv.ptr, dbi.ptr, doi.ptr, None, rows, vocab, threads=threads)
    idx2 = dev.get(doi, np.int32, (rows,))
    dev.free(dl, dbv, dbi, doi, dov)
    want_idx, want_val = O.argmax_rows(lg)
    assert np.array_equal(idx, want_idx) and np.array_equal(idx2, want_idx)
    assert np.array_equal(val.view(np.uint32), want_val.view(np.uint32))


def test_gemv_from_a_gguf_file(dev, tmp_path):
    """File to kernel: tensors written into a GGUF container, read back through the reader's memory maps, uploaded
    unchanged and multiplied - the raw block layout of the file IS the kernels' weight layout."""
    from hipengine_amd.loading import gguf as GG
    from hipengine_amd.quant.gguf import GGMLQuantizationType as T
    k, n = 1024, 96
    w4 = O.random_weight(O.GGML_Q4_K, n, k, seed=21)
    w6 = O.random_weight(O.GGML_Q6_K, n, k, seed=22)
    path = GG.write_gguf(tmp_path / "tiny.gguf", {"general.architecture": "test"},
                         [("a.weight", T.Q4_K, (n, k), w4), ("b.weight", T.Q6_K, (n, k), w6)])
    reader = GG.GGUFReader(path)
    x = np.random.default_rng(3).standard_normal((2, k)).astype(np.float32)
    dx = dev.put(x)
    for name, quant, w in (("a.weight", "gguf_q4_k", w4), ("b.weight", "gguf_q6_k", w6)):
        info = reader.tensor_info(name)
        assert info.shape == (n, k) and info.byte_shape == w.shape
        dw = reader.to_device(name, runtime=dev.runtime)
        dout = dev.empty(2 * n * 4)
        G.FUSED[(SHORT[quant], "f32", "f32")](dx.ptr, dw.ptr, dout.ptr, 2, k, n)
        got = dev.get(dout, np.float32, (2, n))
        dev.free(dw, dout)
        _check_f32(got, O.quantize_q8_1(x), w, QT[quant])
    dev.free(dx)


@pytest.mark.parametrize("rows,k,n", [(1, 5120, 300), (2, 1024, 77), (5, 2048, 64), (8, 512, 33), (1, 5120, 2560),
                                      (2, 5120, 4096), (1, 17408, 1100)])
def test_q5_k_fused_gemv_and_block_dots(dev, rows, k, n):
    """Q5_K (row-strided, stream and phased slab forms by shape): int32 sub-block dots bit-exact, float32 output within the parity gate of the
    reference CPU GEMV on the q8_1-dequantized activations; closed-form weights of the reference tests too."""
    rng = np.random.default_rng(rows + k + n)
    x = rng.standard_normal((rows, k)).astype(np.float32)
    xq = O.quantize_q8_1(x)
    for w in (_random_q5_k(n, k, 9), O.closed_form_q5_k(n, k)):
        dx, dxq, dw = dev.put(x), dev.put(xq), dev.put(w)
        dout = dev.empty(rows * n * 4)
        ddots, dqs = dev.empty(rows * n * (k // 32) * 4), dev.empty(rows * (k // 32) * 4)
        G.FUSED[("q5_k", "f32", "f32")](dx.ptr, dw.ptr, dout.ptr, rows, k, n)
        V.gguf_q8_1_block_dots_i32("gguf_q5_k", dxq.ptr, dw.ptr, ddots.ptr, dqs.ptr, rows, k, n)
        got = dev.get(dout, np.float32, (rows, n))
        dots = dev.get(ddots, np.int32, (rows, n, k // 32))
        dev.free(dx, dxq, dw, dout, ddots, dqs)
        want_dots, _ = O.block_dots_q5_k(O.q8_1_fields(xq)[2], w)
        assert np.array_equal(dots, want_dots)
        ref = O.gguf_quant_gemv(O.dequantize_q8_1(xq), w, O.GGML_Q5_K)
        assert O.max_rel_err(got, ref) <= REL_TOL and O.cosine(got, ref) >= COS_MIN


def _sweep_cases():
    """48 seeded (quant, rows, K, N, activation type) draws: every batch size, K from one block to 34 blocks, N from
    1 to a few thousand, so that every kernel form the launcher picks (stream, run, row-strided, slab, phased slab)
    and its ragged edges are met on shapes no other test names."""
    rng = np.random.default_rng(20240611)
    cases = []
    for i in range(48):
        quant = ("gguf_q4_k", "gguf_q5_k", "gguf_q6_k", "gguf_q8_0")[i % 4]
        rows = int(rng.integers(1, 9))
        k = 256 * int(rng.choice([1, 2, 3, 5, 8, 11, 16, 20, 24, 34]))
        n = int(rng.choice([1, 7, 31, 64, 100, 257, 640, 1000, 2049, 3333, 5120]))
        cases.append((quant, rows, k, n, "bf16" if i % 3 == 0 else "f32"))
    return cases


@pytest.mark.parametrize("quant,rows,k,n,act", _sweep_cases())
def test_fused_gemv_seeded_shape_sweep(dev, quant, rows, k, n, act):
    rng = np.random.default_rng(rows * 1000003 + k * 101 + n)
    x = (rng.standard_normal((rows, k)) * 0.5).astype(np.float32)
    if act == "bf16":
        x = O.bf16_bits_to_f32(O.f32_to_bf16_bits(x))
    qt = O.GGML_Q5_K if quant == "gguf_q5_k" else QT[quant]
    w = _random_q5_k(n, k, seed=k + n) if quant == "gguf_q5_k" else O.random_weight(qt, n, k, seed=k + n)
    xin = x if act == "f32" else O.f32_to_bf16_bits(x)
    dx, dw, dout = dev.put(xin), dev.put(w), dev.empty((rows * n + 4) * 4, fill=0x6B)
    G.FUSED[(quant[5:], act, "f32")](dx.ptr, dw.ptr, dout.ptr, rows, k, n)
    got = dev.get(dout, np.float32, (rows * n + 4,)).copy()
    dev.free(dx, dw, dout)
    assert np.all(got[rows * n:].view(np.uint32) == 0x6B6B6B6B)          # nothing past the output
    _check_f32(got[:rows * n].reshape(rows, n), O.quantize_q8_1(x), w, qt)


@pytest.mark.parametrize("rows,k", [(1, 32), (3, 5120), (8, 2048)])
def test_q8_1x2_planes_bytes_and_gemv_over_both(dev, rows, k):
    """The two-plane quantizer byte for byte; the pre-quantized GEMV over the planes as 2 * rows rows gives two
    partial products whose sum is closer to the float GEMV on the unquantized activations than plane 0 alone (what
    is left is the fp16 rounding of the blocks' raw sums, which the Q4_K min term of a pre-quantized GEMV reads)."""
    rng = np.random.default_rng(rows + k)
    x = (rng.standard_normal((rows, k)) * 0.7).astype(np.float32)
    x[0, :32] = 0.0
    xb = O.f32_to_bf16_bits(x)
    want = O.quantize_q8_1x2(O.bf16_bits_to_f32(xb))
    dx, dq = dev.put(xb), dev.empty(2 * rows * (k // 32) * 36, fill=0x33)
    Q.gguf_q4_k_quantize_bf16_q8_1x2(dx.ptr, dq.ptr, rows, k)
    got = dev.get(dq, np.uint8, want.shape).copy()
    assert np.array_equal(got, want)
    if k % 256 == 0 and 2 * rows <= 8:
        n = 96
        w = O.random_weight(O.GGML_Q4_K, n, k, seed=3)
        dw, dout = dev.put(w), dev.empty(2 * rows * n * 4)
        G.gguf_q4_k_q8_1_dp4a_vdr_bf16_f32_out(dq.ptr, dw.ptr, dout.ptr, 2 * rows, k, n)
        parts = dev.get(dout, np.float32, (2, rows, n)).copy()
        dev.free(dw, dout)
        ref = O.gguf_quant_gemv(O.bf16_bits_to_f32(xb), w, O.GGML_Q4_K)
        both, one = O.max_rel_err(parts[0] + parts[1], ref), O.max_rel_err(parts[0], ref)
        assert both <= 5e-3 and both < 0.6 * one, (both, one)
    dev.free(dx, dq)
