"""GPU tests of the drop-in boundary: the registry keys hipEngine's dispatcher resolves and the way it calls
what it gets (positional pointers and sizes, keyword stream/runtime/threads/library:
hipengine/runtime/gguf_linear.py:11255-11264), the named MoE call kinds, the step-by-step routing index
pipeline of the runner, and the int32 dots of every kernel form that runs on the MFMA.
"""

from __future__ import annotations

import numpy as np
import pytest

from oracle import c_oracle as C
from oracle import gguf_oracle as O
from hipengine_amd.kernels import registry
from hipengine_amd.kernels.hip_gfx950 import register_backend_kernels
from hipengine_amd.kernels.hip_gfx950.moe import group_scatter as GS
from hipengine_amd.kernels.hip_gfx950.quant import gguf_moe as M
from hipengine_amd.kernels.hip_gfx950.quant import gguf_q8_1_gemv as G
from hipengine_amd.kernels.hip_gfx950.quant import gguf_quantize as Q
from hipengine_amd.kernels.hip_gfx950.quant import gguf_verify as V
from hipengine_amd.synthetic import synthetic_blocks

pytestmark = pytest.mark.gpu

REL_TOL = 1e-3
COS_MIN = 0.99999
QT = {"gguf_q4_k": O.GGML_Q4_K, "gguf_q5_k": O.GGML_Q5_K, "gguf_q6_k": O.GGML_Q6_K, "gguf_q8_0": O.GGML_Q8_0}
BACKEND = "hip_gfx950"


def _close(got, ref):
    err, cos = O.max_rel_err(got, ref), O.cosine(got, ref)
    assert err <= REL_TOL, f"max rel err {err}"
    assert cos >= COS_MIN, f"cosine {cos}"


def _resolve(layer, quant, variant):
    register_backend_kernels()
    return registry.resolve(backend=BACKEND, layer=layer, quant=quant, variant=variant, missing="error")


def _act(x, act):
    if act == "bf16":
        bits = O.f32_to_bf16_bits(x)
        return bits, O.bf16_bits_to_f32(bits)
    if act == "fp16":
        h = x.astype(np.float16)
        return h, h.astype(np.float32)
    return x, x


def _out(buf_host, out):
    if out == "bf16":
        return O.bf16_bits_to_f32(buf_host)
    if out == "fp16":
        return buf_host.view(np.float16).astype(np.float32)
    return buf_host


@pytest.mark.parametrize("quant", ["gguf_q4_k", "gguf_q6_k", "gguf_q8_0"])
@pytest.mark.parametrize("act,out", [("bf16", "bf16"), ("bf16", "fp16"), ("bf16", "f32"), ("f32", "f32")])
def test_dispatcher_keys_called_like_launch_raw(dev, quant, act, out):
    """rows = 1 resolves gemv_*, rows > 1 the prefill_* rewrite (consumer_surface.py:134-144); the call is the
    dispatcher's: positional pointers and sizes, then stream / runtime / threads / library by keyword."""
    k, n = 2048, 320
    rng = np.random.default_rng(k + n)
    w = O.random_weight(QT[quant], n, k, seed=7)
    dw = dev.put(w)
    for rows in (1, 5, 19):
        variant = f"{'gemv' if rows == 1 else 'prefill'}_{act}_{out}_out"
        fn = _resolve("linear", quant, variant)
        x = rng.standard_normal((rows, k)).astype(np.float32)
        xin, xf = _act(x, act)
        dx = dev.put(xin)
        dout = dev.empty(rows * n * (4 if out == "f32" else 2))
        fn(dx.ptr, dw.ptr, dout.ptr, rows, k, n, stream=0, runtime=dev.runtime, threads=128, library=dev.library)
        got = _out(dev.get(dout, np.float32 if out == "f32" else np.uint16, (rows, n)), out)
        dev.free(dx, dout)
        ref = O.gguf_quant_gemv(O.dequantize_q8_1(O.quantize_q8_1(xf)), w, QT[quant])
        if out == "f32":
            _close(got, ref)
        else:   # a 16-bit output carries its own rounding: 2^-8 (bf16) / 2^-11 (fp16) relative
            assert O.max_rel_err(got, ref, floor_frac=1e-2) <= (8e-3 if out == "bf16" else 3e-3)
            assert O.cosine(got, ref) >= 0.9999
    dev.free(dw)


@pytest.mark.parametrize("quant", ["gguf_q4_k", "gguf_q6_k", "gguf_q8_0"])
def test_rowtile_keys_are_the_batch_launch(dev, quant):
    """("linear", quant, "rowtile_<act>_<out>_out") (gguf_q4_k_gemv.py:1552-1554) for 2 to 8 rows: the bits of the
    prefill_* key on the same input."""
    k, n = 2048, 200
    rng = np.random.default_rng(k)
    w = O.random_weight(QT[quant], n, k, seed=17)
    dw = dev.put(w)
    for rows, act, out in ((2, "f32", "f32"), (4, "bf16", "f32"), (8, "bf16", "bf16")):
        xin, _ = _act(rng.standard_normal((rows, k)).astype(np.float32), act)
        dx = dev.put(xin)
        got = []
        for family in ("rowtile", "prefill"):
            dout = dev.empty(rows * n * (4 if out == "f32" else 2))
            _resolve("linear", quant, f"{family}_{act}_{out}_out")(dx.ptr, dw.ptr, dout.ptr, rows, k, n, stream=0,
                                                                   runtime=dev.runtime, threads=128, library=dev.library)
            got.append(dev.get(dout, np.float32 if out == "f32" else np.uint16, (rows, n)))
            dev.free(dout)
        dev.free(dx)
        assert np.array_equal(got[0].view(np.uint8), got[1].view(np.uint8))
    dev.free(dw)


@pytest.mark.parametrize("quant,n", [("gguf_q4_k", 352), ("gguf_q6_k", 333), ("gguf_q5_k", 160), ("gguf_q8_0", 75)])
def test_prefill_key_with_workspace_runs_the_mmq(dev, quant, n):
    """prefill_bf16_f32_out with 32 rows or more packs the activations and runs the int8-MFMA MMQ, into a
    caller-owned workspace or - called the way hipEngine's dispatcher calls it, positionally and with no workspace -
    into the pack buffer the library holds: the same bits either way, equal to the MMQ formula of the oracle.  Below
    32 rows the key runs the GEMV in batches of 8 (GEMV-convention q8_1)."""
    rows, k = 70, 1024
    rng = np.random.default_rng(3)
    xb = O.f32_to_bf16_bits((rng.standard_normal((rows, k)) * 0.25).astype(np.float32))
    w = (synthetic_blocks(QT[quant], n, k, seed=5, tile_rows=n) if quant == "gguf_q5_k"
         else O.random_weight(QT[quant], n, k, seed=5))
    fn = _resolve("linear", quant, "prefill_bf16_f32_out")
    need = G.gguf_prefill_workspace_bytes(quant, rows, k)
    assert need == rows * (k // 128) * (144 if quant == "gguf_q4_k" else 160)
    dx, dw = dev.put(xb), dev.put(w)
    dws, d1, d2 = dev.empty(need), dev.empty(rows * n * 4), dev.empty(rows * n * 4)
    fn(dx.ptr, dw.ptr, d1.ptr, rows, k, n, stream=0, runtime=dev.runtime, workspace_ptr=dws.ptr, workspace_bytes=need)
    fn(dx.ptr, dw.ptr, d2.ptr, rows, k, n)
    few = 20
    d3 = dev.empty(few * n * 4)
    fn(dx.ptr, dw.ptr, d3.ptr, few, k, n)
    with_ws, without = dev.get(d1, np.float32, (rows, n)).copy(), dev.get(d2, np.float32, (rows, n)).copy()
    short = dev.get(d3, np.float32, (few, n)).copy()
    packed = dev.get(dws, np.uint8, (rows, k // 128, need // rows // (k // 128)))
    dev.free(dx, dw, dws, d1, d2, d3)
    if quant == "gguf_q4_k":
        want_pack = O.pack_q8_1_ds4(xb)
        ref = O.mmq_q4_k_ds4(want_pack, w)
    elif quant == "gguf_q5_k":
        want_pack = O.pack_q8_1_d4s4(xb)
        ref = O.mmq_q5_k_d4s4(want_pack, w)
    elif quant == "gguf_q8_0":
        want_pack = O.pack_q8_1_d4s4(xb)
        ref = O.mmq_q8_0_d4s4(want_pack, w)
    else:
        want_pack = O.pack_q8_1_d4s4(xb)
        ref = O.mmq_q6_k_d4s4(want_pack, w)
    assert np.array_equal(packed.reshape(want_pack.shape), want_pack)
    _close(with_ws, ref)
    assert np.array_equal(with_ws.view(np.uint32), without.view(np.uint32))
    _close(short, O.gguf_quant_gemv(O.dequantize_q8_1(O.quantize_q8_1(O.bf16_bits_to_f32(xb[:few]))), w, QT[quant]))
    assert O.cosine(with_ws[:few], short) >= 0.9999


@pytest.mark.parametrize("quant,k,n,rows", [("gguf_q4_k", 5120, 1024, 2048), ("gguf_q6_k", 17408, 256, 1100), ("gguf_q8_0", 1024, 77, 560)])
def test_prefill_key_chunks_through_the_library_buffer(dev, quant, k, n, rows):
    """More rows than one chunk of the library's pack buffer holds (512): every chunk's rows equal the MMQ of the same
    rows run on their own, bit for bit, and two calls in a row (which take the two regions of the buffer in turn) agree."""
    rng = np.random.default_rng(rows)
    xb = O.f32_to_bf16_bits((rng.standard_normal((rows, k)) * 0.25).astype(np.float32))
    w = O.random_weight(QT[quant], n, k, seed=6)
    fn = _resolve("linear", quant, "prefill_bf16_bf16_out")
    dx, dw = dev.put(xb), dev.put(w)
    d1, d2 = dev.empty(rows * n * 2), dev.empty(rows * n * 2)
    fn(dx.ptr, dw.ptr, d1.ptr, rows, k, n)
    fn(dx.ptr, dw.ptr, d2.ptr, rows, k, n)
    a, b = dev.get(d1, np.uint16, (rows, n)).copy(), dev.get(d2, np.uint16, (rows, n)).copy()
    assert np.array_equal(a, b)
    # the last, ragged chunk on its own through a caller-owned workspace
    r0 = (rows // 512) * 512 if rows % 512 else rows - 512
    tail = rows - r0
    need = G.gguf_prefill_workspace_bytes(quant, tail, k)
    dws, d3 = dev.empty(need), dev.empty(tail * n * 2)
    dxt = dev.put(xb[r0:])
    fn(dxt.ptr, dw.ptr, d3.ptr, tail, k, n, workspace_ptr=dws.ptr, workspace_bytes=need)
    c = dev.get(d3, np.uint16, (tail, n)).copy()
    dev.free(dx, dw, d1, d2, dws, d3, dxt)
    assert np.array_equal(a[r0:], c)
    pack = O.pack_q8_1_ds4(xb[:64]) if quant == "gguf_q4_k" else O.pack_q8_1_d4s4(xb[:64])
    ref = {"gguf_q4_k": O.mmq_q4_k_ds4, "gguf_q6_k": O.mmq_q6_k_d4s4, "gguf_q8_0": O.mmq_q8_0_d4s4}[quant](pack, w)
    assert np.allclose(O.bf16_bits_to_f32(a[:64]), ref, rtol=2.0 ** -8, atol=1e-3 * np.abs(ref).max())


@pytest.mark.parametrize("quant", ["gguf_q4_k", "gguf_q6_k", "gguf_q8_0"])
@pytest.mark.parametrize("rows", [1, 2, 8])
def test_dense_dual_gemv(dev, quant, rows):
    """Two matrices over one activation (k and v of an attention block): each output equals the single GEMV's."""
    k, n = 5120, 1024
    rng = np.random.default_rng(11 + rows)
    x = rng.standard_normal((rows, k)).astype(np.float32)
    xb = O.f32_to_bf16_bits(x)
    wa, wb = O.random_weight(QT[quant], n, k, seed=1), O.random_weight(QT[quant], n, k, seed=2)
    fn = _resolve("linear", quant, "dual_gemv_bf16_bf16_out")
    dx, dwa, dwb = dev.put(xb), dev.put(wa), dev.put(wb)
    da, db, ds = dev.empty(rows * n * 2), dev.empty(rows * n * 2), dev.empty(rows * n * 2)
    fn(dx.ptr, dwa.ptr, dwb.ptr, da.ptr, db.ptr, rows, k, n, stream=0, runtime=dev.runtime)
    short = quant.removeprefix("gguf_")
    got_a, got_b = dev.get(da, np.uint16, (rows, n)).copy(), dev.get(db, np.uint16, (rows, n)).copy()
    for w_dev, got in ((dwa, got_a), (dwb, got_b)):
        G.FUSED[(short, "bf16", "bf16")](dx.ptr, w_dev.ptr, ds.ptr, rows, k, n)
        assert np.array_equal(got, dev.get(ds, np.uint16, (rows, n)))
    dev.free(dx, dwa, dwb, da, db, ds)


@pytest.mark.parametrize("rows", [1, 2, 3, 5, 8])
@pytest.mark.parametrize("mats", [(("gguf_q4_k", 640), ("gguf_q4_k", 256), ("gguf_q6_k", 256)),
                                  (("gguf_q8_0", 130), ("gguf_q5_k", 1021)),
                                  (("gguf_q6_k", 96), ("gguf_q4_k", 64), ("gguf_q4_k", 32), ("gguf_q8_0", 7))],
                         ids=["qkv", "two_ragged", "four_small"])
def test_multi_gemv_matches_the_single_calls_and_the_oracle(dev, rows, mats):
    """Several matrices of mixed types and row counts over one activation: one launch at rows <= 2; at rows 3..8 the
    Q4_K matrices share one launch of the slab form and the others go one by one; every output has the bits of its
    own fused GEMV call and meets the oracle's tolerance."""
    k = 5120
    rng = np.random.default_rng(31 + rows)
    x = rng.standard_normal((rows, k)).astype(np.float32)
    # Q5_K has no quantizer in the oracle: random valid blocks
    ws = [synthetic_blocks(QT[q], n, k, seed=5 + i, tile_rows=n) if q == "gguf_q5_k" else O.random_weight(QT[q], n, k, seed=5 + i)
          for i, (q, n) in enumerate(mats)]
    fn = _resolve("linear", "gguf", "multi_gemv")
    dx = dev.put(x)
    dws = [dev.put(w) for w in ws]
    outs = [dev.empty(rows * n * 4) for _, n in mats]
    single = [dev.empty(rows * n * 4) for _, n in mats]
    for o, (_, n) in zip(outs, mats):
        dev.runtime.memset(o.ptr, 0xFF, rows * n * 4)
    fn([q for q, _ in mats], dx.ptr, "f32", [d.ptr for d in dws], [o.ptr for o in outs], "f32", rows, k,
       [n for _, n in mats], stream=0, runtime=dev.runtime)
    xq = O.dequantize_q8_1(O.quantize_q8_1(x))
    for (q, n), w, dw, o, sgl in zip(mats, ws, dws, outs, single):
        G.FUSED[(q.removeprefix("gguf_"), "f32", "f32")](dx.ptr, dw.ptr, sgl.ptr, rows, k, n)
        got = dev.get(o, np.float32, (rows, n)).copy()
        alone = dev.get(sgl, np.float32, (rows, n))
        if rows > 2 or G.gguf_gemv_default_form(q, rows, k, n)[0] == "stream":
            # the same kernel form as the call of its own: the same float32 sums
            assert np.array_equal(got.view(np.uint32), alone.view(np.uint32)), (q, n)
        _close(got, O.gguf_quant_gemv(xq, w, QT[q]))
        _close(alone, O.gguf_quant_gemv(xq, w, QT[q]))
    dev.free(dx, *dws, *outs, *single)


@pytest.mark.parametrize("rows", [4, 8])
def test_multi_gemv_attention_shapes_batch_3_to_8(dev, rows):
    """q | k | v of a 27B-shape attention block (Q4_K 5120 and 1024 rows, Q6_K 1024 rows, K = 5120) at batch 4 and 8:
    q and k share one slab launch (213 + 42 workgroups), v takes the phased slab; bits of the single calls."""
    k = 5120
    mats = (("gguf_q4_k", 5120), ("gguf_q4_k", 1024), ("gguf_q6_k", 1024))
    rng = np.random.default_rng(77 + rows)
    x = rng.standard_normal((rows, k)).astype(np.float32)
    ws = [synthetic_blocks(QT[q], n, k, seed=50 + i) for i, (q, n) in enumerate(mats)]
    fn = _resolve("linear", "gguf", "multi_gemv")
    dx = dev.put(x)
    dws = [dev.put(w) for w in ws]
    outs = [dev.empty(rows * n * 4, fill=0x7C) for _, n in mats]
    single = [dev.empty(rows * n * 4) for _, n in mats]
    fn([q for q, _ in mats], dx.ptr, "f32", [d.ptr for d in dws], [o.ptr for o in outs], "f32", rows, k,
       [n for _, n in mats], stream=0, runtime=dev.runtime)
    for (q, n), dw, o, sgl in zip(mats, dws, outs, single):
        G.FUSED[(q.removeprefix("gguf_"), "f32", "f32")](dx.ptr, dw.ptr, sgl.ptr, rows, k, n)
        got, alone = dev.get(o, np.float32, (rows, n)).copy(), dev.get(sgl, np.float32, (rows, n))
        assert np.array_equal(got.view(np.uint32), alone.view(np.uint32)), (q, n)
    dev.free(dx, *dws, *outs, *single)


# ---- MoE call kinds -------------------------------------------------------------------------

E, TOPK, H, I = 12, 4, 1024, 512


def _experts(seed):
    rng = np.random.default_rng(seed)
    gate = np.stack([O.random_weight(O.GGML_Q4_K, I, H, seed=seed + 10 + e) for e in range(E)])
    up = np.stack([O.random_weight(O.GGML_Q4_K, I, H, seed=seed + 40 + e) for e in range(E)])
    down = np.stack([O.random_weight(O.GGML_Q4_K, H, I, seed=seed + 70 + e) for e in range(E)])
    return rng, gate, up, down


@pytest.mark.parametrize("prequantized", [False, True])
def test_selected_dual_gemv_two_outputs(dev, prequantized):
    """The `dual` call kind: gate and up of every lane from one pass, no activation function; over bf16 rows
    and over pre-quantized q8_1 rows (caller-owned scratch written by the quantize entry point)."""
    rng, gate, up, _ = _experts(100)
    tokens = 3
    x = rng.standard_normal((tokens, H)).astype(np.float32)
    xb = O.f32_to_bf16_bits(x)
    sel = np.stack([rng.permutation(E)[:TOPK] for _ in range(tokens)]).astype(np.int64)
    sel[1, 2] = -1   # a dropped lane stays untouched
    lanes = tokens * TOPK
    dx, dsel, dg, du = dev.put(xb), dev.put(sel), dev.put(gate), dev.put(up)
    da, db = dev.empty(lanes * I * 2, fill=0xCD), dev.empty(lanes * I * 2, fill=0xCD)
    xq = O.quantize_q8_1(O.bf16_bits_to_f32(xb))
    if prequantized:
        dq = dev.empty(xq.size)
        Q.gguf_q4_k_quantize_bf16_q8_1(dx.ptr, dq.ptr, tokens, H)
        fn = _resolve("linear", "gguf_q4_k", "selected_dual_gemv_q8_1_dp4a_bf16_bf16_out")
        fn(dq.ptr, dsel.ptr, dg.ptr, du.ptr, da.ptr, db.ptr, tokens, lanes, E, H, I, stream=0, runtime=dev.runtime)
        dev.free(dq)
    else:
        fn = _resolve("linear", "gguf_q4_k", "selected_dual_gemv_bf16_bf16_out")
        fn(dx.ptr, dsel.ptr, dg.ptr, du.ptr, da.ptr, db.ptr, tokens, lanes, E, H, I, stream=0, runtime=dev.runtime)
    got_a = dev.get(da, np.uint16, (lanes, I)).copy()
    got_b = dev.get(db, np.uint16, (lanes, I)).copy()
    dev.free(dx, dsel, dg, du, da, db)
    x_deq = O.dequantize_q8_1(xq)
    for lane in range(lanes):
        e = int(sel.reshape(-1)[lane])
        if e < 0:
            assert np.all(got_a[lane] == 0xCDCD) and np.all(got_b[lane] == 0xCDCD)
            continue
        xt = x_deq[lane // TOPK: lane // TOPK + 1]
        for got, wt in ((got_a, gate), (got_b, up)):
            ref = O.gguf_quant_gemv(xt, wt[e], O.GGML_Q4_K)
            assert O.max_rel_err(O.bf16_bits_to_f32(got[lane:lane + 1]), ref, floor_frac=1e-2) <= 8e-3


def test_weighted_down_call_kind(dev):
    """`weighted_down`: keyword geometry (tokens, top_k, ...) as loading/gguf_selected_contract.py:305-315 passes it."""
    rng, _, _, down = _experts(200)
    tokens = 5
    lanes = tokens * TOPK
    x = (rng.standard_normal((lanes, I)) * 0.5).astype(np.float32)
    xb = O.f32_to_bf16_bits(x)
    sel = np.stack([rng.permutation(E)[:TOPK] for _ in range(tokens)]).astype(np.int64)
    wts = rng.random((tokens, TOPK)).astype(np.float32)
    fn = _resolve("moe_linear", "gguf_q4_k", "selected_weighted_down_gemv_decode_bf16_bf16_out")
    dx, dsel, dwt, dd = dev.put(xb), dev.put(sel), dev.put(wts), dev.put(down)
    dout = dev.empty(tokens * H * 2)
    fn(dx.ptr, dsel.ptr, dwt.ptr, dd.ptr, dout.ptr, tokens=tokens, top_k=TOPK, num_experts=E, in_features=I,
       out_features=H, stream=0, runtime=dev.runtime)
    got = O.bf16_bits_to_f32(dev.get(dout, np.uint16, (tokens, H)))
    dev.free(dx, dsel, dwt, dd, dout)
    x_deq = O.dequantize_q8_1(O.quantize_q8_1(O.bf16_bits_to_f32(xb)))
    ref = np.zeros((tokens, H), dtype=np.float32)
    for t in range(tokens):
        for s in range(TOPK):
            lane = t * TOPK + s
            ref[t] += wts[t, s] * O.gguf_quant_gemv(x_deq[lane:lane + 1], down[sel[t, s]], O.GGML_Q4_K)[0]
    assert O.max_rel_err(got, ref, floor_frac=1e-2) <= 8e-3
    assert O.cosine(got, ref) >= 0.9999


@pytest.mark.parametrize("tokens", [1, 8, 40])
def test_grouped_gemv_over_compact_rows(dev, tokens):
    """Rows gathered in expert-major order x expert_start -> every row times its expert's matrix; experts with
    one or two rows (decode) and with more than eight (several batches) both occur.  Rows between the ranges
    do not exist here (unpadded starts); the row after the last is left untouched."""
    rng, gate, _, _ = _experts(300)
    x = rng.standard_normal((tokens, H)).astype(np.float32)
    xb = O.f32_to_bf16_bits(x)
    sel = np.stack([rng.permutation(E)[:TOPK] for _ in range(tokens)]).astype(np.int64)
    idx = O.build_routing_index(sel, np.ones_like(sel, dtype=np.float32), E)
    total = idx["total"]
    packed = xb[idx["compact_to_source"]]
    fn = _resolve("moe_linear", "gguf_q4_k", "selected_grouped_prefill_compact_rowbatch8_bf16_bf16_out")
    dx, des, dg = dev.put(packed), dev.put(idx["expert_start"]), dev.put(gate)
    dout = dev.empty((total + 1) * I * 2, fill=0xEE)
    fn(dx.ptr, des.ptr, dg.ptr, dout.ptr, total, E, H, I, stream=0, runtime=dev.runtime)
    got = dev.get(dout, np.uint16, (total + 1, I))
    dev.free(dx, des, dg, dout)
    assert np.all(got[total] == 0xEEEE)
    x_deq = O.dequantize_q8_1(O.quantize_q8_1(O.bf16_bits_to_f32(packed)))
    for r in range(total):
        e = int(idx["sorted_experts"][r])
        ref = O.gguf_quant_gemv(x_deq[r:r + 1], gate[e], O.GGML_Q4_K)
        assert O.max_rel_err(O.bf16_bits_to_f32(got[r:r + 1]), ref, floor_frac=1e-2) <= 8e-3, r


@pytest.mark.parametrize("quant", ["gguf_q5_k", "gguf_q6_k", "gguf_q8_0"])
def test_grouped_gemv_other_expert_types(dev, quant):
    """The grouped GEMV for Q5_K, Q6_K and Q8_0 expert weights in the raw layout (float32 in and out): experts
    with 1, 2, several and more than 8 rows, and experts with none."""
    experts, hidden, inter = 6, 1024, 96
    counts = np.array([1, 0, 2, 11, 0, 5])
    start = np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)
    total = int(start[-1])
    rng = np.random.default_rng(77)
    x = (rng.standard_normal((total, hidden)) * 0.5).astype(np.float32)
    w = np.stack([synthetic_blocks(QT[quant], inter, hidden, seed=20 + e, tile_rows=inter) if quant == "gguf_q5_k"
                  else O.random_weight(QT[quant], inter, hidden, seed=20 + e) for e in range(experts)])
    fn = _resolve("moe_linear", quant, "grouped_gemv_rowbatch8")
    dx, des, dw = dev.put(x), dev.put(start), dev.put(w)
    dout = dev.empty((total + 1) * inter * 4, fill=0xEE)
    fn(dx.ptr, des.ptr, dw.ptr, dout.ptr, total, experts, hidden, inter, x_dtype="f32", out_dtype="f32", stream=0,
       runtime=dev.runtime)
    got = dev.get(dout, np.float32, (total + 1, inter))
    dev.free(dx, des, dw, dout)
    assert np.all(got[total].view(np.uint32) == 0xEEEEEEEE)
    x_deq = O.dequantize_q8_1(O.quantize_q8_1(x))
    for e in range(experts):
        lo, hi = int(start[e]), int(start[e + 1])
        if hi > lo:
            _close(got[lo:hi], O.gguf_quant_gemv(x_deq[lo:hi], w[e], QT[quant]))


# ---- the runner's step-by-step routing index ----------------------------------------------------

@pytest.mark.parametrize("tokens,top_k,experts,pad", [(1, 8, 256, 1), (8, 8, 256, 1), (333, 4, 60, 1), (2048, 8, 256, 1),
                                                      (50, 2, 7, 16)])
def test_count_prefix_scatter_gather_pipeline(dev, tokens, top_k, experts, pad):
    """zero counts -> group_count -> group_prefix -> zero offsets -> scatter_gather, in the order of
    runtime/qwen35_gguf_runner.py:34107-34143; every array equals the oracle's stable index bit for bit."""
    rng = np.random.default_rng(tokens * 7 + experts)
    hidden = 384
    sel = rng.integers(0, experts, size=(tokens, top_k)).astype(np.int64)
    if tokens > 2:
        sel[1, 0], sel[2, top_k - 1] = -1, experts + 5
    wts = rng.random((tokens, top_k)).astype(np.float32)
    hs = rng.integers(0, 65536, size=(tokens, hidden)).astype(np.uint16)
    lanes = tokens * top_k
    want = O.build_routing_index(sel, wts, experts, pad_multiple=pad)
    total = want["total"]
    d = {"sel": dev.put(sel), "w": dev.put(wts), "hs": dev.put(hs), "counts": dev.put(np.zeros(experts, np.int32)),
         "padded": dev.empty(experts * 4), "start": dev.empty((experts + 1) * 8), "total": dev.empty(8),
         "offs": dev.put(np.zeros(experts, np.int32)), "lanes": dev.empty(max(total, 1) * 8, fill=0xFF),
         "exps": dev.empty(max(total, 1) * 8, fill=0xFF), "sw": dev.empty(max(total, 1) * 4, fill=0),
         "packed": dev.empty(max(total, 1) * hidden * 2, fill=0x77)}
    GS.qwen35_moe_group_count(d["sel"].ptr, d["counts"].ptr, lanes, experts)
    GS.qwen35_moe_group_prefix(d["counts"].ptr, d["padded"].ptr, d["start"].ptr, d["total"].ptr, experts, pad)
    GS.qwen35_moe_group_scatter_gather_lowp(d["hs"].ptr, d["sel"].ptr, d["w"].ptr, d["start"].ptr, d["offs"].ptr,
                                            d["lanes"].ptr, d["exps"].ptr, d["sw"].ptr, d["packed"].ptr, lanes, experts,
                                            top_k, hidden)
    assert np.array_equal(dev.get(d["counts"], np.int32, (experts,)), want["counts"])
    assert np.array_equal(dev.get(d["start"], np.int64, (experts + 1,)), want["expert_start"])
    assert int(dev.get(d["total"], np.int64, (1,))[0]) == total
    assert np.array_equal(dev.get(d["offs"], np.int32, (experts,)), want["counts"])
    got_lanes = dev.get(d["lanes"], np.int64, (total,))
    filled = want["sorted_lanes"] >= 0
    assert np.array_equal(got_lanes[filled], want["sorted_lanes"][filled])
    assert np.all(got_lanes[~filled] == -1)                      # padding slots keep the caller's fill
    assert np.array_equal(dev.get(d["exps"], np.int64, (total,))[filled], want["sorted_experts"][filled])
    assert np.array_equal(dev.get(d["sw"], np.float32, (total,))[filled].view(np.uint32),
                          want["sorted_weights"][filled].view(np.uint32))
    got_packed = dev.get(d["packed"], np.uint16, (total, hidden))
    assert np.array_equal(got_packed[filled], hs[want["compact_to_source"][filled]])
    assert np.all(got_packed[~filled] == 0x7777)
    # the stand-alone gather over the same index: padding slots (lane -1) give zero rows
    d["packed2"] = dev.empty(max(total, 1) * hidden * 2, fill=0x55)
    GS.qwen35_moe_gather_packed_hidden_lowp(d["hs"].ptr, d["lanes"].ptr, d["packed2"].ptr, total * hidden, tokens, top_k, hidden)
    got2 = dev.get(d["packed2"], np.uint16, (total, hidden))
    assert np.array_equal(got2[filled], hs[want["compact_to_source"][filled]])
    assert np.all(got2[~filled] == 0)
    dev.free(*d.values())


# ---- int32 dots of the forms that run on the MFMA ------------------------------------------------

def _qs(xq):
    return O.q8_1_fields(xq)[2]          # int8 [rows, K/32, 32]


@pytest.mark.parametrize("quant,form,k,n,rows", [
    ("gguf_q4_k", V.FORM_SLAB, 5120, 200, 8),      # two blocks per wave on eight waves, one on four
    ("gguf_q4_k", V.FORM_SLAB, 2048, 70, 3),       # one block per wave, a ragged slab
    ("gguf_q4_k", V.FORM_PSLAB, 17408, 160, 8),    # phased: K does not fit one pass
    ("gguf_q5_k", V.FORM_PSLAB, 5120, 130, 5),
    ("gguf_q6_k", V.FORM_PSLAB, 5120, 300, 8),
    ("gguf_q6_k", V.FORM_PSLAB, 17408, 100, 4),
    ("gguf_q8_0", V.FORM_PSLAB, 5120, 150, 8),
])
def test_gemv_mfma_forms_int32_dots_bit_exact(dev, quant, form, k, n, rows):
    """Every int32 sub-block dot the slab / phased slab kernels feed their float32 combine with, written by the
    production kernel body, equals the oracle's integer dot; the float32 result of the same launch passes the
    usual gate."""
    rng = np.random.default_rng(k + n + rows)
    x = rng.standard_normal((rows, k)).astype(np.float32)
    xq = O.quantize_q8_1(x)
    qt = QT[quant]
    if quant == "gguf_q5_k":
        nblk = n * (k // 256)
        w = O.pack_q5_k_blocks(rng.integers(0, 32, size=(nblk, 8, 32), dtype=np.uint8),
                               rng.integers(0, 64, size=(nblk, 8), dtype=np.uint8),
                               rng.integers(0, 64, size=(nblk, 8), dtype=np.uint8),
                               (rng.random(nblk) * 0.05).astype(np.float32),
                               (rng.random(nblk) * 0.02).astype(np.float32)).reshape(n, -1)
    else:
        w = O.random_weight(qt, n, k, seed=n)
    per = k // 16 if quant == "gguf_q6_k" else k // 32
    dxq, dw = dev.put(xq), dev.put(w)
    ddots, dout = dev.empty(rows * n * per * 4, fill=0x5A), dev.empty(rows * n * 4)
    V.gguf_gemv_mfma_dots_i32(quant, form, dxq.ptr, dw.ptr, ddots.ptr, dout.ptr, rows, k, n)
    got = dev.get(ddots, np.int32, (rows, n, per)).copy()
    out = dev.get(dout, np.float32, (rows, n)).copy()
    dev.free(dxq, dw, ddots, dout)
    qs = _qs(xq)
    if quant == "gguf_q4_k":
        want = O.block_dots_q4_k(qs, w)[0]
    elif quant == "gguf_q5_k":
        want = O.block_dots_q5_k(qs, w)[0]
    elif quant == "gguf_q6_k":
        want = O.block_dots_q6_k(qs, w)
    else:
        want = O.block_dots_q8_0(qs, w)
    assert np.array_equal(got, want.astype(np.int32))
    if quant != "gguf_q5_k":
        assert np.array_equal(got, np.asarray(C.block_dots(xq, w, qt)[0] if quant == "gguf_q4_k" else C.block_dots(xq, w, qt)))
    _close(out, O.gguf_quant_gemv(O.dequantize_q8_1(xq), w, qt))


@pytest.mark.parametrize("quant,rows,k,n", [("gguf_q4_k", 150, 1024, 160), ("gguf_q6_k", 129, 768, 130),
                                            ("gguf_q5_k", 131, 1280, 96), ("gguf_q8_0", 133, 640, 77)])
def test_mmq_int32_dots_bit_exact(dev, quant, rows, k, n):
    """The int32 tiles of the MMQ prefill GEMM (v_mfma_i32_32x32x32_i8 / 32x32x16) against the oracle's integer
    dots of the same packed activations; ragged tiles in both dimensions."""
    rng = np.random.default_rng(rows + k)
    xb = O.f32_to_bf16_bits((rng.standard_normal((rows, k)) * 0.3).astype(np.float32))
    w = (synthetic_blocks(QT[quant], n, k, seed=9, tile_rows=n) if quant == "gguf_q5_k"
         else O.random_weight(QT[quant], n, k, seed=9))
    if quant == "gguf_q4_k":
        xq = O.pack_q8_1_ds4(xb)
        qs = O.ds4_fields(xq)[2].reshape(rows, k // 32, 32)
        want, per = O.block_dots_q4_k(qs, w)[0], k // 32
        ref = O.mmq_q4_k_ds4(xq, w)
    elif quant == "gguf_q5_k":
        xq = O.pack_q8_1_d4s4(xb)
        qs = O.d4s4_fields(xq)[2].reshape(rows, k // 32, 32)
        want, per = O.block_dots_q5_k(qs, w)[0], k // 32
        ref = O.mmq_q5_k_d4s4(xq, w)
    elif quant == "gguf_q8_0":
        xq = O.pack_q8_1_d4s4(xb)
        qs = O.d4s4_fields(xq)[2].reshape(rows, k // 32, 32)
        want, per = O.block_dots_q8_0(qs, w), k // 32
        ref = O.mmq_q8_0_d4s4(xq, w)
    else:
        xq = O.pack_q8_1_d4s4(xb)
        qs = O.d4s4_fields(xq)[2].reshape(rows, k // 32, 32)
        want, per = O.block_dots_q6_k(qs, w), k // 16
        ref = O.mmq_q6_k_d4s4(xq, w)
    dxq, dw = dev.put(xq), dev.put(w)
    ddots, dout = dev.empty(rows * n * per * 4, fill=0x5A), dev.empty(rows * n * 4)
    V.gguf_mmq_dots_i32(quant, dxq.ptr, dw.ptr, ddots.ptr, dout.ptr, rows, k, n)
    got = dev.get(ddots, np.int32, (rows, n, per)).copy()
    out = dev.get(dout, np.float32, (rows, n)).copy()
    dev.free(dxq, dw, ddots, dout)
    assert np.array_equal(got, want.astype(np.int32))
    _close(out, ref)


def test_dense_tuning_variant_names_are_the_dense_launch(dev):
    """hipEngine's per-shape variant names of the Q5_K / Q6_K / Q8_0 GEMV: the bits of the dense entry of the same
    types, at a shape none of them was tuned for; the Q5_K pair names against two single launches."""
    rows, k, n = 3, 1024, 200
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((rows, k)) * 0.4).astype(np.float32)
    weights = {"q5_k": synthetic_blocks(O.GGML_Q5_K, n, k, seed=2, tile_rows=n), "q6_k": O.random_weight(O.GGML_Q6_K, n, k, seed=2),
               "q8_0": O.random_weight(O.GGML_Q8_0, n, k, seed=2)}
    dw = {q: dev.put(w) for q, w in weights.items()}
    dx = {"f32": dev.put(x), "bf16": dev.put(O.f32_to_bf16_bits(x))}
    base = {}
    for (quant, variant), fn in G.DENSE_VARIANTS.items():
        act, out = variant.split("_")[-3], variant.split("_")[-2]
        item = 4 if out == "f32" else 2
        key = (quant, act, out)
        if key not in base:
            dout = dev.empty(rows * n * item)
            G.DENSE[(quant, "gemv", act, out)](dx[act].ptr, dw[quant].ptr, dout.ptr, rows, k, n)
            base[key] = dev.get(dout, np.uint8, (rows * n * item,)).copy()
            dev.free(dout)
        dout = dev.empty(rows * n * item, fill=0x3C)
        fn(dx[act].ptr, dw[quant].ptr, dout.ptr, rows, k, n)
        assert np.array_equal(dev.get(dout, np.uint8, (rows * n * item,)), base[key]), variant
        dev.free(dout)
    nb = 72
    wb = synthetic_blocks(O.GGML_Q5_K, nb, k, seed=9, tile_rows=nb)
    dwb = dev.put(wb)
    for variant, fn in G.Q5_K_PAIR.items():
        out = variant.split("_")[-2]
        item = 4 if out == "f32" else 2
        da, db, sa, sb = (dev.empty(rows * m * item, fill=0x3C) for m in (n, nb, n, nb))
        fn(dx["bf16"].ptr, dw["q5_k"].ptr, dwb.ptr, da.ptr, db.ptr, rows, k, n, nb)
        single = G.DENSE[("q5_k", "gemv", "bf16", out)]
        single(dx["bf16"].ptr, dw["q5_k"].ptr, sa.ptr, rows, k, n)
        single(dx["bf16"].ptr, dwb.ptr, sb.ptr, rows, k, nb)
        assert np.array_equal(dev.get(da, np.uint8, (rows * n * item,)), dev.get(sa, np.uint8, (rows * n * item,))), variant
        assert np.array_equal(dev.get(db, np.uint8, (rows * nb * item,)), dev.get(sb, np.uint8, (rows * nb * item,))), variant
        dev.free(da, db, sa, sb)
    dev.free(dwb, *dw.values(), *dx.values())
