"""GPU parity of the MoE forms through the C ABI: routing index and tile map
(integer, bit-exact against the oracle), the expert-indexed decode GEMV family
and the expert-grouped Q4_K x DS4 MMQ (float32 within max relative error 1e-3 /
cosine 0.99999 of the reference CPU arithmetic on the same quantized
activations), and the whole selected-expert FFN against the reference CPU MoE
(hipengine/kernels/cpu_reference/ops.py:624-678 as restated by the oracle).

The full-chain comparison is against UNQUANTIZED activations, so its gate is the
looser end-to-end one the reference uses for q8_1 paths (cosine, rtol 2e-2;
tests/test_gpu_gguf_q4_k_q8_1_mmq_prefill.py:343-357); the per-stage tests
carry the 1e-3 gate.
"""

from __future__ import annotations

import numpy as np
import pytest

from oracle import gguf_oracle as O
from hipengine_amd.kernels.hip_gfx950.fused import paro_combine as PC
from hipengine_amd.kernels.hip_gfx950.moe import group_scatter as GS
from hipengine_amd.kernels.hip_gfx950.moe import router as RT
from hipengine_amd.kernels.hip_gfx950.quant import gguf_moe as M
from hipengine_amd.kernels.hip_gfx950.quant import gguf_quantize as Q

pytestmark = pytest.mark.gpu

REL_TOL = 1e-3
COS_MIN = 0.99999


def _routing(seed, tokens, top_k, num_experts, bad=False):
    rng = np.random.default_rng(seed)
    sel = np.stack([rng.permutation(num_experts)[:top_k] for _ in range(tokens)]).astype(np.int64)
    w = rng.random((tokens, top_k)).astype(np.float32)
    w /= w.sum(axis=1, keepdims=True)
    if bad and tokens > 2:
        sel[1, 0] = -1
        sel[2, top_k - 1] = num_experts + 3
    return sel, w


def _routing_from_logits(seed, tokens, top_k, num_experts):
    """Routing as the MoE benchmark configuration states it: router logits ~ N(0, 1), top-k of them, softmax
    over the selected logits (the device router's arithmetic, moe/router.hip:628-715)."""
    logits = np.random.default_rng(seed).standard_normal((tokens, num_experts)).astype(np.float32)
    return O.router_topk_softmax(logits, top_k)


def _device_index(dev, sel, w, num_experts, tile_capacity=0):
    """Runs compact_active_source_rows + mmq32_tile_map + lane_to_compact; returns host copies and device buffers."""
    tokens, top_k = sel.shape
    lanes = tokens * top_k
    d = {
        "sel": dev.put(sel), "w": dev.put(w),
        "expert_start": dev.empty((num_experts + 1) * 8), "active": dev.empty(num_experts * 8, fill=0xFF),
        "active_count": dev.empty(8), "sorted_lanes": dev.empty(lanes * 8, fill=0xFF),
        "c2s": dev.empty(lanes * 8, fill=0xFF), "sorted_w": dev.empty(lanes * 4, fill=0),
    }
    GS.qwen35_moe_group_compact_active_source_rows(d["sel"].ptr, d["w"].ptr, d["expert_start"].ptr, d["active"].ptr,
                                                   d["active_count"].ptr, d["sorted_lanes"].ptr, d["c2s"].ptr,
                                                   d["sorted_w"].ptr, lanes, num_experts, top_k)
    host = {
        "expert_start": dev.get(d["expert_start"], np.int64, (num_experts + 1,)),
        "active": dev.get(d["active"], np.int64, (num_experts,)),
        "active_count": int(dev.get(d["active_count"], np.int64, (1,))[0]),
        "sorted_lanes": dev.get(d["sorted_lanes"], np.int64, (lanes,)),
        "c2s": dev.get(d["c2s"], np.int64, (lanes,)),
        "sorted_w": dev.get(d["sorted_w"], np.float32, (lanes,)),
    }
    total = int(host["expert_start"][-1])
    max_tiles = (lanes + 31) // 32 + num_experts
    cap = tile_capacity or max_tiles
    d["mmq_start"] = dev.empty((num_experts + 1) * 8)
    d["tile_expert"] = dev.empty(cap * 8, fill=0x11)
    d["mmq_total"] = dev.empty(8)
    GS.qwen35_moe_mmq32_tile_map(d["expert_start"].ptr, d["mmq_start"].ptr, d["tile_expert"].ptr, d["mmq_total"].ptr,
                                 num_experts, tile_capacity=cap)
    host["mmq_start"] = dev.get(d["mmq_start"], np.int64, (num_experts + 1,))
    host["tile_expert"] = dev.get(d["tile_expert"], np.int64, (cap,))
    host["mmq_total"] = int(dev.get(d["mmq_total"], np.int64, (1,))[0])
    d["l2c"] = dev.empty(lanes * 8, fill=0x22)
    if total > 0:
        GS.moe_lane_to_compact(d["sorted_lanes"].ptr, d["l2c"].ptr, total, lanes)
        host["l2c"] = dev.get(d["l2c"], np.int64, (lanes,))
    host["total"] = total
    # the combined entry: the same index and the inverse in two launches
    es2, sl2, c2s2, sw2 = dev.empty((num_experts + 1) * 8), dev.empty(lanes * 8, fill=0xFF), dev.empty(lanes * 8, fill=0xFF), dev.empty(lanes * 4, fill=0)
    act2, actn2, l2c2 = dev.empty(num_experts * 8, fill=0xFF), dev.empty(8), dev.empty(lanes * 8, fill=0x22)
    GS.moe_group_compact_index(d["sel"].ptr, d["w"].ptr, es2.ptr, act2.ptr, actn2.ptr, sl2.ptr, c2s2.ptr, sw2.ptr, l2c2.ptr,
                               lanes, num_experts, top_k)
    assert np.array_equal(dev.get(es2, np.int64, (num_experts + 1,)), host["expert_start"])
    assert np.array_equal(dev.get(sl2, np.int64, (lanes,))[:total], host["sorted_lanes"][:total])
    assert np.array_equal(dev.get(c2s2, np.int64, (lanes,))[:total], host["c2s"][:total])
    assert np.array_equal(dev.get(sw2, np.float32, (lanes,))[:total].view(np.uint32), host["sorted_w"][:total].view(np.uint32))
    if total > 0:
        assert np.array_equal(dev.get(l2c2, np.int64, (lanes,)), host["l2c"])
    dev.free(es2, sl2, c2s2, sw2, act2, actn2, l2c2)
    return host, d


@pytest.mark.parametrize("tokens,top_k,experts,bad", [(1, 8, 256, False), (300, 4, 64, True), (77, 2, 5, True)])
def test_routing_index_other_entry_names(dev, tokens, top_k, experts, bad):
    """hipEngine's other names for the same index, each against the oracle's arrays: the "parallel" compactions (int64
    and int32 expert ids), the prefix with the active list from counts in memory, the scatter from given starts
    (ascending lanes; offsets end as the counts), and the tile maps of 16- and 64-row tiles."""
    sel, w = _routing(tokens + experts, tokens, top_k, experts, bad)
    want = O.build_routing_index(sel, w, experts)
    total, lanes = want["total"], tokens * top_k
    dsel, dsel32, dw = dev.put(sel), dev.put(sel.astype(np.int32)), dev.put(w)

    def outputs():
        return {"es": dev.empty((experts + 1) * 8), "act": dev.empty(experts * 8, fill=0xFF), "actn": dev.empty(8),
                "sl": dev.empty(lanes * 8, fill=0xFF), "aux": dev.empty(lanes * 8, fill=0xFF), "sw": dev.empty(lanes * 4)}

    def check(o, aux_want):
        assert np.array_equal(dev.get(o["es"], np.int64, (experts + 1,)), want["expert_start"])
        assert int(dev.get(o["actn"], np.int64, (1,))[0]) == want["active_count"]
        assert np.array_equal(dev.get(o["act"], np.int64, (experts,))[:want["active_count"]], want["active_experts"])
        assert np.array_equal(dev.get(o["sl"], np.int64, (lanes,))[:total], want["sorted_lanes"])
        assert np.array_equal(dev.get(o["aux"], np.int64, (lanes,))[:total], aux_want)
        assert np.array_equal(dev.get(o["sw"], np.float32, (lanes,))[:total].view(np.uint32),
                              want["sorted_weights"].view(np.uint32))
        dev.free(*o.values())

    sorted_experts = sel.reshape(-1)[want["sorted_lanes"]]
    o = outputs()
    GS.qwen35_moe_group_compact_active_parallel(dsel.ptr, dw.ptr, o["es"].ptr, o["act"].ptr, o["actn"].ptr, o["sl"].ptr,
                                                o["aux"].ptr, o["sw"].ptr, lanes, experts)
    check(o, sorted_experts)
    o = outputs()
    GS.qwen35_moe_group_compact_active_i32_parallel(dsel32.ptr, dw.ptr, o["es"].ptr, o["act"].ptr, o["actn"].ptr,
                                                    o["sl"].ptr, o["aux"].ptr, o["sw"].ptr, lanes, experts)
    check(o, sorted_experts)
    o = outputs()
    GS.qwen35_moe_group_compact_active_source_rows_parallel(dsel.ptr, dw.ptr, o["es"].ptr, o["act"].ptr, o["actn"].ptr,
                                                            o["sl"].ptr, o["aux"].ptr, o["sw"].ptr, lanes, experts, top_k)
    check(o, want["compact_to_source"])

    # count -> prefix with the active list -> scatter from the starts
    o = outputs()
    counts, offsets = dev.empty(experts * 4, fill=0), dev.empty(experts * 4, fill=0)
    GS.qwen35_moe_group_count(dsel.ptr, counts.ptr, lanes, experts)
    GS.qwen35_moe_group_prefix_active(counts.ptr, o["es"].ptr, o["act"].ptr, o["actn"].ptr, experts)
    GS.qwen35_moe_group_scatter(dsel.ptr, dw.ptr, o["es"].ptr, offsets.ptr, o["sl"].ptr, o["aux"].ptr, o["sw"].ptr,
                                lanes, experts)
    assert np.array_equal(dev.get(offsets, np.int32, (experts,)), np.diff(want["expert_start"]).astype(np.int32))
    es_dev = o["es"]
    for rows, fn in ((16, GS.qwen35_moe_wmma_tile_map), (64, GS.qwen35_moe_mmq64_tile_map)):
        cap = lanes // rows + experts + 1
        ts, te, tt = dev.empty((experts + 1) * 8), dev.empty(cap * 8, fill=0x11), dev.empty(8)
        fn(es_dev.ptr, ts.ptr, te.ptr, tt.ptr, experts, tile_capacity=cap)
        tm = O.tile_map(want["expert_start"], experts, rows, cap)
        assert np.array_equal(dev.get(ts, np.int64, (experts + 1,)), tm["tile_expert_start"])
        assert np.array_equal(dev.get(te, np.int64, (cap,)), tm["tile_expert"])
        assert int(dev.get(tt, np.int64, (1,))[0]) == tm["total"]
        dev.free(ts, te, tt)
    check(o, sorted_experts)
    dev.free(dsel, dsel32, dw, counts, offsets)


@pytest.mark.parametrize("tokens,hidden,rows", [(1, 2048, 256), (9, 2048, 257), (130, 512, 60), (3, 20, 5), (7, 1024, 64),
                                                (300, 2048, 256), (33, 192, 40), (64, 1000, 33), (40, 77, 19), (2, 3, 9)])
@pytest.mark.parametrize("name,hk,wk", [("bf16", "bf16", "bf16"), ("fp16", "fp16", "fp16"), ("bf16_f32w", "bf16", "f32"),
                                        ("fp16_f32w", "fp16", "f32"), ("f32_f32w", "f32", "f32")])
def test_router_logits(dev, name, hk, wk, tokens, hidden, rows):
    """Router logits against the float32 matmul of the reference on the same (rounded) values: float32 rounding apart
    (another summation order); then the selection of the device logits is the oracle's selection of those logits."""
    rng = np.random.default_rng(tokens + hidden + rows)
    x = (rng.standard_normal((tokens, hidden)) * 0.5).astype(np.float32)
    w = (rng.standard_normal((rows, hidden)) * 0.05).astype(np.float32)

    def encode(a, kind):
        if kind == "bf16":
            b = O.f32_to_bf16_bits(a)
            return b, O.bf16_bits_to_f32(b)
        if kind == "fp16":
            h = a.astype(np.float16)
            return h.view(np.uint16), h.astype(np.float32)
        return a, a

    xb, xf = encode(x, hk)
    wb, wf = encode(w, wk)
    dx, dw, dl = dev.put(xb), dev.put(wb), dev.empty(tokens * rows * 4, fill=0x7C)
    getattr(RT, f"qwen35_router_logits_{name}")(dx.ptr, dw.ptr, dl.ptr, tokens, hidden, rows)
    got = dev.get(dl, np.float32, (tokens, rows)).copy()
    want = O.router_logits(xf, wf)
    exact = xf.astype(np.float64) @ wf.astype(np.float64).T
    scale = np.abs(xf).astype(np.float64) @ np.abs(wf).astype(np.float64).T
    assert np.all(np.abs(got - exact) <= scale * 2.0 ** -20 + 1e-30)          # float32 accumulation of `hidden` terms
    assert np.all(np.abs(want - exact) <= scale * 2.0 ** -20 + 1e-30)
    if rows >= 8:
        top_k = 8
        dsel, dr = dev.empty(tokens * top_k * 8), dev.empty(tokens * top_k * 4)
        RT.qwen35_router_select(dl.ptr, dsel.ptr, dr.ptr, tokens, rows, rows, top_k)
        sel = dev.get(dsel, np.int64, (tokens, top_k))
        want_sel, _ = O.router_topk_softmax(got, top_k)
        assert np.array_equal(sel, want_sel)
        dev.free(dsel, dr)
    dev.free(dx, dw, dl)


@pytest.mark.parametrize("tokens,experts,top_k,stride", [(1, 256, 8, 256), (7, 256, 8, 257), (33, 60, 4, 64),
                                                        (5, 1024, 16, 1024), (3, 8, 8, 8), (2048, 256, 8, 256)])
def test_router_select(dev, tokens, experts, top_k, stride):
    """Top-k experts bit-exact (order included, equal logits to the lowest index) and the softmax over the
    selected logits within 2 ulp-ish of the oracle (expf differs between libm and the device)."""
    rng = np.random.default_rng(17 + tokens + experts)
    logits = rng.standard_normal((tokens, stride)).astype(np.float32)
    logits[:, experts:] = 1.0e9                     # padding columns must not be read as experts
    logits[0, : min(experts, 6)] = 0.75             # equal logits
    if tokens > 1:
        logits[1, :experts] = -2.5                  # a whole row of equal logits
    if tokens > 2 and experts >= 8:
        logits[2, :experts] = -np.abs(logits[2, :experts]) - 0.5
        logits[2, [5, 1, 6]] = [-0.0, 0.0, -0.0]    # zeros of either sign are equal: lowest index first
    dl = dev.put(logits)
    dsel, dw = dev.empty(tokens * top_k * 8, fill=0xFF), dev.empty(tokens * top_k * 4, fill=0xFF)
    RT.qwen35_router_select(dl.ptr, dsel.ptr, dw.ptr, tokens, stride, experts, top_k)
    sel = dev.get(dsel, np.int64, (tokens, top_k))
    w = dev.get(dw, np.float32, (tokens, top_k))
    dev.free(dl, dsel, dw)
    want_sel, want_w = O.router_topk_softmax(logits[:, :experts], top_k)
    assert np.array_equal(sel, want_sel)
    assert np.allclose(w, want_w, rtol=2e-6, atol=1e-9)
    assert np.allclose(w.sum(axis=1), 1.0, atol=1e-6)


@pytest.mark.parametrize("tokens,top_k,experts,bad", [(1, 8, 256, False), (8, 8, 256, True), (300, 4, 64, True),
                                                      (2048, 8, 256, False), (77, 2, 5, True)])
def test_routing_index_and_tile_map_bit_exact(dev, tokens, top_k, experts, bad):
    sel, w = _routing(tokens + experts, tokens, top_k, experts, bad)
    host, d = _device_index(dev, sel, w, experts)
    want = O.build_routing_index(sel, w, experts)
    total = want["total"]
    assert host["total"] == total
    assert np.array_equal(host["expert_start"], want["expert_start"])
    assert host["active_count"] == want["active_count"]
    assert np.array_equal(host["active"][:want["active_count"]], want["active_experts"])
    assert np.array_equal(host["sorted_lanes"][:total], want["sorted_lanes"])
    assert np.array_equal(host["c2s"][:total], want["compact_to_source"])
    assert np.array_equal(host["sorted_w"][:total].view(np.uint32), want["sorted_weights"].view(np.uint32))
    tm = O.tile_map(want["expert_start"], experts, 32, tile_capacity=host["tile_expert"].size)
    assert np.array_equal(host["mmq_start"], tm["tile_expert_start"])
    assert host["mmq_total"] == tm["total"]
    assert np.array_equal(host["tile_expert"], tm["tile_expert"])
    inv = np.full(tokens * top_k, -1, dtype=np.int64)
    inv[want["sorted_lanes"]] = np.arange(total)
    assert np.array_equal(host["l2c"], inv)
    dev.free(*d.values())


def _experts(qt, num_experts, n, k, seed):
    return O.stack_experts(O.random_weight(qt, n, k, seed=seed), num_experts, seed=seed % 7)


def _ref_lane(x_row, w_e, qt):
    """Reference CPU GEMV (dequantize -> float32 matmul) on the q8_1-dequantized activations."""
    xq = O.quantize_q8_1(x_row[None, :])
    return O.gguf_quant_gemv(O.dequantize_q8_1(xq), w_e, qt)[0]


@pytest.mark.parametrize("quant,qt", [("gguf_q4_k", O.GGML_Q4_K), ("gguf_q6_k", O.GGML_Q6_K), ("gguf_q5_k", O.GGML_Q5_K),
                                      ("gguf_q8_0", O.GGML_Q8_0)])
@pytest.mark.parametrize("tokens,top_k,experts,k,n", [(1, 8, 16, 2048, 512), (3, 4, 8, 512, 2048), (5, 2, 6, 1280, 80)])
def test_selected_gemv_single(dev, quant, qt, tokens, top_k, experts, k, n):
    sel, _ = _routing(k + n, tokens, top_k, experts)
    if tokens > 1:
        sel[1, 0] = -1                                   # an invalid lane stays unwritten
    w = (O.stack_experts(_random_q5_k(n, k, seed=3), experts, seed=3) if qt == O.GGML_Q5_K
         else _experts(qt, experts, n, k, seed=3))
    x = np.random.default_rng(9).standard_normal((tokens, k)).astype(np.float32)
    lanes = tokens * top_k
    dx, dsel, dw = dev.put(x), dev.put(sel), dev.put(w)
    dout = dev.empty(lanes * n * 4, fill=0x7F)
    M.gguf_selected_gemv(quant, M.SEL_SINGLE, dx.ptr, dsel.ptr, dw.ptr, dout.ptr, tokens, lanes, experts, k, n)
    got = dev.get(dout, np.float32, (lanes, n))
    dev.free(dx, dsel, dw, dout)
    sentinel = np.frombuffer(b"\x7f\x7f\x7f\x7f", dtype=np.uint32)[0]
    for lane in range(lanes):
        e = int(sel.reshape(-1)[lane])
        if e < 0:
            assert np.all(got[lane].view(np.uint32) == sentinel)
            continue
        ref = _ref_lane(x[lane // top_k], w[e], qt)
        assert O.max_rel_err(got[lane], ref) <= REL_TOL and O.cosine(got[lane], ref) >= COS_MIN


def test_selected_gemv_bf16_entry_points(dev):
    tokens, top_k, experts, k, n = 2, 8, 12, 2048, 512
    sel, _ = _routing(4, tokens, top_k, experts)
    wg, wu = _experts(O.GGML_Q4_K, experts, n, k, seed=5), _experts(O.GGML_Q4_K, experts, n, k, seed=6)
    x = (np.random.default_rng(2).standard_normal((tokens, k)) * 0.5).astype(np.float32)
    xb = O.f32_to_bf16_bits(x)
    xf = O.bf16_bits_to_f32(xb)
    lanes = tokens * top_k
    dx, dsel, dg, du = dev.put(xb), dev.put(sel), dev.put(wg), dev.put(wu)
    dout = dev.empty(lanes * n * 2)
    M.gguf_q4_k_selected_gemv_bf16_bf16_out(dx.ptr, dsel.ptr, dg.ptr, dout.ptr, tokens, lanes, experts, k, n)
    single = O.bf16_bits_to_f32(dev.get(dout, np.uint16, (lanes, n)))
    M.gguf_q4_k_selected_dual_silu_gemv_bf16_bf16_out(dx.ptr, dsel.ptr, dg.ptr, du.ptr, dout.ptr, tokens, lanes,
                                                      experts, k, n)
    dual = O.bf16_bits_to_f32(dev.get(dout, np.uint16, (lanes, n)))
    dev.free(dx, dsel, dg, du, dout)
    for lane in range(lanes):
        e = int(sel.reshape(-1)[lane])
        g = _ref_lane(xf[lane // top_k], wg[e], O.GGML_Q4_K)
        u = _ref_lane(xf[lane // top_k], wu[e], O.GGML_Q4_K)
        # bf16 outputs: half a bf16 ulp (2^-9) on top of the float32 gate
        assert O.max_rel_err(single[lane], g, floor_frac=1e-2) <= 6e-3
        gb = O.bf16_bits_to_f32(O.f32_to_bf16_bits(g))
        ub = O.bf16_bits_to_f32(O.f32_to_bf16_bits(u))
        want = (O.silu(gb) * ub).astype(np.float32)
        assert O.cosine(dual[lane], want) >= 0.9999
        assert O.max_rel_err(dual[lane], want, floor_frac=2e-2) <= 2e-2


def _random_q5_k(n, k, seed):
    rng = np.random.default_rng(seed)
    nblk = n * (k // 256)
    blk = O.pack_q5_k_blocks(rng.integers(0, 32, size=(nblk, 8, 32), dtype=np.uint8),
                             rng.integers(0, 64, size=(nblk, 8), dtype=np.uint8),
                             rng.integers(0, 64, size=(nblk, 8), dtype=np.uint8),
                             (rng.random(nblk) * 0.05).astype(np.float32), (rng.random(nblk) * 0.02).astype(np.float32))
    return blk.reshape(n, -1)


@pytest.mark.parametrize("quant,qt", [("q5_k", O.GGML_Q5_K), ("q6_k", O.GGML_Q6_K), ("q8_0", O.GGML_Q8_0)])
@pytest.mark.parametrize("tokens,top_k,experts,k,n", [(1, 8, 12, 512, 2048), (3, 4, 6, 2048, 272), (2, 2, 5, 4352, 40)])
def test_selected_gemv_and_silu_down_for_other_expert_types(dev, quant, qt, tokens, top_k, experts, k, n):
    """gguf_<q>_selected_gemv_bf16_bf16_out and gguf_<q>_selected_silu_gemv_bf16_bf16_out for Q5_K / Q6_K / Q8_0
    experts: the plain projection over `tokens` rows fanned out to tokens * top_k lanes, and the down projection
    whose activation is bf16(silu(gate) * up) of the lane's own row (x_rows == rows)."""
    rng = np.random.default_rng(k + n + tokens)
    sel, _ = _routing(k + n, tokens, top_k, experts)
    if tokens > 1:
        sel[1, 0] = experts                              # an invalid lane stays unwritten
    base = _random_q5_k(n, k, seed=8) if qt == O.GGML_Q5_K else O.random_weight(qt, n, k, seed=8)
    w = O.stack_experts(base, experts, seed=2)
    lanes = tokens * top_k
    single, silu = M.SELECTED_K[quant]
    dsel, dw = dev.put(sel), dev.put(w)

    xb = O.f32_to_bf16_bits((rng.standard_normal((tokens, k)) * 0.5).astype(np.float32))
    dx = dev.put(xb)
    dout = dev.empty(lanes * n * 2, fill=0x7F)
    single(dx.ptr, dsel.ptr, dw.ptr, dout.ptr, tokens, lanes, experts, k, n)
    got_single = dev.get(dout, np.uint16, (lanes, n))
    dev.free(dx, dout)

    gate = O.f32_to_bf16_bits((rng.standard_normal((lanes, k)) * 1.5).astype(np.float32))
    up = O.f32_to_bf16_bits(rng.standard_normal((lanes, k)).astype(np.float32))
    dg, du = dev.put(gate), dev.put(up)
    dout = dev.empty(lanes * n * 2, fill=0x7F)
    silu(dg.ptr, du.ptr, dsel.ptr, dw.ptr, dout.ptr, lanes, lanes, experts, k, n)
    got_silu = dev.get(dout, np.uint16, (lanes, n))
    dev.free(dg, du, dout, dsel, dw)

    xf = O.bf16_bits_to_f32(xb)
    act = O.bf16_bits_to_f32(O.f32_to_bf16_bits(O.silu(O.bf16_bits_to_f32(gate)) * O.bf16_bits_to_f32(up)))
    for lane in range(lanes):
        e = int(sel.reshape(-1)[lane])
        if e >= experts:
            assert np.all(got_single[lane] == 0x7F7F) and np.all(got_silu[lane] == 0x7F7F)
            continue
        # bf16 outputs: half a bf16 ulp (2^-9) on top of the float32 gate
        ref = _ref_lane(xf[lane // top_k], w[e], qt)
        assert O.max_rel_err(O.bf16_bits_to_f32(got_single[lane]), ref, floor_frac=1e-2) <= 6e-3
        assert O.cosine(O.bf16_bits_to_f32(got_single[lane]), ref) >= 0.9999
        ref = _ref_lane(act[lane], w[e], qt)
        assert O.max_rel_err(O.bf16_bits_to_f32(got_silu[lane]), ref, floor_frac=1e-2) <= 6e-3
        assert O.cosine(O.bf16_bits_to_f32(got_silu[lane]), ref) >= 0.9999


@pytest.mark.parametrize("tokens,experts", [(1, 32), (8, 32), (1, 256), (8, 256)])
def test_decode_chain_matches_cpu_moe(dev, tokens, experts):
    """dual SiLU GEMV -> routed down sum (two launches) against the reference CPU MoE FFN."""
    top_k, hidden, inter = 8, 2048, 512
    sel, wts = _routing(tokens, tokens, top_k, experts)
    wg = _experts(O.GGML_Q4_K, experts, inter, hidden, seed=1)
    wu = _experts(O.GGML_Q4_K, experts, inter, hidden, seed=2)
    wd = _experts(O.GGML_Q4_K, experts, hidden, inter, seed=3)
    x = (np.random.default_rng(tokens).standard_normal((tokens, hidden)) * 0.3).astype(np.float32)
    lanes = tokens * top_k
    dx, dsel, dwt = dev.put(x), dev.put(sel), dev.put(wts)
    dg, du, dd = dev.put(wg), dev.put(wu), dev.put(wd)
    dmid, dout = dev.empty(lanes * inter * 4), dev.empty(tokens * hidden * 4)
    M.gguf_selected_gemv("gguf_q4_k", M.SEL_DUAL_SILU, dx.ptr, dsel.ptr, dg.ptr, dmid.ptr, tokens, lanes, experts,
                         hidden, inter, qweight_b_ptr=du.ptr)
    M.gguf_selected_gemv("gguf_q4_k", M.SEL_DOWN_SUM, dmid.ptr, dsel.ptr, dd.ptr, dout.ptr, tokens, lanes, experts,
                         inter, hidden, routing_weights_ptr=dwt.ptr, top_k=top_k)
    mid = dev.get(dmid, np.float32, (lanes, inter))
    got = dev.get(dout, np.float32, (tokens, hidden))
    dev.free(dx, dsel, dwt, dg, du, dd, dmid, dout)
    # stage gates: each stage against the reference arithmetic on the same quantized inputs
    want = np.zeros((tokens, hidden), dtype=np.float32)
    for lane in range(lanes):
        t, e = lane // top_k, int(sel.reshape(-1)[lane])
        g, u = _ref_lane(x[t], wg[e], O.GGML_Q4_K), _ref_lane(x[t], wu[e], O.GGML_Q4_K)
        ref_mid = (O.silu(g) * u).astype(np.float32)
        assert O.max_rel_err(mid[lane], ref_mid) <= REL_TOL and O.cosine(mid[lane], ref_mid) >= COS_MIN
        want[t] += wts.reshape(-1)[lane] * _ref_lane(mid[lane], wd[e], O.GGML_Q4_K)
    assert O.max_rel_err(got, want) <= REL_TOL and O.cosine(got, want) >= COS_MIN
    # end to end against the reference CPU MoE on unquantized activations
    ref = O.moe_selected_ffn(x, sel, wts, wg, wu, wd)
    assert O.cosine(got, ref) >= 0.9995
    np.testing.assert_allclose(got, ref, rtol=2e-2, atol=2e-2 * np.abs(ref).max())


@pytest.mark.parametrize("quant,qt", [("gguf_q5_k", O.GGML_Q5_K), ("gguf_q6_k", O.GGML_Q6_K), ("gguf_q8_0", O.GGML_Q8_0)])
@pytest.mark.parametrize("tokens,hidden,inter", [(1, 1024, 512), (5, 4096, 256), (8, 2048, 768)])
def test_decode_chain_for_other_expert_types(dev, quant, qt, tokens, hidden, inter):
    """The two-launch decode chain (gate/up with SiLU, routed down sum) for Q5_K, Q6_K and Q8_0 experts: each stage
    against the reference arithmetic on the same quantized inputs (4, 16 and 8 blocks per gate/up row: one block and
    two blocks per lane and K slice)."""
    top_k, experts = 8, 12
    sel, wts = _routing(tokens + hidden, tokens, top_k, experts)
    make = ((lambda n, k, seed: O.stack_experts(_random_q5_k(n, k, seed), experts, seed=seed % 5)) if qt == O.GGML_Q5_K
            else (lambda n, k, seed: _experts(qt, experts, n, k, seed=seed)))
    wg, wu, wd = make(inter, hidden, 1), make(inter, hidden, 2), make(hidden, inter, 3)
    x = (np.random.default_rng(tokens).standard_normal((tokens, hidden)) * 0.3).astype(np.float32)
    lanes = tokens * top_k
    dx, dsel, dwt = dev.put(x), dev.put(sel), dev.put(wts)
    dg, du, dd = dev.put(wg), dev.put(wu), dev.put(wd)
    dmid, dout = dev.empty(lanes * inter * 4), dev.empty(tokens * hidden * 4)
    M.gguf_selected_gemv(quant, M.SEL_DUAL_SILU, dx.ptr, dsel.ptr, dg.ptr, dmid.ptr, tokens, lanes, experts,
                         hidden, inter, qweight_b_ptr=du.ptr)
    M.gguf_selected_gemv(quant, M.SEL_DOWN_SUM, dmid.ptr, dsel.ptr, dd.ptr, dout.ptr, tokens, lanes, experts,
                         inter, hidden, routing_weights_ptr=dwt.ptr, top_k=top_k)
    mid = dev.get(dmid, np.float32, (lanes, inter))
    got = dev.get(dout, np.float32, (tokens, hidden))
    dev.free(dx, dsel, dwt, dg, du, dd, dmid, dout)
    want = np.zeros((tokens, hidden), dtype=np.float32)
    for lane in range(lanes):
        t, e = lane // top_k, int(sel.reshape(-1)[lane])
        g, u = _ref_lane(x[t], wg[e], qt), _ref_lane(x[t], wu[e], qt)
        ref_mid = (O.silu(g) * u).astype(np.float32)
        assert O.max_rel_err(mid[lane], ref_mid) <= REL_TOL and O.cosine(mid[lane], ref_mid) >= COS_MIN
        want[t] += wts.reshape(-1)[lane] * _ref_lane(mid[lane], wd[e], qt)
    assert O.max_rel_err(got, want) <= REL_TOL and O.cosine(got, want) >= COS_MIN


def _grouped(dev, host, d, ds4, w_a, w_b, rows_src, k, na, nb, experts, identity=False, out_dtype="f32"):
    total = host["total"]
    dxq, dwa = dev.put(ds4), dev.put(w_a)
    dwb = dev.put(w_b) if w_b is not None else None
    item = 4 if out_dtype == "f32" else 2
    dout = dev.empty(total * (na + nb) * item, fill=0)
    M.gguf_q4_k_grouped_mmq(dxq.ptr, d["expert_start"].ptr, d["mmq_start"].ptr, d["tile_expert"].ptr, dwa.ptr, dout.ptr,
                            total, rows_src, k, na, experts, host["mmq_total"],
                            compact_to_source_ptr=0 if identity else d["c2s"].ptr,
                            qweight_b_ptr=dwb.ptr if dwb else 0, out_features_b=nb, out_dtype=out_dtype)
    got = dev.get(dout, np.float32 if out_dtype == "f32" else np.uint16, (total, na + nb))
    dev.free(dxq, dwa, dout, *([dwb] if dwb else []))
    return got


@pytest.mark.parametrize("tokens,top_k,experts,k,na,nb", [(40, 4, 8, 512, 96, 64), (150, 8, 16, 2048, 512, 512),
                                                          (9, 2, 40, 768, 288, 0)])
def test_grouped_mmq_matches_dense_formula_per_expert(dev, tokens, top_k, experts, k, na, nb):
    sel, wts = _routing(tokens * 3 + k, tokens, top_k, experts, bad=tokens > 20)
    host, d = _device_index(dev, sel, wts, experts)
    x = (np.random.default_rng(k).standard_normal((tokens, k)) * 0.2).astype(np.float32)
    ds4 = O.pack_q8_1_ds4(O.f32_to_bf16_bits(x))
    w_a = _experts(O.GGML_Q4_K, experts, na, k, seed=11)
    w_b = _experts(O.GGML_Q4_K, experts, nb, k, seed=12) if nb else None
    got = _grouped(dev, host, d, ds4, w_a, w_b, tokens, k, na, nb, experts)
    es = host["expert_start"]
    for e in range(experts):
        lo, hi = int(es[e]), int(es[e + 1])
        if hi == lo:
            continue
        src = host["c2s"][lo:hi]
        want_a = O.mmq_q4_k_ds4(ds4[src], w_a[e])
        assert O.max_rel_err(got[lo:hi, :na], want_a) <= REL_TOL and O.cosine(got[lo:hi, :na], want_a) >= COS_MIN
        if nb:
            want_b = O.mmq_q4_k_ds4(ds4[src], w_b[e])
            assert O.max_rel_err(got[lo:hi, na:], want_b) <= REL_TOL and O.cosine(got[lo:hi, na:], want_b) >= COS_MIN
    dev.free(*d.values())


@pytest.mark.parametrize("tokens,top_k,experts,k,na,nb,identity", [
    (40, 4, 8, 512, 96, 40, False),        # ragged widths, experts of a few rows
    (300, 4, 6, 1024, 200, 0, False),      # experts of several 128-row tiles (about 200 rows each)
    (64, 1, 5, 768, 130, 64, True),        # compact rows read as they are (an already gathered intermediate)
])
@pytest.mark.parametrize("quant", ["q6_k", "q8_0"])
def test_grouped_mmq_q6_k_matches_dense_formula_per_expert(dev, quant, tokens, top_k, experts, k, na, nb, identity):
    """The expert-grouped MMQ for Q6_K and for Q8_0 experts over D4S4 blocks and a map of 128-row tiles: per expert
    the float64 value of the dense formula on the rows it owns; rows of no expert and tiles past an expert's rows
    stay unwritten."""
    qt, run, formula = ((O.GGML_Q6_K, M.gguf_q6_k_grouped_mmq, O.mmq_q6_k_d4s4) if quant == "q6_k"
                        else (O.GGML_Q8_0, M.gguf_q8_0_grouped_mmq, O.mmq_q8_0_d4s4))
    sel, wts = _routing(tokens * 5 + k, tokens, top_k, experts, bad=tokens > 20)
    host, d = _device_index(dev, sel, wts, experts)
    total, lanes = host["total"], tokens * top_k
    rows_src = total if identity else tokens
    x = (np.random.default_rng(k).standard_normal((rows_src, k)) * 0.2).astype(np.float32)
    d4s4 = O.pack_q8_1_d4s4(O.f32_to_bf16_bits(x))
    w_a = _experts(qt, experts, na, k, seed=13)
    w_b = _experts(qt, experts, nb, k, seed=14) if nb else None
    cap = lanes // 128 + experts
    ts, te, tt = dev.empty((experts + 1) * 8), dev.empty(cap * 8, fill=0x11), dev.empty(8)
    GS.moe_tile_map(d["expert_start"].ptr, ts.ptr, te.ptr, tt.ptr, experts, tile_rows=128, tile_capacity=cap)
    want_map = O.tile_map(host["expert_start"], experts, 128, cap)
    assert np.array_equal(dev.get(ts, np.int64, (experts + 1,)), want_map["tile_expert_start"])
    assert np.array_equal(dev.get(te, np.int64, (cap,)), want_map["tile_expert"])
    assert int(dev.get(tt, np.int64, (1,))[0]) == want_map["total"]
    dxq, dwa = dev.put(d4s4), dev.put(w_a)
    dwb = dev.put(w_b) if nb else None
    dout = dev.empty((total + 1) * (na + nb) * 4, fill=0x7D)
    run(dxq.ptr, d["expert_start"].ptr, ts.ptr, te.ptr, dwa.ptr, dout.ptr, total, rows_src, k, na, experts, cap * 128,
        compact_to_source_ptr=0 if identity else d["c2s"].ptr, qweight_b_ptr=dwb.ptr if dwb else 0, out_features_b=nb)
    got = dev.get(dout, np.float32, (total + 1, na + nb))
    dev.free(dxq, dwa, dout, ts, te, tt, *([dwb] if dwb else []))
    assert np.all(got[total].view(np.uint32) == 0x7D7D7D7D)
    es = host["expert_start"]
    for e in range(experts):
        lo, hi = int(es[e]), int(es[e + 1])
        if hi == lo:
            continue
        src = np.arange(lo, hi) if identity else host["c2s"][lo:hi]
        want_a = formula(d4s4[src], w_a[e])
        assert O.max_rel_err(got[lo:hi, :na], want_a) <= REL_TOL and O.cosine(got[lo:hi, :na], want_a) >= COS_MIN
        if nb:
            want_b = formula(d4s4[src], w_b[e])
            assert O.max_rel_err(got[lo:hi, na:], want_b) <= REL_TOL and O.cosine(got[lo:hi, na:], want_b) >= COS_MIN
    dev.free(*d.values())


@pytest.mark.parametrize("tokens,top_k,experts,k,na,nb", [(40, 4, 8, 512, 96, 64), (120, 8, 12, 1024, 288, 0)])
def test_grouped_mmq_q5_k_matches_dense_formula_per_expert(dev, tokens, top_k, experts, k, na, nb):
    """The expert-grouped MMQ for Q5_K experts over D4S4 blocks (the 32-row tile map of the Q4_K one): per expert the
    float64 value of the dense Q5_K x D4S4 formula on the rows it owns."""
    sel, wts = _routing(tokens * 7 + k, tokens, top_k, experts, bad=True)
    host, d = _device_index(dev, sel, wts, experts)
    total = host["total"]
    x = (np.random.default_rng(k + 1).standard_normal((tokens, k)) * 0.2).astype(np.float32)
    d4s4 = O.pack_q8_1_d4s4(O.f32_to_bf16_bits(x))
    w_a = O.stack_experts(_random_q5_k(na, k, seed=21), experts, seed=2)
    w_b = O.stack_experts(_random_q5_k(nb, k, seed=22), experts, seed=3) if nb else None
    dxq, dwa = dev.put(d4s4), dev.put(w_a)
    dwb = dev.put(w_b) if nb else None
    dout = dev.empty((total + 1) * (na + nb) * 4, fill=0x7D)
    M.gguf_q5_k_grouped_mmq(dxq.ptr, d["expert_start"].ptr, d["mmq_start"].ptr, d["tile_expert"].ptr, dwa.ptr, dout.ptr,
                            total, tokens, k, na, experts, host["mmq_total"], compact_to_source_ptr=d["c2s"].ptr,
                            qweight_b_ptr=dwb.ptr if dwb else 0, out_features_b=nb)
    got = dev.get(dout, np.float32, (total + 1, na + nb))
    dev.free(dxq, dwa, dout, *([dwb] if dwb else []))
    assert np.all(got[total].view(np.uint32) == 0x7D7D7D7D)
    es = host["expert_start"]
    for e in range(experts):
        lo, hi = int(es[e]), int(es[e + 1])
        if hi == lo:
            continue
        src = host["c2s"][lo:hi]
        want_a = O.mmq_q5_k_d4s4(d4s4[src], w_a[e])
        assert O.max_rel_err(got[lo:hi, :na], want_a) <= REL_TOL and O.cosine(got[lo:hi, :na], want_a) >= COS_MIN
        if nb:
            want_b = O.mmq_q5_k_d4s4(d4s4[src], w_b[e])
            assert O.max_rel_err(got[lo:hi, na:], want_b) <= REL_TOL and O.cosine(got[lo:hi, na:], want_b) >= COS_MIN
    dev.free(*d.values())


def test_silu_mul_d4s4_pack_bytes(dev):
    """SiLU * up fused with the D4S4 pack: the bytes of the two-step path (SiLU * up to bf16, then the pack)."""
    rows, inter = 37, 384
    rng = np.random.default_rng(5)
    gu = O.f32_to_bf16_bits((rng.standard_normal((rows, 2 * inter)) * 1.5).astype(np.float32))
    dgu = dev.put(gu)
    mid, want, got = dev.empty(rows * inter * 2), dev.empty(rows * (inter // 128) * 160), dev.empty(rows * (inter // 128) * 160)
    M.moe_silu_mul(dgu.ptr, mid.ptr, rows, inter, in_dtype="bf16", out_dtype="bf16")
    Q.gguf_q8_1_d4s4_f32_quantize_bf16(mid.ptr, want.ptr, rows, inter)
    M.moe_silu_mul_d4s4_pack(dgu.ptr, got.ptr, rows, inter, in_dtype="bf16")
    a, b = dev.get(got, np.uint8, (rows, inter // 128, 160)), dev.get(want, np.uint8, (rows, inter // 128, 160))
    dev.free(dgu, mid, want, got)
    assert np.array_equal(a, b)


def test_grouped_mmq_bf16_named_entry(dev):
    tokens, top_k, experts, k, na, nb = 64, 4, 8, 1024, 128, 128
    sel, wts = _routing(31, tokens, top_k, experts)
    host, d = _device_index(dev, sel, wts, experts)
    x = (np.random.default_rng(1).standard_normal((tokens, k)) * 0.2).astype(np.float32)
    ds4 = O.pack_q8_1_ds4(O.f32_to_bf16_bits(x))
    w_a, w_b = _experts(O.GGML_Q4_K, experts, na, k, seed=21), _experts(O.GGML_Q4_K, experts, nb, k, seed=22)
    f32 = _grouped(dev, host, d, ds4, w_a, w_b, tokens, k, na, nb, experts)
    total = host["total"]
    dxq, dwa, dwb = dev.put(ds4), dev.put(w_a), dev.put(w_b)
    dout = dev.empty(total * (na + nb) * 2, fill=0)
    M.gguf_q4_k_selected_dual_q8_1_ds4_mmq32_prefill_compact32_bf16_bf16_out(
        dxq.ptr, d["c2s"].ptr, d["expert_start"].ptr, d["mmq_start"].ptr, d["tile_expert"].ptr, dwa.ptr, dwb.ptr,
        dout.ptr, total, k, na, nb, experts, host["mmq_total"])
    b16 = dev.get(dout, np.uint16, (total, na + nb)).copy()
    dev.runtime.memset(dout.ptr, 0, total * (na + nb) * 2)
    M.gguf_q4_k_selected_dual_q8_1_ds4_mmq32x128_prefill_compact32_bf16_bf16_out(
        dxq.ptr, d["c2s"].ptr, d["expert_start"].ptr, d["mmq_start"].ptr, d["tile_expert"].ptr, dwa.ptr, dwb.ptr,
        dout.ptr, total, k, na, nb, experts, host["mmq_total"])
    wide = dev.get(dout, np.uint16, (total, na + nb)).copy()
    dev.free(dxq, dwa, dwb, dout, *d.values())
    assert np.array_equal(b16, O.f32_to_bf16_bits(f32))
    assert np.array_equal(wide, b16)              # hipEngine's 32 x 128 variant name: the same GEMM


def test_grouped_mmq_named_entry_with_mostly_dropped_lanes(dev):
    """Most lanes name no expert, so there are fewer compact rows than tokens: under hipEngine's name (which has
    no source row count) the last tokens' rows must still be the ones their compact_to_source entries name."""
    tokens, top_k, experts, k, na, nb = 64, 2, 4, 512, 64, 32
    rng = np.random.default_rng(41)
    sel = np.full((tokens, top_k), -1, dtype=np.int64)
    keep = [3, 17, 40, 58, 61, 63]                       # 6 tokens keep one lane each: 6 compact rows, source rows up to 63
    for i, t in enumerate(keep):
        sel[t, i % top_k] = i % experts
    wts = np.full((tokens, top_k), 0.5, dtype=np.float32)
    host, d = _device_index(dev, sel, wts, experts)
    total = host["total"]
    assert total == len(keep) and int(host["c2s"][:total].max()) >= total
    x = (rng.standard_normal((tokens, k)) * 0.2).astype(np.float32)
    ds4 = O.pack_q8_1_ds4(O.f32_to_bf16_bits(x))
    w_a, w_b = _experts(O.GGML_Q4_K, experts, na, k, seed=23), _experts(O.GGML_Q4_K, experts, nb, k, seed=24)
    dxq, dwa, dwb = dev.put(ds4), dev.put(w_a), dev.put(w_b)
    dout = dev.empty(total * (na + nb) * 2, fill=0)
    M.gguf_q4_k_selected_dual_q8_1_ds4_mmq32_prefill_compact32_bf16_bf16_out(
        dxq.ptr, d["c2s"].ptr, d["expert_start"].ptr, d["mmq_start"].ptr, d["tile_expert"].ptr, dwa.ptr, dwb.ptr,
        dout.ptr, total, k, na, nb, experts, host["mmq_total"])
    got = O.bf16_bits_to_f32(dev.get(dout, np.uint16, (total, na + nb)).copy())
    dev.free(dxq, dwa, dwb, dout, *d.values())
    es = host["expert_start"]
    for e in range(experts):
        lo, hi = int(es[e]), int(es[e + 1])
        if hi > lo:
            src = host["c2s"][lo:hi]
            want = np.concatenate([O.mmq_q4_k_ds4(ds4[src], w_a[e]), O.mmq_q4_k_ds4(ds4[src], w_b[e])], axis=1)
            assert np.array_equal(O.f32_to_bf16_bits(got[lo:hi]), O.f32_to_bf16_bits(O.bf16_bits_to_f32(O.f32_to_bf16_bits(want)))) or \
                O.max_rel_err(got[lo:hi], want, floor_frac=1e-2) <= 2.0 ** -7


@pytest.mark.parametrize("tokens,experts", [(256, 32), (2048, 256)])
def test_prefill_chain_matches_cpu_moe(dev, tokens, experts):
    """index -> DS4 pack -> grouped gate|up MMQ -> SiLU*up -> DS4 pack -> grouped down MMQ ->
    ordered weighted gather, against the reference CPU MoE FFN on a token subsample."""
    top_k, hidden, inter = 8, 2048, 512
    sel, wts = _routing_from_logits(77, tokens, top_k, experts)
    host, d = _device_index(dev, sel, wts, experts)
    total, lanes = host["total"], tokens * top_k
    wg = _experts(O.GGML_Q4_K, experts, inter, hidden, seed=1)
    wu = _experts(O.GGML_Q4_K, experts, inter, hidden, seed=2)
    wd = _experts(O.GGML_Q4_K, experts, hidden, inter, seed=3)
    x = (np.random.default_rng(8).standard_normal((tokens, hidden)) * 0.3).astype(np.float32)
    xb = O.f32_to_bf16_bits(x)
    dxb, dg, du, dd = dev.put(xb), dev.put(wg), dev.put(wu), dev.put(wd)
    dxq = dev.empty(tokens * (hidden // 128) * 144)
    Q.gguf_q8_1_mmq_ds4_pack_bf16(dxb.ptr, dxq.ptr, tokens, hidden)
    dgu = dev.empty(total * 2 * inter * 4)
    M.gguf_q4_k_grouped_mmq(dxq.ptr, d["expert_start"].ptr, d["mmq_start"].ptr, d["tile_expert"].ptr, dg.ptr, dgu.ptr,
                            total, tokens, hidden, inter, experts, host["mmq_total"], compact_to_source_ptr=d["c2s"].ptr,
                            qweight_b_ptr=du.ptr, out_features_b=inter)
    dmid = dev.empty(total * inter * 2)
    M.moe_silu_mul(dgu.ptr, dmid.ptr, total, inter, in_dtype="f32", out_dtype="bf16")
    dmq = dev.empty(total * (inter // 128) * 144)
    Q.gguf_q8_1_mmq_ds4_pack_bf16(dmid.ptr, dmq.ptr, total, inter)
    two_step = dev.get(dmq, np.uint8, (total, inter // 128, 144)).copy()
    M.moe_silu_mul_ds4_pack(dgu.ptr, dmq.ptr, total, inter, in_dtype="f32")     # the same bytes in one launch
    assert np.array_equal(dev.get(dmq, np.uint8, (total, inter // 128, 144)), two_step)
    ddown = dev.empty(total * hidden * 4)
    M.gguf_q4_k_grouped_mmq(dmq.ptr, d["expert_start"].ptr, d["mmq_start"].ptr, d["tile_expert"].ptr, dd.ptr, ddown.ptr,
                            total, total, inter, hidden, experts, host["mmq_total"])
    dout = dev.empty(tokens * hidden * 4)
    M.moe_weighted_gather_sum(ddown.ptr, d["l2c"].ptr, d["w"].ptr, dout.ptr, tokens, top_k, hidden, total)
    got = dev.get(dout, np.float32, (tokens, hidden))
    gu = dev.get(dgu, np.float32, (total, 2 * inter))
    mid_bits = dev.get(dmid, np.uint16, (total, inter))
    mid = O.bf16_bits_to_f32(mid_bits)
    down = dev.get(ddown, np.float32, (total, hidden))
    dev.free(dxb, dg, du, dd, dxq, dgu, dmid, dmq, ddown, dout, *d.values())
    # gate|up stage: the MMQ formula on the packed activations of each expert's rows, every fifth expert
    x_ds4 = O.pack_q8_1_ds4(xb)
    es, c2s = host["expert_start"], host["c2s"]
    for e in range(0, experts, 5):
        lo, hi = int(es[e]), int(es[e + 1])
        if hi > lo:
            rows_e = x_ds4[c2s[lo:hi]]
            for half, we in ((0, wg[e]), (1, wu[e])):
                want_gu = O.mmq_q4_k_ds4(rows_e, we)
                got_gu = gu[lo:hi, half * inter:(half + 1) * inter]
                assert O.max_rel_err(got_gu, want_gu) <= REL_TOL and O.cosine(got_gu, want_gu) >= COS_MIN
    # elementwise stage: bf16(silu(gate)*up) of the device's own gate|up
    want_mid = O.bf16_bits_to_f32(O.f32_to_bf16_bits((O.silu(gu[:, :inter]) * gu[:, inter:]).astype(np.float32)))
    assert O.max_rel_err(mid, want_mid, floor_frac=1e-2) <= 1e-2
    # down stage: the MMQ formula on the device's own intermediate, expert by expert
    mid_ds4 = O.pack_q8_1_ds4(mid_bits)
    for e in range(0, experts, 5):
        lo, hi = int(es[e]), int(es[e + 1])
        if hi > lo:
            want_down = O.mmq_q4_k_ds4(mid_ds4[lo:hi], wd[e])
            assert O.max_rel_err(down[lo:hi], want_down) <= REL_TOL and O.cosine(down[lo:hi], want_down) >= COS_MIN
    # ordered weighted gather of the device's own down rows
    want_out = np.zeros((tokens, hidden), dtype=np.float64)
    for lane in range(lanes):
        want_out[lane // top_k] += np.float64(wts.reshape(-1)[lane]) * down[host["l2c"][lane]]
    assert O.max_rel_err(got, want_out.astype(np.float32), floor_frac=1e-3) <= 1e-4
    # end to end on a token subsample (the CPU MoE is a Python loop over tokens x slots)
    pick = np.arange(0, tokens, max(16, tokens // 16))
    # (two q8_1 quantizations and a bf16 intermediate separate the two: ~0.4% noise per stage)
    ref = O.moe_selected_ffn(O.bf16_bits_to_f32(xb)[pick], sel[pick], wts[pick], wg, wu, wd)
    assert O.cosine(got[pick], ref) >= 0.999
    np.testing.assert_allclose(got[pick], ref, rtol=2e-2, atol=5e-2 * np.abs(ref).max())
    assert np.all(np.isfinite(got))


def test_prefill_chain_with_bf16_intermediates(dev):
    """The same chain with hipEngine's own intermediate types: gate|up through the named bf16 entry, SiLU*up +
    DS4 pack from bf16, down projection stored as bf16, gather from bf16.  Every stage is held to the float32
    stage on the same inputs (bf16 output = bf16_round(float32 output) bit for bit, packed bytes equal to the
    oracle's), the end to the reference CPU MoE with the gate hipEngine's q8_1 tests use."""
    tokens, experts, top_k, hidden, inter = 96, 16, 8, 2048, 512
    sel, wts = _routing(79, tokens, top_k, experts)
    host, d = _device_index(dev, sel, wts, experts)
    total, lanes = host["total"], tokens * top_k
    wg = _experts(O.GGML_Q4_K, experts, inter, hidden, seed=4)
    wu = _experts(O.GGML_Q4_K, experts, inter, hidden, seed=5)
    wd = _experts(O.GGML_Q4_K, experts, hidden, inter, seed=6)
    x = (np.random.default_rng(9).standard_normal((tokens, hidden)) * 0.3).astype(np.float32)
    xb = O.f32_to_bf16_bits(x)
    dxb, dg, du, dd = dev.put(xb), dev.put(wg), dev.put(wu), dev.put(wd)
    dxq = dev.empty(tokens * (hidden // 128) * 144)
    Q.gguf_q8_1_mmq_ds4_pack_bf16(dxb.ptr, dxq.ptr, tokens, hidden)
    idx = (d["expert_start"].ptr, d["mmq_start"].ptr, d["tile_expert"].ptr)
    # gate|up: named bf16 entry against the float32 form
    dgu32, dgu16 = dev.empty(total * 2 * inter * 4), dev.empty(total * 2 * inter * 2)
    M.gguf_q4_k_grouped_mmq(dxq.ptr, *idx, dg.ptr, dgu32.ptr, total, tokens, hidden, inter, experts, host["mmq_total"],
                            compact_to_source_ptr=d["c2s"].ptr, qweight_b_ptr=du.ptr, out_features_b=inter)
    M.gguf_q4_k_selected_dual_q8_1_ds4_mmq32_prefill_compact32_bf16_bf16_out(
        dxq.ptr, d["c2s"].ptr, *idx, dg.ptr, du.ptr, dgu16.ptr, total, hidden, inter, inter, experts, host["mmq_total"])
    gu16 = dev.get(dgu16, np.uint16, (total, 2 * inter)).copy()
    assert np.array_equal(gu16, O.f32_to_bf16_bits(dev.get(dgu32, np.float32, (total, 2 * inter))))
    # SiLU*up + DS4 pack from the bf16 gate|up: the oracle's bytes
    dmq = dev.empty(total * (inter // 128) * 144)
    M.moe_silu_mul_ds4_pack(dgu16.ptr, dmq.ptr, total, inter, in_dtype="bf16")
    guf = O.bf16_bits_to_f32(gu16)
    mid_bits = O.f32_to_bf16_bits((O.silu(guf[:, :inter]) * guf[:, inter:]).astype(np.float32))
    got_mq = dev.get(dmq, np.uint8, (total, inter // 128, 144)).copy()
    want_mq = O.pack_q8_1_ds4(mid_bits)
    assert np.mean(got_mq != want_mq) < 2e-3          # silu through expf on the device: a few last-place differences
    # down: bf16 store of the float32 result on the same packed intermediate
    ddown32, ddown16 = dev.empty(total * hidden * 4), dev.empty(total * hidden * 2)
    M.gguf_q4_k_grouped_mmq(dmq.ptr, *idx, dd.ptr, ddown32.ptr, total, total, inter, hidden, experts, host["mmq_total"])
    M.gguf_q4_k_grouped_mmq(dmq.ptr, *idx, dd.ptr, ddown16.ptr, total, total, inter, hidden, experts, host["mmq_total"],
                            out_dtype="bf16")
    down16 = dev.get(ddown16, np.uint16, (total, hidden)).copy()
    assert np.array_equal(down16, O.f32_to_bf16_bits(dev.get(ddown32, np.float32, (total, hidden))))
    # ordered weighted gather from bf16 rows
    dout = dev.empty(tokens * hidden * 4)
    M.moe_weighted_gather_sum(ddown16.ptr, d["l2c"].ptr, d["w"].ptr, dout.ptr, tokens, top_k, hidden, total,
                              in_dtype="bf16")
    got = dev.get(dout, np.float32, (tokens, hidden)).copy()
    dev.free(dxb, dg, du, dd, dxq, dgu32, dgu16, dmq, ddown32, ddown16, dout, *d.values())
    downf = O.bf16_bits_to_f32(down16)
    want_out = np.zeros((tokens, hidden), dtype=np.float64)
    for lane in range(lanes):
        want_out[lane // top_k] += np.float64(wts.reshape(-1)[lane]) * downf[host["l2c"][lane]]
    assert O.max_rel_err(got, want_out.astype(np.float32), floor_frac=1e-3) <= 1e-4
    pick = np.arange(0, tokens, 8)
    ref = O.moe_selected_ffn(O.bf16_bits_to_f32(xb)[pick], sel[pick], wts[pick], wg, wu, wd)
    assert O.cosine(got[pick], ref) >= 0.999
    np.testing.assert_allclose(got[pick], ref, rtol=2e-2, atol=5e-2 * np.abs(ref).max())


def test_moe_wrappers_reject_bad_arguments(dev):
    with pytest.raises(ValueError, match="num_experts"):
        GS.qwen35_moe_mmq32_tile_map(1, 1, 1, 1, 0)
    with pytest.raises(ValueError, match="multiple of x_rows"):
        M.gguf_q4_k_selected_gemv_bf16_bf16_out(1, 1, 1, 1, 3, 8, 4, 256, 32)
    with pytest.raises(ValueError, match="divisible"):
        M.gguf_q4_k_selected_gemv_bf16_bf16_out(1, 1, 1, 1, 1, 8, 4, 200, 32)
    with pytest.raises(ValueError, match="multiples of 32"):
        M.gguf_q4_k_grouped_mmq(1, 1, 1, 1, 1, 1, 8, 8, 256, 40, 4, 32)


def _bf16_steps_apart(got_bits, want_f32):
    """|got - want| in units of the bf16 spacing at the larger magnitude, the unit no smaller than 1e-6: where the
    three terms of order 0.2 cancel, a float32 rounding of one of them (1e-8) is many bf16 steps of the tiny sum."""
    got = O.bf16_bits_to_f32(got_bits)
    step = np.spacing(np.maximum(np.abs(got), np.abs(want_f32)).astype(np.float32)) * np.float32(65536.0)
    return np.abs(got - want_f32) / np.maximum(step, np.float32(1e-6))


@pytest.mark.parametrize("tokens,hidden", [(1, 17), (3, 2048), (4, 5120), (2, 8200), (130, 256)])
@pytest.mark.parametrize("mode", ["aggregate", "slots", "gather"])
def test_moe_tail_next_rmsnorm(dev, mode, tokens, hidden):
    """The MoE tail fused with the next RMSNorm (hipEngine's GGUF bf16 entries and the form that gathers compact
    rows) against the restated CPU reference: the combined residual equal bit for bit except where the device's
    expf moves a value across a bf16 rounding boundary (at most one step, in under 0.5 % of the values); the norm
    within one bf16 step of the reference's norm of that residual (the sum of squares is taken in another order).  Inputs as in hipEngine's own test
    (tests/test_gpu_moe_tail_next_rmsnorm.py:147-160): N(0, 0.2) rows, weights in (-0.5, 0.75), gate stride 3."""
    rng = np.random.default_rng(0x21A0 + tokens * 37 + hidden + len(mode))
    top_k, gate_stride, eps = 8, 3, 1e-6
    bits = lambda a: O.f32_to_bf16_bits(a.astype(np.float32))
    shared_b, residual_b = bits(rng.standard_normal((tokens, hidden)) * 0.2), bits(rng.standard_normal((tokens, hidden)) * 0.2)
    routing = rng.uniform(-0.5, 0.75, size=(tokens, top_k)).astype(np.float32)
    gate = rng.uniform(-4.0, 4.0, size=(tokens, gate_stride)).astype(np.float32)
    weight = rng.uniform(0.5, 1.5, size=hidden).astype(np.float32)
    d = {"shared": dev.put(shared_b), "residual": dev.put(residual_b), "gate": dev.put(gate), "weight": dev.put(weight),
         "routing": dev.put(routing), "norm": dev.empty(tokens * hidden * 2, fill=0x5A),
         "res_out": dev.empty(tokens * hidden * 2, fill=0x5A)}
    shared, residual = O.bf16_bits_to_f32(shared_b), O.bf16_bits_to_f32(residual_b)
    if mode == "aggregate":
        sel_b = bits(rng.standard_normal((tokens, hidden)) * 0.2)
        d["sel"] = dev.put(sel_b)
        PC.shared_gate_combine_residual_rmsnorm_gguf_bf16_out(d["sel"].ptr, d["shared"].ptr, d["gate"].ptr,
                                                              d["residual"].ptr, d["weight"].ptr, d["norm"].ptr,
                                                              d["res_out"].ptr, tokens, hidden, gate_stride, eps)
        want_r, want_n = O.moe_tail_next_rmsnorm(O.bf16_bits_to_f32(sel_b), shared, gate, residual, weight, eps=eps)
    elif mode == "slots":
        sel_b = bits(rng.standard_normal((tokens, top_k, hidden)) * 0.2)
        d["sel"] = dev.put(sel_b)
        PC.weighted_sum_shared_gate_combine_residual_rmsnorm_gguf_bf16_out(
            d["sel"].ptr, d["routing"].ptr, d["shared"].ptr, d["gate"].ptr, d["residual"].ptr, d["weight"].ptr,
            d["norm"].ptr, d["res_out"].ptr, tokens, top_k, hidden, gate_stride, eps)
        want_r, want_n = O.moe_tail_next_rmsnorm(O.bf16_bits_to_f32(sel_b), shared, gate, residual, weight,
                                                 routing_weights=routing, eps=eps)
    else:
        compact_rows = tokens * top_k - 2 if tokens > 1 else tokens * top_k
        l2c = rng.permutation(tokens * top_k).astype(np.int64)
        l2c[l2c >= compact_rows] = -1                       # two lanes of no expert
        sel_b = bits(rng.standard_normal((compact_rows, hidden)) * 0.2)
        d["sel"], d["l2c"] = dev.put(sel_b), dev.put(l2c)
        PC.moe_gather_tail_rmsnorm_bf16(d["sel"].ptr, d["l2c"].ptr, d["routing"].ptr, d["shared"].ptr, d["gate"].ptr,
                                        d["residual"].ptr, d["weight"].ptr, d["norm"].ptr, d["res_out"].ptr, tokens,
                                        top_k, hidden, compact_rows, gate_stride, eps)
        want_r, want_n = O.moe_tail_next_rmsnorm(O.bf16_bits_to_f32(sel_b), shared, gate, residual, weight,
                                                 routing_weights=routing, lane_to_compact=l2c, eps=eps)
    got_r = dev.get(d["res_out"], np.uint16, (tokens, hidden))
    got_n = dev.get(d["norm"], np.uint16, (tokens, hidden))
    # in place: the combined residual over the residual it read
    PC.shared_gate_combine_residual_rmsnorm_gguf_bf16_out(d["res_out"].ptr, d["shared"].ptr, d["gate"].ptr,
                                                          d["residual"].ptr, d["weight"].ptr, d["norm"].ptr,
                                                          d["residual"].ptr, tokens, hidden, gate_stride, eps)
    again_r = dev.get(d["residual"], np.uint16, (tokens, hidden))
    want_again, _ = O.moe_tail_next_rmsnorm(O.bf16_bits_to_f32(got_r), shared, gate, residual, weight, eps=eps)
    dev.free(*d.values())
    apart_r = _bf16_steps_apart(got_r, want_r)
    assert apart_r.max() <= 1.0 and np.mean(apart_r == 0) >= 0.995, (apart_r.max(), np.mean(apart_r == 0))
    # the norm of the combined residual the device formed (where that is a step off, so is its norm)
    zeros = np.zeros((tokens, hidden), np.float32)
    _, norm_of_got = O.moe_tail_next_rmsnorm(zeros, zeros, gate, O.bf16_bits_to_f32(got_r), weight, eps=eps)
    apart_n = _bf16_steps_apart(got_n, norm_of_got)
    assert apart_n.max() <= 1.0 and np.mean(apart_n == 0) >= 0.97, (apart_n.max(), np.mean(apart_n == 0))
    assert np.mean(_bf16_steps_apart(got_n, want_n) == 0) >= 0.97
    apart_again = _bf16_steps_apart(again_r, want_again)
    assert apart_again.max() <= 1.0 and np.mean(apart_again == 0) >= 0.995
