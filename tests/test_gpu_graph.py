"""A whole greedy decode step of the matmul path captured in ONE HIP graph and replayed:
embedding lookup -> projection -> projection + residual -> gate/up pair with SiLU -> down projection +
residual -> lm_head -> row-wise arg-max.  Every entry point is launched on a capture stream (no allocation,
no synchronization, no memset nodes); the graph is replayed several times with different token ids and
eager work and synchronizations between the replays, and every replay is compared bit for bit with the eager
run of the same chain (hipEngine replays decode graphs in production: core/hip.py:261-306).
"""

from __future__ import annotations

import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest

from oracle import gguf_oracle as O
from hipengine_amd.kernels.hip_gfx950.linear import lm_head as L
from hipengine_amd.kernels.hip_gfx950.quant import gguf_embedding as E
from hipengine_amd.kernels.hip_gfx950.quant import gguf_q8_1_gemv as G

pytestmark = pytest.mark.gpu

H, F, V = 4096, 6144, 8192


def _chain(bufs, stream, B):
    E.gguf_q4_k_embedding_bf16_out(bufs["ids"].ptr, bufs["emb"].ptr, bufs["x"].ptr, B, H, V, stream=stream)
    G.FUSED[("q4_k", "bf16", "bf16")](bufs["x"].ptr, bufs["wq"].ptr, bufs["q"].ptr, B, H, H, stream=stream)
    G.gguf_gemv_residual("gguf_q4_k", bufs["q"].ptr, "bf16", bufs["wo"].ptr, bufs["x"].ptr, bufs["h1"].ptr, "bf16", B, H, H,
                         stream=stream)
    if B <= 2:
        G.gguf_pair_silu_gemv("gguf_q4_k", bufs["h1"].ptr, "bf16", bufs["wg"].ptr, bufs["wu"].ptr, bufs["mid"].ptr, "bf16",
                              B, H, F, stream=stream)
    else:   # the pair form stops at batch 2: the gate projection alone stands in for the FFN's first half
        G.FUSED[("q4_k", "bf16", "bf16")](bufs["h1"].ptr, bufs["wg"].ptr, bufs["mid"].ptr, B, H, F, stream=stream)
    G.gguf_gemv_residual("gguf_q6_k", bufs["mid"].ptr, "bf16", bufs["wd"].ptr, bufs["h1"].ptr, bufs["h2"].ptr, "bf16", B, F, H,
                         stream=stream)
    G.FUSED[("q6_k", "bf16", "f32")](bufs["h2"].ptr, bufs["wl"].ptr, bufs["logits"].ptr, B, H, V, stream=stream)
    L.argmax_f32_rows_i32(bufs["logits"].ptr, bufs["bv"].ptr, bufs["bi"].ptr, bufs["next"].ptr, None, B, V, stream=stream)


@pytest.mark.parametrize("B", [2, 8])
def test_decode_step_graph_replays_match_eager(dev, B):
    """Batch 2 takes the stream / run forms and the fused FFN; batch 8 the slab and phased slab forms on the
    MFMA.  The chain is captured cold - no launch of it precedes the capture: whatever set-up the kernels need
    was done per device when the library was loaded (hipengine_gfx950_init)."""
    rt = dev.runtime
    bufs = {
        "emb": dev.put(O.random_weight(O.GGML_Q4_K, V, H, seed=1, std=1.0)),
        "wq": dev.put(O.random_weight(O.GGML_Q4_K, H, H, seed=2)),
        "wo": dev.put(O.random_weight(O.GGML_Q4_K, H, H, seed=3)),
        "wg": dev.put(O.random_weight(O.GGML_Q4_K, F, H, seed=4)),
        "wu": dev.put(O.random_weight(O.GGML_Q4_K, F, H, seed=5)),
        "wd": dev.put(O.random_weight(O.GGML_Q6_K, H, F, seed=6)),
        "wl": dev.put(O.random_weight(O.GGML_Q6_K, V, H, seed=7)),
        "ids": dev.put(np.arange(B, dtype=np.int64)),
        "x": dev.empty(B * H * 2), "q": dev.empty(B * H * 2), "h1": dev.empty(B * H * 2), "mid": dev.empty(B * F * 2),
        "h2": dev.empty(B * H * 2), "logits": dev.empty(B * V * 4), "next": dev.empty(B * 4),
    }
    n = L.argmax_scratch_entries(B, V)
    bufs["bv"], bufs["bi"] = dev.empty(n * 4), dev.empty(n * 4)

    def read():
        return (dev.get(bufs["h2"], np.uint16, (B, H)).copy(), dev.get(bufs["logits"], np.uint32, (B, V)).copy(),
                dev.get(bufs["next"], np.int32, (B,)).copy())

    stream = rt.stream_create()
    rt.stream_begin_capture(stream)
    _chain(bufs, stream, B)
    graph = rt.stream_end_capture(stream)
    assert graph
    graph_exec = rt.graph_instantiate(graph)
    assert graph_exec

    for ids in ([3, 4097], [8191, 0], [77, 77], [5000, 123]):
        host_ids = np.resize(np.array(ids, dtype=np.int64), B)
        # eager reference of this step
        rt.memcpy(bufs["ids"].ptr, host_ids.ctypes.data, host_ids.nbytes, 1)
        _chain(bufs, stream, B)
        rt.stream_synchronize(stream)
        want = read()
        for name in ("x", "q", "h1", "mid", "h2", "logits", "next"):      # poison the outputs
            rt.memset(bufs[name].ptr, 0x5C, bufs[name].nbytes)
        rt.device_synchronize()
        rt.graph_launch(graph_exec, stream)
        rt.stream_synchronize(stream)
        got = read()
        assert np.array_equal(got[0], want[0])
        assert np.array_equal(got[1], want[1])
        assert np.array_equal(got[2], want[2])
        # and the arg-max is the arg-max of those logits
        assert np.array_equal(got[2], O.argmax_rows(got[1].view(np.float32))[0])

    rt.graph_exec_destroy(graph_exec)
    rt.graph_destroy(graph)
    rt.stream_destroy(stream)
    dev.free(*bufs.values())


def test_moe_block_graph_replays_and_matches_cpu(dev):
    """A whole MoE FFN block on the device in one HIP graph: router logits -> top-k + softmax -> routed experts
    (gate/up with SiLU, routed down sum) -> shared expert (Q8_0 gate|up in one GEMV, SiLU, down) -> shared gate logit
    -> tail (routed sum + gated shared expert + residual) with the next RMSNorm.  Replays equal the eager chain bit for
    bit; the block output follows the reference CPU block (kernels/cpu_reference/ops.py gguf_moe_ffn_block) to the
    accuracy of q8_1 activations and bf16 boundaries, with the routing taken from the device's own logits."""
    from hipengine_amd.kernels.hip_gfx950.fused import paro_combine as PC
    from hipengine_amd.kernels.hip_gfx950.moe import router as RT
    from hipengine_amd.kernels.hip_gfx950.quant import gguf_moe as M

    rt = dev.runtime
    T, E, K8, HID, INTER, SI = 2, 32, 8, 2048, 512, 256
    rng = np.random.default_rng(41)
    host = {
        "wr": (rng.standard_normal((E, HID)) * 0.05).astype(np.float32),
        "wgate": (rng.standard_normal((1, HID)) * 0.05).astype(np.float32),
        "wg": O.stack_experts(O.random_weight(O.GGML_Q4_K, INTER, HID, seed=1), E, seed=1),
        "wu": O.stack_experts(O.random_weight(O.GGML_Q4_K, INTER, HID, seed=2), E, seed=2),
        "wd": O.stack_experts(O.random_weight(O.GGML_Q4_K, HID, INTER, seed=3), E, seed=3),
        "sg": O.random_weight(O.GGML_Q8_0, SI, HID, seed=4), "su": O.random_weight(O.GGML_Q8_0, SI, HID, seed=5),
        "sd": O.random_weight(O.GGML_Q8_0, HID, SI, seed=6),
        "norm": rng.uniform(0.5, 1.5, HID).astype(np.float32),
    }
    lanes = T * K8
    bufs = {k: dev.put(v) for k, v in host.items()}
    bufs["sgu"] = dev.put(np.concatenate([host["sg"], host["su"]], axis=0))      # gate rows, then up rows
    for name, nbytes in (("x", T * HID * 2), ("logits", T * E * 4), ("sel", lanes * 8), ("routing", lanes * 4),
                         ("mid", lanes * INTER * 4), ("routed", T * HID * 2), ("gu", T * 2 * SI * 4),
                         ("smid", T * SI * 2), ("shared", T * HID * 2), ("glogit", T * 4), ("norm_out", T * HID * 2),
                         ("res_out", T * HID * 2)):
        bufs[name] = dev.empty(nbytes)

    def chain(stream):
        RT.qwen35_router_logits_bf16_f32w(bufs["x"].ptr, bufs["wr"].ptr, bufs["logits"].ptr, T, HID, E, stream=stream)
        RT.qwen35_router_select(bufs["logits"].ptr, bufs["sel"].ptr, bufs["routing"].ptr, T, E, E, K8, stream=stream)
        M.gguf_selected_gemv("gguf_q4_k", M.SEL_DUAL_SILU, bufs["x"].ptr, bufs["sel"].ptr, bufs["wg"].ptr, bufs["mid"].ptr,
                             T, lanes, E, HID, INTER, qweight_b_ptr=bufs["wu"].ptr, x_dtype="bf16", stream=stream)
        M.gguf_selected_gemv("gguf_q4_k", M.SEL_DOWN_SUM, bufs["mid"].ptr, bufs["sel"].ptr, bufs["wd"].ptr,
                             bufs["routed"].ptr, T, lanes, E, INTER, HID, routing_weights_ptr=bufs["routing"].ptr,
                             top_k=K8, out_dtype="bf16", stream=stream)
        G.FUSED[("q8_0", "bf16", "f32")](bufs["x"].ptr, bufs["sgu"].ptr, bufs["gu"].ptr, T, HID, 2 * SI, stream=stream)
        M.moe_silu_mul(bufs["gu"].ptr, bufs["smid"].ptr, T, SI, out_dtype="bf16", stream=stream)
        G.FUSED[("q8_0", "bf16", "bf16")](bufs["smid"].ptr, bufs["sd"].ptr, bufs["shared"].ptr, T, SI, HID, stream=stream)
        RT.qwen35_router_logits_bf16_f32w(bufs["x"].ptr, bufs["wgate"].ptr, bufs["glogit"].ptr, T, HID, 1, stream=stream)
        PC.shared_gate_combine_residual_rmsnorm_gguf_bf16_out(bufs["routed"].ptr, bufs["shared"].ptr, bufs["glogit"].ptr,
                                                              bufs["x"].ptr, bufs["norm"].ptr, bufs["norm_out"].ptr,
                                                              bufs["res_out"].ptr, T, HID, 1, 1e-6, stream=stream)

    outputs = ("logits", "sel", "routing", "mid", "routed", "gu", "smid", "shared", "glogit", "norm_out", "res_out")

    def read():
        return {name: dev.get(bufs[name], np.uint8, (bufs[name].nbytes,)).copy() for name in outputs}

    stream = rt.stream_create()
    rt.stream_begin_capture(stream)        # cold: nothing of this chain has been launched before
    chain(stream)
    graph = rt.stream_end_capture(stream)
    graph_exec = rt.graph_instantiate(graph)
    assert graph and graph_exec
    for step in range(3):
        x = (np.random.default_rng(100 + step).standard_normal((T, HID)) * 0.3).astype(np.float32)
        xb = O.f32_to_bf16_bits(x)
        rt.memcpy(bufs["x"].ptr, xb.ctypes.data, xb.nbytes, 1)
        chain(stream)
        rt.stream_synchronize(stream)
        want = read()
        for name in outputs:
            rt.memset(bufs[name].ptr, 0x5C, bufs[name].nbytes)
        rt.device_synchronize()
        rt.graph_launch(graph_exec, stream)
        rt.stream_synchronize(stream)
        got = read()
        for name in outputs:
            assert np.array_equal(got[name], want[name]), name
        # against the CPU block, with the device's own selection (its logits decide near-ties)
        xf = O.bf16_bits_to_f32(xb)
        logits = got["logits"].view(np.float32).reshape(T, E)
        ref_logits = O.router_logits(xf, host["wr"])
        assert np.allclose(logits, ref_logits, rtol=1e-5, atol=1e-5)
        sel, routing = O.router_topk_softmax(logits, K8)
        assert np.array_equal(got["sel"].view(np.int64).reshape(T, K8), sel)
        assert np.allclose(got["routing"].view(np.float32).reshape(T, K8), routing, rtol=1e-5, atol=1e-6)
        block = O.moe_ffn_block(xf, xf, sel, routing, host["wg"], host["wu"], host["wd"], host["wgate"][0], host["sg"],
                                host["su"], host["sd"])
        res = O.bf16_bits_to_f32(got["res_out"].view(np.uint16).reshape(T, HID))
        assert O.cosine(res, block) >= 0.9995
        np.testing.assert_allclose(res, block, rtol=2e-2, atol=2e-2 * np.abs(block).max())
        zeros = np.zeros((T, HID), np.float32)
        _, norm = O.moe_tail_next_rmsnorm(zeros, zeros, np.zeros(T, np.float32), res, host["norm"])
        got_norm = O.bf16_bits_to_f32(got["norm_out"].view(np.uint16).reshape(T, HID))
        np.testing.assert_allclose(got_norm, norm, rtol=2.0 ** -7, atol=1e-6)
    rt.graph_exec_destroy(graph_exec)
    rt.graph_destroy(graph)
    rt.stream_destroy(stream)
    dev.free(*bufs.values())


def test_graphs_capture_cold_in_a_fresh_process():
    """The captures above run after other tests of the same process have launched, and so set up, the same
    kernels.  Here a child process loads the library (whose per-device set-up is all the set-up there is) and
    captures as its very first launches: a kernel missing from that set-up would fail the capture."""
    code = ("from tests._device import Device\n"
            "import tests.test_gpu_graph as t\n"
            "d = Device()\n"
            "t.test_decode_step_graph_replays_match_eager(d, 8)\n"
            "t.test_moe_block_graph_replays_and_matches_cpu(d)\n"
            "d2 = Device()\n"
            "t.test_decode_step_graph_replays_match_eager(d2, 2)\n"
            "print('COLD_CAPTURE_OK')\n")
    root = Path(__file__).resolve().parents[1]
    proc = subprocess.run([sys.executable, "-c", code], cwd=root, capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0 and "COLD_CAPTURE_OK" in proc.stdout, proc.stdout[-2000:] + proc.stderr[-4000:]
