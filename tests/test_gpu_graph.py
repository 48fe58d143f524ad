"""A whole greedy decode step of the matmul path captured in ONE HIP graph and replayed:
embedding lookup -> projection -> projection + residual -> gate/up pair with SiLU -> down projection +
residual -> lm_head -> row-wise arg-max.  Every entry point is launched on a capture stream (no allocation,
no synchronization, no memset nodes); the graph is replayed several times with different token ids and
eager work and synchronizations between the replays, and every replay is compared bit for bit with the eager
run of the same chain (hipEngine replays decode graphs in production: core/hip.py:261-306).
"""

from __future__ import annotations

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
