"""CPU oracle for the GGUF k-quant matmul path.  TEST INFRASTRUCTURE ONLY.

This module restates, in NumPy, the arithmetic of hipEngine's CPU reference
backend and of the device-side specifications it is compared with.  It is the
checker for the gfx950 kernels: only the test-suite, the smoke entry and the
``cpu_baseline`` leg of the benchmark may import it.  Nothing in
``hipengine_amd`` imports it, and no kernel falls back to it.

Every function names the reference source it follows (paths relative to the
hipEngine tree).  Pinning status of each function (what independent evidence
the tests hold for it) is listed here; a function without any is marked
"parity unpinned".

===========================  =================================================
function                     pinned by
===========================  =================================================
q4_k_scale_min               inverse packer round trip over boundary + random
                             6-bit tuples; scalar per-sub-block restatement
dequant_q4_k                 reference one-block known answer
                             (tests/test_unit_gguf_quant_layout.py:68-80);
                             scalar per-element map (Appendix-style) in
                             float64; closed-form weight generator identity
dequant_q6_k                 exact inverse of the reference block builder
                             (tests/_gguf_synthetic_weights.py:123-158);
                             scalar per-element map in float64
dequant_q8_0                 reference one-block known answer
                             (tests/test_unit_gguf_quant_layout.py:48-53)
gguf_quant_gemv              float64 matmul of the dequantized weight;
                             reference closed-form case
                             (tests/test_gpu_gguf_q4_k_gemv.py:102-112)
moe_selected_ffn             committed golden of the reference
                             (tests/fixtures/cpu_reference/moe/
                             moe_ffn_selected_gguf_q4_k.json, copied as data
                             to tests/golden/); independent dense recompute
moe_ffn_block                same golden file (``expected_block``)
argmax_rows                  brute-force loop with the reference's pair comparison, ties
embedding_lookup             definition: dequantize(qweight[ids]); error cases of the reference
dequant_q5_k                 block builder inverse (reference generator restated),
                             scalar per-element loop, qh = 0 equals Q4_K
quantize_q8_1                float64 brute force, invariants (|q|<=127,
                             q[argmax]=+-127, zero block), tie cases built
                             from exact binary fractions
quantize_q8_1x2              plane 0 = quantize_q8_1; the two planes reconstruct x to 2^-13 of the
                             block's amax (float64 check); a block plane 0 represents exactly
                             has a zero plane 1
pack_q8_1_ds4                same, half-to-even tie case, fp16 clamp case
pack_q8_1_d4s4               same, summation tree spelled out independently
block_dots_*                 int64 einsum over independently unpacked integers
mmq_q8_0_d4s4                float64 product of the dequantized weight and activations
gemv_q8_1_* / mmq_*          float64 evaluation of the same formula
                             (tests/test_gpu_gguf_q4_k_q8_1_mmq_prefill.py
                             :115-165 style)
router_logits                float64 matmul (a float32 matmul by definition)
router_topk_softmax          brute-force argsort; ties -> lowest index
mtp_moe_routing              closed form on tiny cases
build_routing_index          invariants (prefix sums, permutation, stability,
                             compact_to_source = lane // top_k) + brute force
moe_tail_next_rmsnorm        reference known answer with both rounding boundaries
                             (tests/test_gpu_moe_tail_next_rmsnorm.py:98-119);
                             scalar float64 loop on a small case within one bf16 step;
                             slot-weighted == aggregate of the separately formed sum
quantize_q4_k / q6_k / q8_0  the reference ships NO fp32->Q4_K/Q6_K quantizer;
                             these only shape test data.  PARITY UNPINNED
                             (and not needed: parity is defined on block
                             bytes).  Q8_0 follows the reference's ad-hoc
                             script quantizer and is pinned by round trip.
===========================  =================================================
"""

from __future__ import annotations

import numpy as np

QK_K = 256
Q4_K_BLOCK_BYTES = 144
Q5_K_BLOCK_BYTES = 176
Q6_K_BLOCK_BYTES = 210
Q8_0_BLOCK_BYTES = 34
Q8_1_BLOCK = 32
Q8_1_BLOCK_BYTES = 36
DS4_BLOCK = 128
DS4_BLOCK_BYTES = 144
D4S4_BLOCK_BYTES = 160
FP16_MAX = np.float32(65504.0)

GGML_Q8_0 = 8
GGML_Q4_K = 12
GGML_Q5_K = 13
GGML_Q6_K = 14

_BLOCK_GEOMETRY = {
    GGML_Q8_0: (32, Q8_0_BLOCK_BYTES),
    GGML_Q4_K: (QK_K, Q4_K_BLOCK_BYTES),
    GGML_Q5_K: (QK_K, Q5_K_BLOCK_BYTES),
    GGML_Q6_K: (QK_K, Q6_K_BLOCK_BYTES),
}


# --------------------------------------------------------------------------
# scalar helpers
# --------------------------------------------------------------------------

def bf16_bits_to_f32(bits) -> np.ndarray:
    """bf16 bit patterns (uint16) -> float32 (hipengine/quant/gguf.py:491-493)."""
    u16 = np.ascontiguousarray(bits, dtype=np.uint16)
    return (u16.astype(np.uint32) << np.uint32(16)).view(np.float32)


def f32_to_bf16_bits(values) -> np.ndarray:
    """float32 -> bf16 bits, round to nearest even by ``+0x7FFF+lsb`` with no NaN
    special case (kernels/hip_gfx1100/quant/gguf_q4_k_gemv.hip:32-41)."""
    u32 = np.ascontiguousarray(values, dtype=np.float32).view(np.uint32).astype(np.uint64)
    lsb = (u32 >> np.uint64(16)) & np.uint64(1)
    return (((u32 + np.uint64(0x7FFF) + lsb) >> np.uint64(16)) & np.uint64(0xFFFF)).astype(np.uint16)


def _fp16_field(blocks: np.ndarray, offset: int) -> np.ndarray:
    """Little-endian fp16 at ``offset`` of every block row, widened to float32."""
    return np.ascontiguousarray(blocks[:, offset:offset + 2]).view(np.float16).astype(np.float32)[:, 0]


def _as_blocks(data, type_size: int) -> tuple[np.ndarray, tuple[int, ...]]:
    raw = np.ascontiguousarray(data).view(np.uint8)
    if raw.size % type_size:
        raise ValueError(f"byte size {raw.size} is not a multiple of block size {type_size}")
    return raw.reshape(-1, type_size), raw.shape


def round_half_away(values: np.ndarray) -> np.ndarray:
    """C ``roundf``: ties go away from zero."""
    v = np.asarray(values, dtype=np.float32)
    t = np.trunc(v)
    frac = np.abs(v - t)
    return np.where(frac >= np.float32(0.5), t + np.sign(v), t).astype(np.float32)


# --------------------------------------------------------------------------
# block unpack / dequant  (reference: hipengine/quant/gguf.py)
# --------------------------------------------------------------------------

def q4_k_scale_min(scale_bytes) -> tuple[np.ndarray, np.ndarray]:
    """12 packed bytes per block -> (scales[8], mins[8]) as uint8.

    Follows ``unpack_q4_k_scale_min`` (hipengine/quant/gguf.py:611-624) and the
    device twins ``gguf_q4_k_scale/min`` (gguf_q4_k_gemv.hip:74-88).
    """
    s = np.ascontiguousarray(scale_bytes, dtype=np.uint8).reshape(-1, 12)
    lo_s, lo_m, hi = s[:, 0:4], s[:, 4:8], s[:, 8:12]
    sc = np.empty((s.shape[0], 8), dtype=np.uint8)
    mn = np.empty((s.shape[0], 8), dtype=np.uint8)
    sc[:, :4] = lo_s & 0x3F
    mn[:, :4] = lo_m & 0x3F
    sc[:, 4:] = (hi & 0x0F) | ((lo_s >> 2) & 0x30)
    mn[:, 4:] = (hi >> 4) | ((lo_m >> 2) & 0x30)
    return sc, mn


def pack_q4_k_scale_min(scales, mins) -> np.ndarray:
    """Inverse of :func:`q4_k_scale_min` (hipengine/quant/gguf_q4_k.py:285-296)."""
    sc = np.ascontiguousarray(scales, dtype=np.uint8).reshape(-1, 8)
    mn = np.ascontiguousarray(mins, dtype=np.uint8).reshape(-1, 8)
    out = np.empty((sc.shape[0], 12), dtype=np.uint8)
    out[:, 0:4] = (sc[:, :4] & 0x3F) | ((sc[:, 4:] & 0x30) << 2)
    out[:, 4:8] = (mn[:, :4] & 0x3F) | ((mn[:, 4:] & 0x30) << 2)
    out[:, 8:12] = (sc[:, 4:] & 0x0F) | ((mn[:, 4:] & 0x0F) << 4)
    return out


def q4_k_quants(blocks: np.ndarray) -> np.ndarray:
    """[n,144] block bytes -> unsigned 4-bit values [n,8,32] in element order.

    Byte ``j`` of 32-byte group ``g`` carries element ``64g+j`` in its low nibble
    and ``64g+32+j`` in its high nibble (gguf.py:641-643, gguf_q4_k_gemv.hip:90-106).
    """
    qs = blocks[:, 16:144].reshape(-1, 4, 32)
    out = np.empty((blocks.shape[0], 8, 32), dtype=np.uint8)
    out[:, 0::2] = qs & 0x0F
    out[:, 1::2] = qs >> 4
    return out


def dequant_q4_k(blocks: np.ndarray) -> np.ndarray:
    """``(d*sc)*q - (dmin*mn)`` in float32 (gguf.py:631-643)."""
    d = _fp16_field(blocks, 0)
    dmin = _fp16_field(blocks, 2)
    sc, mn = q4_k_scale_min(blocks[:, 4:16])
    scale = (d[:, None] * sc.astype(np.float32))[:, :, None]
    offset = (dmin[:, None] * mn.astype(np.float32))[:, :, None]
    q = q4_k_quants(blocks).astype(np.float32)
    return (scale * q - offset).reshape(-1, QK_K)


def q5_k_quants(blocks: np.ndarray) -> np.ndarray:
    """[n,176] block bytes -> unsigned 5-bit values [n,8,32] in element order.

    ``{half d; half dmin; u8 scales[12]; u8 qh[32]; u8 qs[128]}``: the low four bits as in
    Q4_K (byte ``j`` of 32-byte group ``g`` of ``qs``: element ``64g+j`` low nibble,
    ``64g+32+j`` high nibble); bit 4 of the value of sub-block ``s``, lane ``l`` is bit
    ``s`` of ``qh[l]`` (gguf.py:646-662, gguf_q6_k_embedding.hip q5_k_weight)."""
    n = blocks.shape[0]
    qs = blocks[:, 48:176].reshape(n, 4, 32)
    qh = blocks[:, 16:48]
    out = np.empty((n, 8, 32), dtype=np.uint8)
    out[:, 0::2] = qs & 0x0F
    out[:, 1::2] = qs >> 4
    for sb in range(8):
        out[:, sb] |= ((qh >> sb) & 1) << 4
    return out


def dequant_q5_k(blocks: np.ndarray) -> np.ndarray:
    """``(d*sc)*q - (dmin*mn)`` in float32 with 5-bit ``q`` (gguf.py:646-662)."""
    d = _fp16_field(blocks, 0)
    dmin = _fp16_field(blocks, 2)
    sc, mn = q4_k_scale_min(blocks[:, 4:16])
    scale = (d[:, None] * sc.astype(np.float32))[:, :, None]
    offset = (dmin[:, None] * mn.astype(np.float32))[:, :, None]
    q = q5_k_quants(blocks).astype(np.float32)
    return (scale * q - offset).reshape(-1, QK_K)


def q6_k_quants(blocks: np.ndarray) -> np.ndarray:
    """[n,210] block bytes -> signed 6-bit values [n,8,32] (already ``-32``).

    Element ``k``: ``g=k>>5``; low nibble source ``ql[64*(g>=4) + 32*(g&1) + lane]``,
    low half if ``(g&2)==0``; two high bits ``qh[32*(g>=4)+lane] >> 2*(g&3)``
    (gguf.py:665-681, gguf_k_gemv.hip:139-160).
    """
    n = blocks.shape[0]
    ql = blocks[:, 0:128].reshape(n, 2, 2, 32)      # [half, byte-group, lane]
    qh = blocks[:, 128:192].reshape(n, 2, 32)       # [half, lane]
    out = np.empty((n, 8, 32), dtype=np.int16)
    for g in range(8):
        half, which, upper = g >> 2, g & 1, (g >> 1) & 1
        nib = (ql[:, half, which] >> (4 * upper)) & 0x0F
        top = (qh[:, half] >> (2 * (g & 3))) & 0x03
        out[:, g] = (nib | (top << 4)).astype(np.int16) - 32
    return out.astype(np.int8)


def dequant_q6_k(blocks: np.ndarray) -> np.ndarray:
    """``(d*scale_i8[k/16])*q`` in float32 (gguf.py:665-681)."""
    n = blocks.shape[0]
    scales = blocks[:, 192:208].view(np.int8).astype(np.float32)
    d = _fp16_field(blocks, 208)
    step = (d[:, None] * scales)[:, :, None]                     # [n,16,1]
    q = q6_k_quants(blocks).reshape(n, 16, 16).astype(np.float32)
    return (step * q).reshape(n, QK_K)


def dequant_q8_0(blocks: np.ndarray) -> np.ndarray:
    """``q*d`` in float32 (gguf.py:604-608)."""
    d = _fp16_field(blocks, 0)
    q = blocks[:, 2:34].view(np.int8).astype(np.float32)
    return q * d[:, None]


_DEQUANT = {GGML_Q8_0: dequant_q8_0, GGML_Q4_K: dequant_q4_k, GGML_Q5_K: dequant_q5_k, GGML_Q6_K: dequant_q6_k}


def dequantize(data, qtype: int) -> np.ndarray:
    """Block bytes with GGUF byte shape ``[..., bytes_per_row]`` -> float32
    ``[..., values_per_row]`` (``dequantize_gguf_data``, gguf.py:497-547)."""
    block_size, type_size = _BLOCK_GEOMETRY[int(qtype)]
    blocks, shape = _as_blocks(data, type_size)
    if shape[-1] % type_size:
        raise ValueError(f"bytes per row {shape[-1]} is not a multiple of {type_size}")
    out = _DEQUANT[int(qtype)](blocks).astype(np.float32, copy=False)
    return out.reshape(*shape[:-1], shape[-1] // type_size * block_size)


# --------------------------------------------------------------------------
# CPU reference backend GEMV / MoE  (reference: kernels/cpu_reference/ops.py)
# --------------------------------------------------------------------------

def gguf_quant_gemv(x, qweight, qtype: int) -> np.ndarray:
    """``matmul(x, dequant(W).T)`` in float32 (ops.py:466-484)."""
    xa = np.asarray(x, dtype=np.float32)
    qw = np.asarray(qweight)
    if xa.ndim != 2:
        raise ValueError("x must have shape [rows, in_features]")
    if qw.ndim != 2:
        raise ValueError("qweight must have GGUF byte shape [out_features, bytes_per_row]")
    w = dequantize(qw, qtype)
    if xa.shape[1] != w.shape[1]:
        raise ValueError("x.shape[1] must match qweight in_features")
    return np.matmul(xa, w.T).astype(np.float32)


def gguf_quant_gemv_chunked(x, qweight, qtype: int, chunk_rows: int = 8192) -> np.ndarray:
    """Same value as :func:`gguf_quant_gemv` column by column, dequantizing
    ``chunk_rows`` weight rows at a time so a 151936-row weight never needs
    its 3 GB float32 image at once."""
    xa = np.asarray(x, dtype=np.float32)
    qw = np.asarray(qweight)
    out = np.empty((xa.shape[0], qw.shape[0]), dtype=np.float32)
    for lo in range(0, qw.shape[0], chunk_rows):
        hi = min(qw.shape[0], lo + chunk_rows)
        out[:, lo:hi] = gguf_quant_gemv(xa, qw[lo:hi], qtype)
    return out


def embedding_lookup(token_ids, qweight, qtype: int) -> np.ndarray:
    """Rows ``token_ids`` of a quantized table, dequantized to float32
    (``_gguf_k_embedding``, kernels/cpu_reference/ops.py:511-524)."""
    ids = np.asarray(token_ids, dtype=np.int64)
    qw = np.asarray(qweight)
    if ids.ndim != 1:
        raise ValueError("token_ids must have shape [rows]")
    if qw.ndim != 2:
        raise ValueError("qweight must have GGUF byte shape [vocab_size, bytes_per_row]")
    if np.any(ids < 0) or np.any(ids >= qw.shape[0]):
        raise ValueError("token_ids contain out-of-range token IDs")
    return dequantize(qw[ids], qtype).astype(np.float32)


def argmax_rows(logits) -> tuple[np.ndarray, np.ndarray]:
    """Row-wise (index, value) of the maximum, lowest index among equal values
    (``better_pair_i32``, kernels/hip_gfx1100/linear/lm_head.hip:188-190)."""
    lg = np.asarray(logits, dtype=np.float32)
    idx = np.argmax(lg, axis=-1).astype(np.int32)          # first occurrence = lowest index
    return idx, np.take_along_axis(lg, idx[:, None].astype(np.int64), axis=-1)[:, 0]


def silu(v: np.ndarray) -> np.ndarray:
    v = np.asarray(v, dtype=np.float32)
    return (v / (np.float32(1.0) + np.exp(-v).astype(np.float32))).astype(np.float32)


def moe_selected_ffn(x, selected, routing, gate_q, up_q, down_q,
                     gate_t: int = GGML_Q4_K, up_t: int = GGML_Q4_K, down_t: int = GGML_Q4_K,
                     cache: bool = True) -> np.ndarray:
    """Selected-expert MoE FFN (ops.py:624-678): for token t, slot k, expert e:
    ``out[t] += w[t,k] * Wd_e( silu(Wg_e x_t) * (Wu_e x_t) )``.

    ``cache=True`` keeps each expert's dequantized matrices for the duration of
    the call; values are unchanged (same float32 matmul per (token, slot)).
    """
    xa = np.asarray(x, dtype=np.float32)
    sel = np.asarray(selected, dtype=np.int64)
    wts = np.asarray(routing, dtype=np.float32)
    tokens, hidden = xa.shape
    if sel.shape != wts.shape or sel.ndim != 2 or sel.shape[0] != tokens:
        raise ValueError("selected/routing must both have shape [tokens, top_k]")
    gq, uq, dq = np.asarray(gate_q), np.asarray(up_q), np.asarray(down_q)
    if gq.ndim != 3 or uq.ndim != 3 or dq.ndim != 3:
        raise ValueError("expert weights must be rank-3 [E, out, row_bytes]")
    experts = gq.shape[0]
    memo: dict[int, tuple[np.ndarray, np.ndarray, np.ndarray]] = {}

    def mats(e: int):
        if e in memo:
            return memo[e]
        m = (dequantize(gq[e], gate_t), dequantize(uq[e], up_t), dequantize(dq[e], down_t))
        if cache:
            memo[e] = m
        return m

    out = np.zeros((tokens, hidden), dtype=np.float32)
    for t in range(tokens):
        xt = xa[t:t + 1]
        for k in range(sel.shape[1]):
            e = int(sel[t, k])
            if not 0 <= e < experts:
                raise ValueError("selected expert id out of range")
            wg, wu, wd = mats(e)
            gate = np.matmul(xt, wg.T).astype(np.float32)
            up = np.matmul(xt, wu.T).astype(np.float32)
            inter = (silu(gate) * up).astype(np.float32)
            down = np.matmul(inter, wd.T).astype(np.float32)
            out[t] += np.float32(wts[t, k]) * down[0]
    return out


def moe_ffn_block(x, residual, selected, routing, gate_q, up_q, down_q,
                  shared_gate_logit_w, shared_gate_q, shared_up_q, shared_down_q,
                  shared_t: int = GGML_Q8_0) -> np.ndarray:
    """Full MoE FFN block used by the reference golden: residual + selected
    experts + sigmoid(x.w) * shared-expert FFN (ops.py ``gguf_moe_ffn_block``;
    tests/test_unit_cpu_reference_moe_ffn.py:133-146)."""
    xa = np.asarray(x, dtype=np.float32)
    sel_out = moe_selected_ffn(xa, selected, routing, gate_q, up_q, down_q)
    g = gguf_quant_gemv(xa, shared_gate_q, shared_t)
    u = gguf_quant_gemv(xa, shared_up_q, shared_t)
    shared = gguf_quant_gemv((silu(g) * u).astype(np.float32), shared_down_q, shared_t)
    logit = xa @ np.asarray(shared_gate_logit_w, dtype=np.float32)
    gate = (np.float32(1.0) / (np.float32(1.0) + np.exp(-logit))).astype(np.float32)
    return (np.asarray(residual, dtype=np.float32) + sel_out + gate[:, None] * shared).astype(np.float32)


def moe_tail_next_rmsnorm(selected_values, shared, gate_logits, residual, norm_weight, *, routing_weights=None,
                          lane_to_compact=None, eps: float = 1e-6) -> tuple[np.ndarray, np.ndarray]:
    """MoE tail and the next layer's RMSNorm with bf16 boundaries (kernels/cpu_reference/ops.py:33-102):
    the routed sum (given, or formed in slot order in float32, product and sum rounded separately, then rounded
    to bf16), ``residual' = bf16((residual + selected) + sigmoid(gate[:, 0]) * shared)``,
    ``norm = bf16(residual' / sqrt(mean(residual'^2) + eps) * weight)`` (ops.py:25-29).
    ``selected_values`` is ``[tokens, hidden]`` without ``routing_weights``, ``[tokens, top_k, hidden]`` with them,
    or compact rows ``[compact_rows, hidden]`` with ``lane_to_compact`` ``[tokens * top_k]`` (a lane < 0 or past the
    compact rows contributes nothing).  Float32 values in, float32 values of the bf16 results out."""
    res = np.asarray(residual, dtype=np.float32)
    sh = np.asarray(shared, dtype=np.float32)
    sel = np.asarray(selected_values, dtype=np.float32)
    w = np.asarray(norm_weight, dtype=np.float32)
    if res.ndim != 2 or sh.shape != res.shape or w.shape != (res.shape[1],):
        raise ValueError("residual and shared must be [tokens, hidden] and norm_weight [hidden]")
    tokens, hidden = res.shape

    def rnd(v):
        return bf16_bits_to_f32(f32_to_bf16_bits(np.asarray(v, dtype=np.float32)))

    if routing_weights is None:
        if sel.shape != res.shape:
            raise ValueError("an already formed routed sum must match the residual shape")
        selected_sum = sel
    else:
        rw = np.asarray(routing_weights, dtype=np.float32).reshape(tokens, -1)
        top_k = rw.shape[1]
        if lane_to_compact is not None:
            l2c = np.asarray(lane_to_compact, dtype=np.int64).reshape(tokens, top_k)
            live = (l2c >= 0) & (l2c < sel.shape[0])
            rows = sel[np.where(live, l2c, 0)]
            rows = np.where(live[..., None], rows, np.float32(0.0))
            rw = np.where(live, rw, np.float32(0.0))
        else:
            if sel.shape != (tokens, top_k, hidden):
                raise ValueError("slot values must be [tokens, top_k, hidden]")
            rows = sel
        selected_sum = np.zeros_like(res)
        for slot in range(top_k):
            selected_sum = (selected_sum + (rows[:, slot] * rw[:, slot, None]).astype(np.float32)).astype(np.float32)
        selected_sum = rnd(selected_sum)
    gate = np.asarray(gate_logits, dtype=np.float32)
    gate_first = gate if gate.ndim == 1 else gate[:, 0]
    if gate_first.shape != (tokens,):
        raise ValueError("gate_logits must be [tokens] or [tokens, gate_stride]")
    sig = (np.float32(1.0) / (np.float32(1.0) + np.exp(-gate_first))).astype(np.float32)
    combined = (res + selected_sum).astype(np.float32)
    combined = (combined + (sig[:, None] * sh).astype(np.float32)).astype(np.float32)
    rounded = rnd(combined)
    variance = np.mean(rounded * rounded, axis=-1, keepdims=True, dtype=np.float32)
    inv = np.reciprocal(np.sqrt(variance + np.float32(eps))).astype(np.float32)
    return rounded, rnd(((rounded * inv).astype(np.float32) * w).astype(np.float32))


# --------------------------------------------------------------------------
# activation quantizers  (device specifications)
# --------------------------------------------------------------------------

def _tree_sum32(groups: np.ndarray) -> np.ndarray:
    """Sum of the last axis (32 wide) in the order of a 32-lane ``shfl_down``
    tree: lane i += lane i+16, then +8, +4, +2, +1 (gguf_q4_k_gemv.hip:130-135)."""
    v = groups.astype(np.float32)
    width = 32
    while width > 1:
        width //= 2
        v = (v[..., :width] + v[..., width:2 * width]).astype(np.float32)
    return v[..., 0]


def quantize_q8_1(x) -> np.ndarray:
    """float32 rows -> 36-byte ``block_q8_1 {half d; half s; int8 qs[32]}``.

    GEMV convention (gguf_q4_k_gemv.hip:740-772): ``d = amax/127`` in float32,
    ``q = clamp(roundf(x/d), -128, 127)``, zero block -> zeros; ``d`` and the
    lane-tree sum of the raw inputs are stored as fp16.
    Returns uint8 ``[rows, K/32, 36]``.
    """
    xa = np.ascontiguousarray(x, dtype=np.float32)
    rows, k = xa.shape
    if k % Q8_1_BLOCK:
        raise ValueError("in_features must be a multiple of 32")
    g = xa.reshape(rows, k // 32, 32)
    amax = np.max(np.abs(g), axis=-1)
    d = (amax / np.float32(127.0)).astype(np.float32)
    safe = np.where(amax > 0, d, np.float32(1.0)).astype(np.float32)
    q = round_half_away((g / safe[..., None]).astype(np.float32))
    q = np.clip(q, -128, 127)
    q = np.where(amax[..., None] > 0, q, 0).astype(np.int8)
    out = np.empty((rows, k // 32, Q8_1_BLOCK_BYTES), dtype=np.uint8)
    out[..., 0:2] = d.astype(np.float16)[..., None].view(np.uint8)
    out[..., 2:4] = _tree_sum32(g).astype(np.float16)[..., None].view(np.uint8)
    out[..., 4:] = q.view(np.uint8)
    return out


def quantize_q8_1x2(x) -> np.ndarray:
    """Two planes of q8_1 blocks, uint8 ``[2, rows, K/32, 36]`` (gguf_q4_k_gemv.hip:777-829): plane 0 is
    ``quantize_q8_1(x)``; plane 1 the same quantization of the residual ``x - float(half d0) * q0``."""
    xa = np.ascontiguousarray(x, dtype=np.float32)
    p0 = quantize_q8_1(xa)
    d0, _, q0 = q8_1_fields(p0)
    residual = (xa.reshape(q0.shape) - (d0[..., None] * q0.astype(np.float32)).astype(np.float32)).astype(np.float32)
    return np.stack([p0, quantize_q8_1(residual.reshape(xa.shape))])


def q8_1_fields(xq) -> tuple[np.ndarray, np.ndarray, np.ndarray]:
    """36-byte blocks -> (d float32 [rows,nb], s float32 [rows,nb], qs int8 [rows,nb,32])."""
    b = np.ascontiguousarray(xq, dtype=np.uint8)
    b = b.reshape(b.shape[0], -1, Q8_1_BLOCK_BYTES)
    d = np.ascontiguousarray(b[..., 0:2]).view(np.float16)[..., 0].astype(np.float32)
    s = np.ascontiguousarray(b[..., 2:4]).view(np.float16)[..., 0].astype(np.float32)
    qs = np.ascontiguousarray(b[..., 4:]).view(np.int8)
    return d, s, qs


def dequantize_q8_1(xq) -> np.ndarray:
    """Activation values a q8_1 consumer sees: ``float(half d) * q``."""
    d, _, qs = q8_1_fields(xq)
    return (d[..., None] * qs.astype(np.float32)).reshape(qs.shape[0], -1)


def pack_q8_1_ds4(x_bf16_bits) -> np.ndarray:
    """bf16 rows -> 144-byte DS4 blocks ``{half ds4[8]; int8 qs[128]}``.

    MMQ convention (``pack_q8_1_mmq_ds4_from_bf16`` gguf_q4_k.py:1288-1319; device
    gguf_q4_k_q8_1_selected_prefill.hip:627-690): per 32 values
    ``scale = min(65504, amax/127)``, ``q = clamp(rint(x/scale), -127, 127)``
    (ties to even), ``ds4[2g] = half(scale)``, ``ds4[2g+1] = half(clamp(sum))``.
    The sum uses the 32-lane shfl_down tree order of the device kernel.
    Returns uint8 ``[rows, K/128, 144]``.
    """
    xa = bf16_bits_to_f32(np.ascontiguousarray(x_bf16_bits, dtype=np.uint16))
    rows, k = xa.shape
    if k % DS4_BLOCK:
        raise ValueError("hidden must be a multiple of 128")
    g = xa.reshape(rows, k // DS4_BLOCK, 4, 32)
    amax = np.max(np.abs(g), axis=-1)
    scale = np.minimum(FP16_MAX, (amax / np.float32(127.0)).astype(np.float32))
    safe = np.where(scale > 0, scale, np.float32(1.0)).astype(np.float32)
    q = np.rint((g / safe[..., None]).astype(np.float32))
    q = np.clip(q, -127, 127)
    q = np.where(scale[..., None] > 0, q, 0).astype(np.int8)
    sums = np.clip(_tree_sum32(g), -FP16_MAX, FP16_MAX).astype(np.float32)
    out = np.empty((rows, k // DS4_BLOCK, DS4_BLOCK_BYTES), dtype=np.uint8)
    ds = np.empty((rows, k // DS4_BLOCK, 4, 2), dtype=np.float16)
    ds[..., 0] = scale.astype(np.float16)
    ds[..., 1] = sums.astype(np.float16)
    out[..., :16] = ds.reshape(rows, k // DS4_BLOCK, 8).view(np.uint8)
    out[..., 16:] = q.reshape(rows, k // DS4_BLOCK, 128).view(np.uint8)
    return out


def ds4_fields(xds4) -> tuple[np.ndarray, np.ndarray, np.ndarray]:
    """DS4 blocks -> (scale [rows,K/32], sum [rows,K/32], qs int8 [rows,K/32,32])."""
    b = np.ascontiguousarray(xds4, dtype=np.uint8)
    rows = b.shape[0]
    b = b.reshape(rows, -1, DS4_BLOCK_BYTES)
    ds = np.ascontiguousarray(b[..., :16]).view(np.float16).astype(np.float32).reshape(rows, -1, 4, 2)
    qs = np.ascontiguousarray(b[..., 16:]).view(np.int8).reshape(rows, -1, 32)
    return ds[..., 0].reshape(rows, -1), ds[..., 1].reshape(rows, -1), qs


def pack_q8_1_d4s4(x_bf16_bits) -> np.ndarray:
    """bf16 rows -> 160-byte D4S4 blocks ``{float d4[4]; float s4[4]; int8 qs[128]}``.

    (gguf_k_mmq_prefill.hip:50-56,264-307): float32 ``d = amax/127``,
    ``q = clamp(roundf(x/d), -128, 127)``; the sum is four sequential adds per
    lane followed by an xor tree over 8 lanes (4, 2, 1).
    """
    xa = bf16_bits_to_f32(np.ascontiguousarray(x_bf16_bits, dtype=np.uint16))
    rows, k = xa.shape
    if k % DS4_BLOCK:
        raise ValueError("hidden must be a multiple of 128")
    g = xa.reshape(rows, k // DS4_BLOCK, 4, 32)
    amax = np.max(np.abs(g), axis=-1)
    d = np.where(amax > 0, (amax / np.float32(127.0)).astype(np.float32), np.float32(0.0)).astype(np.float32)
    safe = np.where(d > 0, d, np.float32(1.0)).astype(np.float32)
    q = np.clip(round_half_away((g / safe[..., None]).astype(np.float32)), -128, 127)
    q = np.where(d[..., None] > 0, q, 0).astype(np.int8)
    lanes = g.reshape(rows, k // DS4_BLOCK, 4, 8, 4)
    part = ((lanes[..., 0] + lanes[..., 1]).astype(np.float32) + lanes[..., 2]).astype(np.float32)
    part = (part + lanes[..., 3]).astype(np.float32)                       # [.., 8]
    part = (part[..., :4] + part[..., 4:]).astype(np.float32)
    part = (part[..., :2] + part[..., 2:]).astype(np.float32)
    sums = (part[..., 0] + part[..., 1]).astype(np.float32)
    out = np.empty((rows, k // DS4_BLOCK, D4S4_BLOCK_BYTES), dtype=np.uint8)
    out[..., 0:16] = d.view(np.uint8).reshape(rows, -1, 16)
    out[..., 16:32] = sums.view(np.uint8).reshape(rows, -1, 16)
    out[..., 32:] = q.reshape(rows, -1, 128).view(np.uint8)
    return out


def d4s4_fields(xd4s4) -> tuple[np.ndarray, np.ndarray, np.ndarray]:
    b = np.ascontiguousarray(xd4s4, dtype=np.uint8)
    rows = b.shape[0]
    b = b.reshape(rows, -1, D4S4_BLOCK_BYTES)
    d = np.ascontiguousarray(b[..., 0:16]).view(np.float32).reshape(rows, -1)
    s = np.ascontiguousarray(b[..., 16:32]).view(np.float32).reshape(rows, -1)
    qs = np.ascontiguousarray(b[..., 32:]).view(np.int8).reshape(rows, -1, 32)
    return d, s, qs


# --------------------------------------------------------------------------
# integer sub-block dots and the q8_1 combine formulas
# --------------------------------------------------------------------------

def block_dots_q4_k(qs_i8: np.ndarray, qweight: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """Per 32-wide sub-block: ``dot[r,n,j] = sum q4*q8`` and ``qsum[r,j] = sum q8``
    as int32 (gguf_q4_k_gemv.hip:893-904).  ``qs_i8`` is ``[rows, K/32, 32]``."""
    n = qweight.shape[0]
    blocks, _ = _as_blocks(qweight, Q4_K_BLOCK_BYTES)
    q4 = q4_k_quants(blocks).reshape(n, -1, 32).astype(np.int32)
    a = qs_i8.astype(np.int32)
    dots = np.einsum("rjk,njk->rnj", a, q4, optimize=True).astype(np.int32)
    return dots, a.sum(axis=-1, dtype=np.int32)


def block_dots_q5_k(qs_i8: np.ndarray, qweight: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """Per 32-wide sub-block ``dot[r,n,j] = sum q5*q8`` and ``qsum[r,j] = sum q8`` as int32
    (Q5_K through the Q4_K q8_1 formula with 5-bit quants, gguf_k_gemv.hip:115-137)."""
    n = qweight.shape[0]
    blocks, _ = _as_blocks(qweight, Q5_K_BLOCK_BYTES)
    q5 = q5_k_quants(blocks).reshape(n, -1, 32).astype(np.int32)
    a = qs_i8.astype(np.int32)
    dots = np.einsum("rjk,njk->rnj", a, q5, optimize=True).astype(np.int32)
    return dots, a.sum(axis=-1, dtype=np.int32)


def block_dots_q6_k(qs_i8: np.ndarray, qweight: np.ndarray) -> np.ndarray:
    """Per 16-wide sub-block: ``dot = sum u6*q8 - 32*sum q8 = sum (u6-32)*q8``
    as int32 ``[rows, N, K/16]`` (gguf_k_gemv.hip:233-246)."""
    n = qweight.shape[0]
    blocks, _ = _as_blocks(qweight, Q6_K_BLOCK_BYTES)
    q6 = q6_k_quants(blocks).reshape(n, -1, 16).astype(np.int32)
    a = qs_i8.reshape(qs_i8.shape[0], -1, 16).astype(np.int32)
    return np.einsum("rjk,njk->rnj", a, q6, optimize=True).astype(np.int32)


def block_dots_q8_0(qs_i8: np.ndarray, qweight: np.ndarray) -> np.ndarray:
    """Per 32-wide block ``dot = sum w8*q8`` as int32 (gguf_q8_0_dp4a_gemv.hip:122-129)."""
    n = qweight.shape[0]
    blocks, _ = _as_blocks(qweight, Q8_0_BLOCK_BYTES)
    w = blocks[:, 2:34].view(np.int8).reshape(n, -1, 32).astype(np.int32)
    return np.einsum("rjk,njk->rnj", qs_i8.astype(np.int32), w, optimize=True).astype(np.int32)


def _q4_k_scales_f32(qweight: np.ndarray, block_bytes: int = Q4_K_BLOCK_BYTES) -> tuple[np.ndarray, np.ndarray]:
    """(d*sc, dmin*mn) per (row, sub-block) as float32 ``[N, K/32]``; Q5_K blocks carry the same 16-byte header."""
    n = qweight.shape[0]
    blocks, _ = _as_blocks(qweight, block_bytes)
    sc, mn = q4_k_scale_min(blocks[:, 4:16])
    ds = (_fp16_field(blocks, 0)[:, None] * sc.astype(np.float32)).astype(np.float32)
    dm = (_fp16_field(blocks, 2)[:, None] * mn.astype(np.float32)).astype(np.float32)
    return ds.reshape(n, -1), dm.reshape(n, -1)


def gemv_q8_1_q4_k(xq, qweight, dtype=np.float64) -> np.ndarray:
    """q8_1 x Q4_K GEMV: ``sum_j xd_j*(d*sc_j*dot_j - dmin*mn_j*qsum_j)`` with the
    integer q8 sum (gguf_q4_k_gemv.hip:893-904,
    gguf_q4_k_q8_1_dp4a_vdr_gemv.hip:212-228).  Evaluated in ``dtype``."""
    xd, _, qs = q8_1_fields(xq)
    dots, qsum = block_dots_q4_k(qs, np.asarray(qweight))
    ds, dm = _q4_k_scales_f32(np.asarray(qweight))
    t = ds[None].astype(dtype) * dots.astype(dtype) - dm[None].astype(dtype) * qsum[:, None, :].astype(dtype)
    return (xd[:, None, :].astype(dtype) * t).sum(axis=-1)


def gemv_q8_1_q6_k(xq, qweight, dtype=np.float64) -> np.ndarray:
    """q8_1 x Q6_K GEMV: ``sum xd*d*sc16*dot16`` (gguf_k_gemv.hip:233-246)."""
    xd, _, qs = q8_1_fields(xq)
    qw = np.asarray(qweight)
    n = qw.shape[0]
    blocks, _ = _as_blocks(qw, Q6_K_BLOCK_BYTES)
    sc = blocks[:, 192:208].view(np.int8).astype(np.float32)
    dsc = (_fp16_field(blocks, 208)[:, None] * sc).reshape(n, -1)          # [N, K/16]
    dots = block_dots_q6_k(qs, qw)                                         # [r, N, K/16]
    xd16 = np.repeat(xd, 2, axis=-1)
    return (xd16[:, None, :].astype(dtype) * dsc[None].astype(dtype) * dots.astype(dtype)).sum(axis=-1)


def gemv_q8_1_q8_0(xq, qweight, dtype=np.float64) -> np.ndarray:
    """q8_1 x Q8_0 GEMV: ``sum wd*xd*dot`` (gguf_q8_0_dp4a_gemv.hip:100-137)."""
    xd, _, qs = q8_1_fields(xq)
    qw = np.asarray(qweight)
    n = qw.shape[0]
    blocks, _ = _as_blocks(qw, Q8_0_BLOCK_BYTES)
    wd = _fp16_field(blocks, 0).reshape(n, -1)
    dots = block_dots_q8_0(qs, qw)
    return (wd[None].astype(dtype) * xd[:, None, :].astype(dtype) * dots.astype(dtype)).sum(axis=-1)


def mmq_q4_k_ds4(xds4, qweight, dtype=np.float64) -> np.ndarray:
    """DS4 x Q4_K MMQ: ``sum_j (d*sc_j)*xd_j*dot_j - (dmin*mn_j)*xsum_j`` with the
    fp16 raw sum (gguf_q4_k_q8_1_mmq_prefill.hip:265-276; NumPy preview
    gguf_q4_k.py:1376-1406)."""
    xd, xs, qs = ds4_fields(xds4)
    qw = np.asarray(qweight)
    dots, _ = block_dots_q4_k(qs, qw)
    ds, dm = _q4_k_scales_f32(qw)
    main = (ds[None].astype(dtype) * xd[:, None, :].astype(dtype) * dots.astype(dtype)).sum(axis=-1)
    corr = xs.astype(dtype) @ dm.astype(dtype).T
    return main - corr


def mmq_q5_k_d4s4(xd4s4, qweight, dtype=np.float64) -> np.ndarray:
    """D4S4 x Q5_K MMQ: ``sum_j xd_j*(d*sc_j)*dot_j - (dmin*mn_j)*s4_j`` with the float32 raw sum of the
    32 activation values (gguf_k_mmq_prefill.hip:563-572 scales, :655-664 combine)."""
    xd, xs, qs = d4s4_fields(xd4s4)
    qw = np.asarray(qweight)
    dots, _ = block_dots_q5_k(qs, qw)
    ds, dm = _q4_k_scales_f32(qw, Q5_K_BLOCK_BYTES)
    main = (ds[None].astype(dtype) * xd[:, None, :].astype(dtype) * dots.astype(dtype)).sum(axis=-1)
    return main - xs.astype(dtype) @ dm.astype(dtype).T


def mmq_q8_0_d4s4(xd4s4, qweight, dtype=np.float64) -> np.ndarray:
    """D4S4 x Q8_0 MMQ: ``sum_b xd_b * wd_b * dot_b`` over the 32-value blocks: the q8_1 x Q8_0 formula
    (gguf_q8_0_dp4a_gemv.hip:100-137) with the float32 activation scales of the D4S4 block
    (gguf_k_mmq_prefill.hip:655-664).  hipEngine has no such kernel; pinned by the float64 product of the
    dequantized weight with the dequantized activations."""
    xd, _, qs = d4s4_fields(xd4s4)
    qw = np.asarray(qweight)
    n = qw.shape[0]
    blocks, _ = _as_blocks(qw, Q8_0_BLOCK_BYTES)
    wd = _fp16_field(blocks, 0).reshape(n, -1)
    dots = block_dots_q8_0(qs, qw)
    return (wd[None].astype(dtype) * xd[:, None, :].astype(dtype) * dots.astype(dtype)).sum(axis=-1)


def mmq_q6_k_d4s4(xd4s4, qweight, dtype=np.float64) -> np.ndarray:
    """D4S4 x Q6_K MMQ: ``sum_g xd_g*(s0*dot0 + s1*dot1)``
    (gguf_k_mmq_prefill.hip:652-667)."""
    xd, _, qs = d4s4_fields(xd4s4)
    qw = np.asarray(qweight)
    n = qw.shape[0]
    blocks, _ = _as_blocks(qw, Q6_K_BLOCK_BYTES)
    sc = blocks[:, 192:208].view(np.int8).astype(np.float32)
    dsc = (_fp16_field(blocks, 208)[:, None] * sc).reshape(n, -1)
    dots = block_dots_q6_k(qs, qw)
    xd16 = np.repeat(xd, 2, axis=-1)
    return (xd16[:, None, :].astype(dtype) * dsc[None].astype(dtype) * dots.astype(dtype)).sum(axis=-1)


# --------------------------------------------------------------------------
# routing
# --------------------------------------------------------------------------

def router_logits(hidden, weight) -> np.ndarray:
    """``logits[t, e] = hidden[t] . weight[e]`` as a float32 matmul of float32 values
    (kernels/cpu_reference/ops.py:609, the first step of the routing reference)."""
    return np.matmul(np.asarray(hidden, dtype=np.float32), np.asarray(weight, dtype=np.float32).T).astype(np.float32)


def router_topk_softmax(logits, top_k: int) -> tuple[np.ndarray, np.ndarray]:
    """Device router (moe/router.hip:628-715): iterative argmax on the logits
    (strict ``>``, so ties go to the lowest index), then a softmax over the
    ``top_k`` selected logits.  Returns (selected int64 [T,k], weights f32 [T,k])."""
    lg = np.asarray(logits, dtype=np.float32)
    order = np.argsort(-lg, axis=-1, kind="stable")[:, :top_k].astype(np.int64)
    vals = np.take_along_axis(lg, order, axis=-1)
    e = np.exp((vals - vals[:, :1]).astype(np.float32)).astype(np.float32)
    denom = np.maximum(e.sum(axis=-1, keepdims=True, dtype=np.float32), np.float32(1e-20))
    return order, (e / denom).astype(np.float32)


def mtp_moe_routing(logits, top_k: int, scale: float = 1.0) -> tuple[np.ndarray, np.ndarray]:
    """CPU-backend routing (ops.py:575-621) from precomputed logits: softmax over
    all experts, stable top-k of the probabilities, renormalize (floor 2^-14),
    optional scale."""
    lg = np.asarray(logits, dtype=np.float32)
    z = lg - lg.max(axis=-1, keepdims=True)
    p = np.exp(z).astype(np.float32)
    p = (p / p.sum(axis=-1, keepdims=True)).astype(np.float32)
    sel = np.argsort(-p, axis=-1, kind="stable")[:, :top_k].astype(np.int64)
    w = np.take_along_axis(p, sel, axis=-1).astype(np.float32)
    w = (w / np.maximum(w.sum(axis=-1, keepdims=True), np.float32(6.103515625e-5))).astype(np.float32)
    if scale not in (0.0, 1.0):
        w = (w * np.float32(scale)).astype(np.float32)
    return sel, w


def build_routing_index(selected, routing, num_experts: int, pad_multiple: int = 1) -> dict:
    """Expert-major routing index (moe/group_scatter.hip:9-141,328-389).

    ``selected``/``routing`` are ``[T, top_k]`` (or flat ``[T*top_k]`` with
    ``top_k`` inferred as 1).  Lane = ``t*top_k + slot``.  Within an expert the
    lanes keep ascending order (the stable compact variants).  Out-of-range
    expert ids are dropped, as the device kernels do.
    """
    sel = np.asarray(selected, dtype=np.int64)
    top_k = sel.shape[1] if sel.ndim == 2 else 1
    flat = sel.reshape(-1)
    w = np.asarray(routing, dtype=np.float32).reshape(-1)
    valid = (flat >= 0) & (flat < num_experts)
    lanes = np.nonzero(valid)[0].astype(np.int64)
    order = lanes[np.argsort(flat[lanes], kind="stable")]
    counts = np.bincount(flat[lanes], minlength=num_experts).astype(np.int64)
    padded = counts if pad_multiple <= 1 else (counts + pad_multiple - 1) // pad_multiple * pad_multiple
    start = np.zeros(num_experts + 1, dtype=np.int64)
    np.cumsum(padded, out=start[1:])
    total = int(start[-1])
    sorted_lanes = np.full(total, -1, dtype=np.int64)
    sorted_experts = np.full(total, -1, dtype=np.int64)
    sorted_weights = np.zeros(total, dtype=np.float32)
    pos = 0
    for e in range(num_experts):
        c = int(counts[e])
        if c:
            dst = int(start[e])
            sorted_lanes[dst:dst + c] = order[pos:pos + c]
            sorted_experts[dst:dst + c] = e
            sorted_weights[dst:dst + c] = w[order[pos:pos + c]]
            pos += c
    compact_to_source = np.where(sorted_lanes >= 0, sorted_lanes // top_k, -1)
    active = np.nonzero(counts)[0].astype(np.int64)
    return {
        "counts": counts.astype(np.int32),
        "expert_start": start,
        "sorted_lanes": sorted_lanes,
        "sorted_experts": sorted_experts,
        "sorted_weights": sorted_weights,
        "compact_to_source": compact_to_source,
        "active_experts": active,
        "active_count": int(active.size),
        "total": total,
        "top_k": top_k,
    }


def tile_map(expert_start, num_experts: int, tile_rows: int, tile_capacity: int = 0) -> dict:
    """Per-expert row ranges rounded up to ``tile_rows`` and the tile -> expert map,
    ``-1`` padded (moe/group_scatter.hip:328-389)."""
    es = np.asarray(expert_start, dtype=np.int64)
    counts = es[1:num_experts + 1] - es[:num_experts]
    padded = (counts + tile_rows - 1) // tile_rows * tile_rows
    start = np.zeros(num_experts + 1, dtype=np.int64)
    np.cumsum(padded, out=start[1:])
    tiles = int(start[-1] // tile_rows)
    cap = tile_capacity if tile_capacity > 0 else tiles
    te = np.full(cap, -1, dtype=np.int64)
    for e in range(num_experts):
        lo, hi = int(start[e] // tile_rows), int(start[e + 1] // tile_rows)
        te[lo:min(hi, cap)] = e
    return {"tile_expert_start": start, "tile_expert": te, "total": int(start[-1])}


# --------------------------------------------------------------------------
# synthetic block generators
# --------------------------------------------------------------------------

def _f16_bytes(values: np.ndarray) -> np.ndarray:
    return np.ascontiguousarray(values, dtype=np.float16)[..., None].view(np.uint8)


def closed_form_q4_k(out_features: int, in_features: int) -> np.ndarray:
    """Closed-form Q4_K weight of the reference tests, vectorized.  Block
    (o, b): ``d = 2^-6*(1+o%5)``, ``dmin = 2^-7*(1+b%3)``,
    ``sc_j = (3j+o+b)%63+1``, ``mn_j = (5j+2o+b)%17``, ``q_k = (k+7o+11b)%16``
    (tests/_gguf_synthetic_weights.py:38-80)."""
    if in_features % QK_K:
        raise ValueError("in_features must be a multiple of 256")
    nb = in_features // QK_K
    o = np.arange(out_features, dtype=np.int64)[:, None]
    b = np.arange(nb, dtype=np.int64)[None, :]
    j = np.arange(8, dtype=np.int64)
    k = np.arange(QK_K, dtype=np.int64)
    sc = ((3 * j + (o + b)[..., None]) % 63 + 1).astype(np.uint8)
    mn = ((5 * j + (2 * o + b)[..., None]) % 17).astype(np.uint8)
    q = ((k + (7 * o + 11 * b)[..., None]) % 16).astype(np.uint8).reshape(out_features, nb, 4, 2, 32)
    blk = np.empty((out_features, nb, Q4_K_BLOCK_BYTES), dtype=np.uint8)
    blk[..., 0:2] = _f16_bytes(np.broadcast_to(0.015625 * (1 + o % 5), (out_features, nb)))
    blk[..., 2:4] = _f16_bytes(np.broadcast_to(0.0078125 * (1 + b % 3), (out_features, nb)))
    blk[..., 4:16] = pack_q4_k_scale_min(sc.reshape(-1, 8), mn.reshape(-1, 8)).reshape(out_features, nb, 12)
    blk[..., 16:] = (q[..., 0, :] | (q[..., 1, :] << 4)).reshape(out_features, nb, 128)
    return blk.reshape(out_features, nb * Q4_K_BLOCK_BYTES)


def pack_q5_k_blocks(q5: np.ndarray, sc: np.ndarray, mn: np.ndarray, d: np.ndarray, dmin: np.ndarray) -> np.ndarray:
    """Inverse of :func:`q5_k_quants` + header: ``q5`` [n,8,32] in 0..31, ``sc``/``mn`` [n,8] 6-bit,
    ``d``/``dmin`` [n] -> [n,176] block bytes (builder of tests/_gguf_synthetic_weights.py:81-108)."""
    q5 = np.asarray(q5, dtype=np.uint8)
    n = q5.shape[0]
    blk = np.empty((n, Q5_K_BLOCK_BYTES), dtype=np.uint8)
    blk[:, 0:2] = _f16_bytes(d)
    blk[:, 2:4] = _f16_bytes(dmin)
    blk[:, 4:16] = pack_q4_k_scale_min(sc, mn)
    qh = np.zeros((n, 32), dtype=np.uint8)
    for sb in range(8):
        qh |= ((q5[:, sb] >> 4) & 1) << sb
    blk[:, 16:48] = qh
    lo = q5 & 0x0F
    blk[:, 48:176] = (lo[:, 0::2] | (lo[:, 1::2] << 4)).reshape(n, 128)
    return blk


def closed_form_q5_k(out_features: int, in_features: int) -> np.ndarray:
    """Closed-form Q5_K weight of the reference tests, vectorized.  Block (o, b): ``d``, ``dmin``,
    ``sc_j``, ``mn_j`` as in :func:`closed_form_q4_k`, ``q_k = (k+13o+17b)%32``
    (tests/_gguf_synthetic_weights.py:81-121)."""
    if in_features % QK_K:
        raise ValueError("in_features must be a multiple of 256")
    nb = in_features // QK_K
    o = np.repeat(np.arange(out_features, dtype=np.int64), nb)
    b = np.tile(np.arange(nb, dtype=np.int64), out_features)
    j = np.arange(8, dtype=np.int64)
    k = np.arange(QK_K, dtype=np.int64)
    sc = ((3 * j + (o + b)[:, None]) % 63 + 1).astype(np.uint8)
    mn = ((5 * j + (2 * o + b)[:, None]) % 17).astype(np.uint8)
    q = ((k + (13 * o + 17 * b)[:, None]) % 32).astype(np.uint8).reshape(-1, 8, 32)
    blk = pack_q5_k_blocks(q, sc, mn, 0.015625 * (1 + o % 5), 0.0078125 * (1 + b % 3))
    return blk.reshape(out_features, nb * Q5_K_BLOCK_BYTES)


def pack_q6_k_blocks(q_signed: np.ndarray, scales_i8: np.ndarray, d: np.ndarray) -> np.ndarray:
    """(q in [-32,31] [n,256], int8 scales [n,16], d [n]) -> [n,210] block bytes,
    the inverse of :func:`q6_k_quants` (tests/_gguf_synthetic_weights.py:123-158)."""
    n = q_signed.shape[0]
    u = (np.asarray(q_signed, dtype=np.int16) + 32).astype(np.uint8).reshape(n, 8, 32)
    blk = np.zeros((n, Q6_K_BLOCK_BYTES), dtype=np.uint8)
    ql = blk[:, 0:128].reshape(n, 2, 2, 32)
    qh = blk[:, 128:192].reshape(n, 2, 32)
    for g in range(8):
        half, which, upper = g >> 2, g & 1, (g >> 1) & 1
        ql[:, half, which] |= (u[:, g] & 0x0F) << (4 * upper)
        qh[:, half] |= ((u[:, g] >> 4) & 0x03) << (2 * (g & 3))
    blk[:, 192:208] = np.asarray(scales_i8, dtype=np.int8).view(np.uint8)
    blk[:, 208:210] = _f16_bytes(np.asarray(d))
    return blk


def closed_form_q6_k(out_features: int, in_features: int) -> np.ndarray:
    """Closed-form Q6_K weight of the reference tests: ``d = 2^-7*(1+o%7)``,
    ``sc_i = (3i+o+b)%33-16``, ``q_k = (k+11o+19b)%64-32``
    (tests/_gguf_synthetic_weights.py:123-172)."""
    if in_features % QK_K:
        raise ValueError("in_features must be a multiple of 256")
    nb = in_features // QK_K
    o = np.arange(out_features, dtype=np.int64)[:, None]
    b = np.arange(nb, dtype=np.int64)[None, :]
    i = np.arange(16, dtype=np.int64)
    k = np.arange(QK_K, dtype=np.int64)
    sc = (((3 * i + (o + b)[..., None]) % 33) - 16).astype(np.int8)
    q = (((k + (11 * o + 19 * b)[..., None]) % 64) - 32).astype(np.int8)
    d = np.broadcast_to(0.0078125 * (1 + o % 7), (out_features, nb))
    blk = pack_q6_k_blocks(q.reshape(-1, QK_K), sc.reshape(-1, 16), d.reshape(-1))
    return blk.reshape(out_features, nb * Q6_K_BLOCK_BYTES)


def closed_form_q8_0(out_features: int, in_features: int) -> np.ndarray:
    """Closed-form Q8_0 weight of the reference tests: ``d = 2^-5*(1+o%5)``,
    ``q_k = (k+7o+3b)%31-15`` (tests/_gguf_synthetic_weights.py:175-190)."""
    if in_features % 32:
        raise ValueError("in_features must be a multiple of 32")
    nb = in_features // 32
    o = np.arange(out_features, dtype=np.int64)[:, None]
    b = np.arange(nb, dtype=np.int64)[None, :]
    k = np.arange(32, dtype=np.int64)
    q = (((k + (7 * o + 3 * b)[..., None]) % 31) - 15).astype(np.int8)
    blk = np.empty((out_features, nb, Q8_0_BLOCK_BYTES), dtype=np.uint8)
    blk[..., 0:2] = _f16_bytes(np.broadcast_to(0.03125 * (1 + o % 5), (out_features, nb)))
    blk[..., 2:] = q.view(np.uint8)
    return blk.reshape(out_features, nb * Q8_0_BLOCK_BYTES)


def stack_experts(base: np.ndarray, num_experts: int, seed: int = 1) -> np.ndarray:
    """Expert e = rows of ``base`` rolled by ``e + seed``
    (tests/test_unit_cpu_reference_moe_ffn.py:53-55)."""
    return np.stack([np.roll(base, e + seed, axis=0) for e in range(num_experts)], axis=0)


def quantize_q8_0(w) -> np.ndarray:
    """fp32 [N,K] -> Q8_0 bytes: ``d = amax/127``, ``q = rint(w/d)``
    (scripts/laguna_f16_decode_q8_screen.py:94-121 style)."""
    wa = np.ascontiguousarray(w, dtype=np.float32)
    n, k = wa.shape
    g = wa.reshape(n, k // 32, 32)
    amax = np.max(np.abs(g), axis=-1)
    d = (amax / np.float32(127.0)).astype(np.float16)
    df = d.astype(np.float32)
    safe = np.where(df > 0, df, np.float32(1.0))
    q = np.clip(np.rint(g / safe[..., None]), -127, 127)
    q = np.where(df[..., None] > 0, q, 0).astype(np.int8)
    blk = np.empty((n, k // 32, Q8_0_BLOCK_BYTES), dtype=np.uint8)
    blk[..., 0:2] = d[..., None].view(np.uint8)
    blk[..., 2:] = q.view(np.uint8)
    return blk.reshape(n, -1)


def quantize_q4_k(w) -> np.ndarray:
    """fp32 [N,K] -> Q4_K bytes.  PARITY UNPINNED (the reference has no such
    quantizer); a min/max affine fit per 32-wide sub-block followed by 6-bit
    quantization of the sub-block scales and mins against the per-block
    maxima, in the spirit of ggml's reference quantizer.  Only the block
    bytes it emits take part in parity."""
    wa = np.ascontiguousarray(w, dtype=np.float32)
    n, k = wa.shape
    if k % QK_K:
        raise ValueError("in_features must be a multiple of 256")
    nb = k // QK_K
    g = wa.reshape(n * nb, 8, 32)
    lo = np.minimum(g.min(axis=-1), 0.0)
    hi = g.max(axis=-1)
    sub_scale = np.maximum(hi - lo, 0.0) / np.float32(15.0)
    sub_min = -lo
    d = (sub_scale.max(axis=-1) / np.float32(63.0)).astype(np.float16)
    dmin = (sub_min.max(axis=-1) / np.float32(63.0)).astype(np.float16)
    df, dmf = d.astype(np.float32), dmin.astype(np.float32)
    sc = np.where(df[:, None] > 0, np.rint(sub_scale / np.where(df > 0, df, 1.0)[:, None]), 0)
    mn = np.where(dmf[:, None] > 0, np.rint(sub_min / np.where(dmf > 0, dmf, 1.0)[:, None]), 0)
    sc = np.clip(sc, 0, 63).astype(np.uint8)
    mn = np.clip(mn, 0, 63).astype(np.uint8)
    eff_scale = df[:, None] * sc.astype(np.float32)
    eff_min = dmf[:, None] * mn.astype(np.float32)
    q = np.where(eff_scale[..., None] > 0,
                 np.rint((g + eff_min[..., None]) / np.where(eff_scale > 0, eff_scale, 1.0)[..., None]), 0)
    q = np.clip(q, 0, 15).astype(np.uint8).reshape(n * nb, 4, 2, 32)
    blk = np.empty((n * nb, Q4_K_BLOCK_BYTES), dtype=np.uint8)
    blk[:, 0:2] = d[:, None].view(np.uint8)
    blk[:, 2:4] = dmin[:, None].view(np.uint8)
    blk[:, 4:16] = pack_q4_k_scale_min(sc, mn)
    blk[:, 16:] = (q[:, :, 0] | (q[:, :, 1] << 4)).reshape(n * nb, 128)
    return blk.reshape(n, nb * Q4_K_BLOCK_BYTES)


def quantize_q6_k(w) -> np.ndarray:
    """fp32 [N,K] -> Q6_K bytes.  PARITY UNPINNED (no reference quantizer):
    symmetric per-16 scale ``amax/32`` quantized to int8 against the block
    maximum, ``q = clamp(rint(w/(d*sc)), -32, 31)``."""
    wa = np.ascontiguousarray(w, dtype=np.float32)
    n, k = wa.shape
    if k % QK_K:
        raise ValueError("in_features must be a multiple of 256")
    nb = k // QK_K
    g = wa.reshape(n * nb, 16, 16)
    sub = np.max(np.abs(g), axis=-1) / np.float32(32.0)
    d = (sub.max(axis=-1) / np.float32(127.0)).astype(np.float16)
    df = d.astype(np.float32)
    sc = np.where(df[:, None] > 0, np.rint(sub / np.where(df > 0, df, 1.0)[:, None]), 0)
    sc = np.clip(sc, -128, 127).astype(np.int8)
    eff = df[:, None] * sc.astype(np.float32)
    q = np.where(eff[..., None] != 0, np.rint(g / np.where(eff != 0, eff, 1.0)[..., None]), 0)
    q = np.clip(q, -32, 31).astype(np.int8).reshape(n * nb, QK_K)
    return pack_q6_k_blocks(q, sc, df).reshape(n, nb * Q6_K_BLOCK_BYTES)


_QUANTIZE = {GGML_Q8_0: quantize_q8_0, GGML_Q4_K: quantize_q4_k, GGML_Q6_K: quantize_q6_k}


def random_weight(qtype: int, out_features: int, in_features: int, seed: int,
                  std: float = 0.02, chunk_rows: int = 4096) -> np.ndarray:
    """Seeded fp32 ``N(0, std)`` rows quantized with the oracle's own quantizer,
    generated ``chunk_rows`` at a time."""
    rng = np.random.default_rng(seed)
    block_size, type_size = _BLOCK_GEOMETRY[int(qtype)]
    out = np.empty((out_features, in_features // block_size * type_size), dtype=np.uint8)
    for lo in range(0, out_features, chunk_rows):
        hi = min(out_features, lo + chunk_rows)
        w = rng.standard_normal((hi - lo, in_features), dtype=np.float32) * np.float32(std)
        out[lo:hi] = _QUANTIZE[int(qtype)](w)
    return out


# --------------------------------------------------------------------------
# comparison metrics
# --------------------------------------------------------------------------

def max_rel_err(got, want, floor_frac: float = 1e-3) -> float:
    """``max |a-b| / max(|b|, floor_frac*max|b|)``: relative error with a magnitude
    floor so outputs that cancel to ~0 do not dominate (reference precedent:
    kernels/cpu_reference/fixtures.py:94-101)."""
    a = np.asarray(got, dtype=np.float64)
    b = np.asarray(want, dtype=np.float64)
    floor = floor_frac * float(np.max(np.abs(b))) if b.size else 0.0
    den = np.maximum(np.abs(b), max(floor, 1e-30))
    return float(np.max(np.abs(a - b) / den)) if b.size else 0.0


def cosine(got, want) -> float:
    a = np.asarray(got, dtype=np.float64).ravel()
    b = np.asarray(want, dtype=np.float64).ravel()
    den = float(np.linalg.norm(a) * np.linalg.norm(b))
    return float(a @ b / den) if den else 1.0


def softmax_kl_top1(ref, cand) -> tuple[float, float]:
    """Max row KL(softmax(ref) || softmax(cand)) and top-1 agreement
    (tests/test_gpu_gguf_x8_selected_gemv.py:204-219)."""
    r = np.asarray(ref, dtype=np.float64)
    c = np.asarray(cand, dtype=np.float64)

    def logsm(v):
        s = v - v.max(axis=-1, keepdims=True)
        return s - np.log(np.exp(s).sum(axis=-1, keepdims=True))

    lr, lc = logsm(r), logsm(c)
    kl = np.sum(np.exp(lr) * (lr - lc), axis=-1)
    return float(np.max(kl)), float(np.mean(r.argmax(axis=-1) == c.argmax(axis=-1)))
