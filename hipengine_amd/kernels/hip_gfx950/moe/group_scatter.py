"""Routing index of the MoE path: expert-major compaction of the selected lanes
and the 32-row tile map the grouped MMQ walks.

Signatures follow hipEngine's ``kernels/hip_gfx1100/moe/group_scatter.py``
(``qwen35_moe_group_compact_active`` :184-241, ``..._source_rows`` :243-308,
``qwen35_moe_mmq32_tile_map`` :423-462); registry keys as in :746-806.
All arguments are raw device pointers; int64 index arrays, float32 weights.
"""

from __future__ import annotations

import ctypes

from hipengine_amd.core.hip import HipRuntime
from hipengine_amd.kernels.hip_gfx950._launch import I64, VOID, check_launch, entry, validate_pointers
from hipengine_amd.kernels.registry import KernelKey, register

MAX_EXPERTS = 2048


def _check_num_experts(num_experts: int) -> None:
    if num_experts <= 0 or num_experts > MAX_EXPERTS:
        raise ValueError(f"num_experts must be in 1..{MAX_EXPERTS}")


def qwen35_moe_group_compact_active(selected_experts_ptr: int, routing_weights_ptr: int, expert_start_ptr: int,
                                    active_experts_ptr: int, active_count_ptr: int, sorted_lanes_ptr: int,
                                    sorted_experts_ptr: int, sorted_weights_ptr: int, total_lanes: int,
                                    num_experts: int, *, parallel: bool = False, stream: int = 0,
                                    library: ctypes.CDLL | None = None, runtime: HipRuntime | None = None) -> None:
    """Expert-major compaction: starts, active list, lanes (ascending within an
    expert), experts and weights in that order.  ``parallel`` is accepted for signature compatibility."""
    _check_num_experts(num_experts)
    if total_lanes <= 0:
        raise ValueError("total_lanes must be positive")
    validate_pointers(selected_experts_ptr=selected_experts_ptr, expert_start_ptr=expert_start_ptr,
                      sorted_lanes_ptr=sorted_lanes_ptr)
    fn = entry("hipengine_qwen35_moe_group_compact_active", [VOID] * 8 + [I64, I64, VOID], library)
    check_launch(fn(selected_experts_ptr, routing_weights_ptr, expert_start_ptr, active_experts_ptr, active_count_ptr,
                    sorted_lanes_ptr, sorted_experts_ptr, sorted_weights_ptr, total_lanes, num_experts, stream), runtime)


def qwen35_moe_group_compact_active_source_rows(selected_experts_ptr: int, routing_weights_ptr: int,
                                                expert_start_ptr: int, active_experts_ptr: int, active_count_ptr: int,
                                                sorted_lanes_ptr: int, compact_to_source_ptr: int,
                                                sorted_weights_ptr: int, total_lanes: int, num_experts: int,
                                                top_k: int, *, parallel: bool = False, stream: int = 0,
                                                library: ctypes.CDLL | None = None,
                                                runtime: HipRuntime | None = None) -> None:
    """The same with each compact row's source token (``lane // top_k``).
    ``parallel`` is accepted for signature compatibility: there is one kernel form here."""
    _check_num_experts(num_experts)
    if total_lanes <= 0 or top_k <= 0:
        raise ValueError("total_lanes and top_k must be positive")
    validate_pointers(selected_experts_ptr=selected_experts_ptr, expert_start_ptr=expert_start_ptr,
                      sorted_lanes_ptr=sorted_lanes_ptr)
    fn = entry("hipengine_qwen35_moe_group_compact_active_source_rows", [VOID] * 8 + [I64, I64, I64, VOID], library)
    check_launch(fn(selected_experts_ptr, routing_weights_ptr, expert_start_ptr, active_experts_ptr, active_count_ptr,
                    sorted_lanes_ptr, compact_to_source_ptr, sorted_weights_ptr, total_lanes, num_experts, top_k,
                    stream), runtime)


def moe_tile_map(expert_start_compact_ptr: int, tile_expert_start_ptr: int, tile_expert_ptr: int, total_ptr: int,
                 num_experts: int, *, tile_rows: int = 32, tile_capacity: int = 0, stream: int = 0,
                 library: ctypes.CDLL | None = None, runtime: HipRuntime | None = None) -> None:
    """``qwen35_moe_mmq32_tile_map`` for tiles of 32, 64 or 128 rows (C symbol ``hipengine_gfx950_moe_tile_map``)."""
    _check_num_experts(num_experts)
    if tile_rows not in (32, 64, 128):
        raise ValueError("tile_rows must be 32, 64 or 128")
    if tile_capacity < 0:
        raise ValueError("tile_capacity must be non-negative")
    validate_pointers(expert_start_compact_ptr=expert_start_compact_ptr, tile_expert_start_ptr=tile_expert_start_ptr,
                      tile_expert_ptr=tile_expert_ptr, total_ptr=total_ptr)
    fn = entry("hipengine_gfx950_moe_tile_map", [VOID] * 4 + [I64, I64, ctypes.c_int32, VOID], library)
    check_launch(fn(expert_start_compact_ptr, tile_expert_start_ptr, tile_expert_ptr, total_ptr, num_experts,
                    tile_capacity, tile_rows, stream), runtime)


def moe_group_compact_index(selected_experts_ptr: int, routing_weights_ptr: int, expert_start_ptr: int,
                            active_experts_ptr: int, active_count_ptr: int, sorted_lanes_ptr: int,
                            compact_to_source_ptr: int, sorted_weights_ptr: int, lane_to_compact_ptr: int,
                            total_lanes: int, num_experts: int, top_k: int, *, stream: int = 0,
                            library: ctypes.CDLL | None = None, runtime: HipRuntime | None = None) -> None:
    """``qwen35_moe_group_compact_active_source_rows`` and ``moe_lane_to_compact`` in the two launches of the former
    (C symbol ``hipengine_gfx950_moe_group_compact_index``): the same arrays, bit for bit."""
    _check_num_experts(num_experts)
    if total_lanes <= 0 or top_k <= 0:
        raise ValueError("total_lanes and top_k must be positive")
    validate_pointers(selected_experts_ptr=selected_experts_ptr, expert_start_ptr=expert_start_ptr,
                      sorted_lanes_ptr=sorted_lanes_ptr, lane_to_compact_ptr=lane_to_compact_ptr)
    fn = entry("hipengine_gfx950_moe_group_compact_index", [VOID] * 9 + [I64, I64, I64, VOID], library)
    check_launch(fn(selected_experts_ptr, routing_weights_ptr, expert_start_ptr, active_experts_ptr, active_count_ptr,
                    sorted_lanes_ptr, compact_to_source_ptr, sorted_weights_ptr, lane_to_compact_ptr, total_lanes,
                    num_experts, top_k, stream), runtime)


def qwen35_moe_mmq32_tile_map(expert_start_compact_ptr: int, mmq_expert_start_ptr: int, tile_expert_ptr: int,
                              mmq_total_ptr: int, num_experts: int, *, tile_capacity: int = 0, stream: int = 0,
                              library: ctypes.CDLL | None = None, runtime: HipRuntime | None = None) -> None:
    """Compact expert starts -> 32-row tile starts and the tile -> expert map."""
    _check_num_experts(num_experts)
    if tile_capacity < 0:
        raise ValueError("tile_capacity must be non-negative")
    validate_pointers(expert_start_compact_ptr=expert_start_compact_ptr, mmq_expert_start_ptr=mmq_expert_start_ptr,
                      tile_expert_ptr=tile_expert_ptr, mmq_total_ptr=mmq_total_ptr)
    fn = entry("hipengine_qwen35_moe_mmq32_tile_map", [VOID] * 4 + [I64, I64, VOID], library)
    check_launch(fn(expert_start_compact_ptr, mmq_expert_start_ptr, tile_expert_ptr, mmq_total_ptr, num_experts,
                    tile_capacity, stream), runtime)


def qwen35_moe_group_compact_active_parallel(*args, **kwargs) -> None:
    """hipEngine's parallel compaction (``moe/group_scatter.py:310-314``): the same arrays from the same kernels."""
    kwargs["parallel"] = True
    qwen35_moe_group_compact_active(*args, **kwargs)


def qwen35_moe_group_compact_active_source_rows_parallel(*args, **kwargs) -> None:
    """hipEngine's parallel compaction with source rows (``moe/group_scatter.py:372-379``)."""
    kwargs["parallel"] = True
    qwen35_moe_group_compact_active_source_rows(*args, **kwargs)


def qwen35_moe_group_compact_active_i32_parallel(selected_experts_ptr: int, routing_weights_ptr: int,
                                                 expert_start_ptr: int, active_experts_ptr: int, active_count_ptr: int,
                                                 sorted_lanes_ptr: int, sorted_experts_ptr: int, sorted_weights_ptr: int,
                                                 total_lanes: int, num_experts: int, *, stream: int = 0,
                                                 library: ctypes.CDLL | None = None,
                                                 runtime: HipRuntime | None = None) -> None:
    """The compaction for int32 selected-expert ids (``moe/group_scatter.py:317-369``)."""
    _check_num_experts(num_experts)
    if total_lanes <= 0:
        raise ValueError("total_lanes must be positive")
    validate_pointers(selected_experts_ptr=selected_experts_ptr, routing_weights_ptr=routing_weights_ptr,
                      expert_start_ptr=expert_start_ptr, sorted_lanes_ptr=sorted_lanes_ptr,
                      sorted_weights_ptr=sorted_weights_ptr)
    fn = entry("hipengine_qwen35_moe_group_compact_active_i32_parallel", [VOID] * 8 + [I64, I64, VOID], library)
    check_launch(fn(selected_experts_ptr, routing_weights_ptr, expert_start_ptr, active_experts_ptr, active_count_ptr,
                    sorted_lanes_ptr, sorted_experts_ptr, sorted_weights_ptr, total_lanes, num_experts, stream), runtime)


def qwen35_moe_group_prefix_active(counts_ptr: int, expert_start_ptr: int, active_experts_ptr: int,
                                   active_count_ptr: int, num_experts: int, *, stream: int = 0,
                                   library: ctypes.CDLL | None = None, runtime: HipRuntime | None = None) -> None:
    """int32 counts -> int64 compact starts ``[num_experts + 1]`` and the ascending list of the experts with rows
    (``moe/group_scatter.py:147-181``)."""
    _check_num_experts(num_experts)
    validate_pointers(counts_ptr=counts_ptr, expert_start_ptr=expert_start_ptr, active_experts_ptr=active_experts_ptr,
                      active_count_ptr=active_count_ptr)
    fn = entry("hipengine_qwen35_moe_group_prefix_active", [VOID] * 4 + [I64, VOID], library)
    check_launch(fn(counts_ptr, expert_start_ptr, active_experts_ptr, active_count_ptr, num_experts, stream), runtime)


def qwen35_moe_group_scatter(selected_experts_ptr: int, routing_weights_ptr: int, expert_start_ptr: int,
                             scatter_offsets_ptr: int, sorted_lanes_ptr: int, sorted_experts_ptr: int,
                             sorted_weights_ptr: int, total_lanes: int, num_experts: int, *,
                             include_routing_weights: bool = True, stream: int = 0,
                             library: ctypes.CDLL | None = None, runtime: HipRuntime | None = None) -> None:
    """Scatter of the lanes into per-expert compact order from given starts; the caller zeroes the offsets
    (``moe/group_scatter.py:505-555``).  hipEngine's scatter takes its slots with atomics in arrival order; here an
    expert's lanes are placed in ascending order, one of the orders that can produce."""
    _check_positive(total_lanes, "total_lanes")
    _check_num_experts(num_experts)
    validate_pointers(selected_experts_ptr=selected_experts_ptr, expert_start_ptr=expert_start_ptr,
                      scatter_offsets_ptr=scatter_offsets_ptr, sorted_lanes_ptr=sorted_lanes_ptr,
                      sorted_experts_ptr=sorted_experts_ptr)
    if include_routing_weights:
        validate_pointers(routing_weights_ptr=routing_weights_ptr, sorted_weights_ptr=sorted_weights_ptr)
    fn = entry("hipengine_qwen35_moe_group_scatter", [VOID] * 7 + [I64, I64, ctypes.c_bool, VOID], library)
    check_launch(fn(selected_experts_ptr, routing_weights_ptr or None, expert_start_ptr, scatter_offsets_ptr,
                    sorted_lanes_ptr, sorted_experts_ptr, sorted_weights_ptr or None, total_lanes, num_experts,
                    bool(include_routing_weights), stream), runtime)


def _tile_map(symbol: str, rows: int):
    def wrapper(expert_start_compact_ptr: int, tile_expert_start_ptr: int, tile_expert_ptr: int, total_ptr: int,
                num_experts: int, *, tile_capacity: int = 0, stream: int = 0, library: ctypes.CDLL | None = None,
                runtime: HipRuntime | None = None) -> None:
        _check_num_experts(num_experts)
        if tile_capacity < 0:
            raise ValueError("tile_capacity must be non-negative")
        validate_pointers(expert_start_compact_ptr=expert_start_compact_ptr, tile_expert_start_ptr=tile_expert_start_ptr,
                          tile_expert_ptr=tile_expert_ptr, total_ptr=total_ptr)
        fn = entry(symbol, [VOID] * 4 + [I64, I64, VOID], library)
        check_launch(fn(expert_start_compact_ptr, tile_expert_start_ptr, tile_expert_ptr, total_ptr, num_experts,
                        tile_capacity, stream), runtime)

    wrapper.__doc__ = f"Compact expert starts -> {rows}-row tile starts and the tile -> expert map (``{symbol}``)."
    return wrapper


qwen35_moe_wmma_tile_map = _tile_map("hipengine_qwen35_moe_wmma_tile_map", 16)      # moe/group_scatter.py:382-420
qwen35_moe_mmq64_tile_map = _tile_map("hipengine_qwen35_moe_mmq64_tile_map", 64)    # moe/group_scatter.py:464-502


def moe_lane_to_compact(sorted_lanes_ptr: int, lane_to_compact_ptr: int, compact_rows: int, total_lanes: int, *,
                        stream: int = 0, library: ctypes.CDLL | None = None,
                        runtime: HipRuntime | None = None) -> None:
    """Inverse of ``sorted_lanes`` (-1 for dropped lanes)."""
    if compact_rows <= 0 or total_lanes <= 0:
        raise ValueError("compact_rows and total_lanes must be positive")
    validate_pointers(sorted_lanes_ptr=sorted_lanes_ptr, lane_to_compact_ptr=lane_to_compact_ptr)
    fn = entry("hipengine_gfx950_moe_lane_to_compact", [VOID, VOID, I64, I64, VOID], library)
    check_launch(fn(sorted_lanes_ptr, lane_to_compact_ptr, compact_rows, total_lanes, stream), runtime)


def _check_positive(value: int, name: str) -> None:
    if value <= 0:
        raise ValueError(f"{name} must be positive")


def qwen35_moe_group_count(selected_experts_ptr: int, counts_ptr: int, total_lanes: int, num_experts: int, *,
                           stream: int = 0, library: ctypes.CDLL | None = None,
                           runtime: HipRuntime | None = None) -> None:
    """Count routed lanes per expert into int32 ``counts``; the caller zeroes it (hipEngine :77-103)."""
    _check_positive(total_lanes, "total_lanes")
    _check_positive(num_experts, "num_experts")
    validate_pointers(selected_experts_ptr=selected_experts_ptr, counts_ptr=counts_ptr)
    fn = entry("hipengine_qwen35_moe_group_count", [VOID, VOID, I64, I64, VOID], library)
    check_launch(fn(selected_experts_ptr, counts_ptr, total_lanes, num_experts, stream), runtime)


def qwen35_moe_group_prefix(counts_ptr: int, padded_counts_ptr: int, expert_start_ptr: int, total_padded_ptr: int,
                            num_experts: int, pad_multiple: int, *, stream: int = 0,
                            library: ctypes.CDLL | None = None, runtime: HipRuntime | None = None) -> None:
    """Per-expert counts -> counts padded to ``pad_multiple``, their exclusive prefix and total (hipEngine :106-146)."""
    _check_num_experts(num_experts)
    _check_positive(pad_multiple, "pad_multiple")
    validate_pointers(counts_ptr=counts_ptr, padded_counts_ptr=padded_counts_ptr, expert_start_ptr=expert_start_ptr,
                      total_padded_ptr=total_padded_ptr)
    fn = entry("hipengine_qwen35_moe_group_prefix", [VOID] * 4 + [I64, I64, VOID], library)
    check_launch(fn(counts_ptr, padded_counts_ptr, expert_start_ptr, total_padded_ptr, num_experts, pad_multiple, stream),
                 runtime)


def qwen35_moe_group_scatter_gather_lowp(hidden_states_ptr: int, selected_experts_ptr: int, routing_weights_ptr: int,
                                         expert_start_ptr: int, scatter_offsets_ptr: int, sorted_lanes_ptr: int,
                                         sorted_experts_ptr: int, sorted_weights_ptr: int, packed_hidden_ptr: int,
                                         total_lanes: int, num_experts: int, top_k: int, hidden_size: int, *,
                                         stream: int = 0, library: ctypes.CDLL | None = None,
                                         runtime: HipRuntime | None = None) -> None:
    """Scatter lanes into expert order and gather their 16-bit hidden rows (hipEngine :558-619).  Lanes of an
    expert land in ascending lane order (hipEngine: arrival order); ``scatter_offsets`` (int32, zeroed by the
    caller) ends as the per-expert lane counts."""
    _check_positive(total_lanes, "total_lanes")
    _check_num_experts(num_experts)
    _check_positive(top_k, "top_k")
    _check_positive(hidden_size, "hidden_size")
    validate_pointers(hidden_states_ptr=hidden_states_ptr, selected_experts_ptr=selected_experts_ptr,
                      routing_weights_ptr=routing_weights_ptr, expert_start_ptr=expert_start_ptr,
                      scatter_offsets_ptr=scatter_offsets_ptr, sorted_lanes_ptr=sorted_lanes_ptr,
                      sorted_experts_ptr=sorted_experts_ptr, sorted_weights_ptr=sorted_weights_ptr,
                      packed_hidden_ptr=packed_hidden_ptr)
    fn = entry("hipengine_qwen35_moe_group_scatter_gather_lowp", [VOID] * 9 + [I64] * 4 + [VOID], library)
    check_launch(fn(hidden_states_ptr, selected_experts_ptr, routing_weights_ptr, expert_start_ptr, scatter_offsets_ptr,
                    sorted_lanes_ptr, sorted_experts_ptr, sorted_weights_ptr, packed_hidden_ptr, total_lanes,
                    num_experts, top_k, hidden_size, stream), runtime)


def qwen35_moe_gather_packed_hidden_lowp(hidden_states_ptr: int, sorted_lanes_ptr: int, packed_hidden_ptr: int,
                                         total_elements: int, tokens: int, top_k: int, hidden_size: int, *,
                                         stream: int = 0, library: ctypes.CDLL | None = None,
                                         runtime: HipRuntime | None = None) -> None:
    """Gather 16-bit hidden rows by sorted lane ids into packed rows (hipEngine :622-668)."""
    _check_positive(total_elements, "total_elements")
    _check_positive(tokens, "tokens")
    _check_positive(top_k, "top_k")
    _check_positive(hidden_size, "hidden_size")
    if total_elements % hidden_size != 0:
        raise ValueError("total_elements must be a multiple of hidden_size")
    validate_pointers(hidden_states_ptr=hidden_states_ptr, sorted_lanes_ptr=sorted_lanes_ptr,
                      packed_hidden_ptr=packed_hidden_ptr)
    fn = entry("hipengine_qwen35_moe_gather_packed_hidden_lowp", [VOID] * 3 + [I64] * 4 + [VOID], library)
    check_launch(fn(hidden_states_ptr, sorted_lanes_ptr, packed_hidden_ptr, total_elements, tokens, top_k, hidden_size,
                    stream), runtime)


def register_kernels(backend: str = "hip_gfx950", *, replace: bool = False) -> None:
    # keys of hipEngine's moe/group_scatter.py:713-806
    for quant, variant in (("generic", "selected_experts"), ("w4_paro", "qwen35")):
        register(KernelKey(backend, "moe_group_count", quant, variant), qwen35_moe_group_count, replace=replace)
    register(KernelKey(backend, "moe_group_prefix", "w4_paro", "qwen35"), qwen35_moe_group_prefix, replace=replace)
    register(KernelKey(backend, "moe_group_prefix", "generic", "pad_multiple"), qwen35_moe_group_prefix, replace=replace)
    for quant, variant in (("generic", "bf16_lane_rows"), ("w4_paro", "qwen35_lowp")):
        register(KernelKey(backend, "moe_group_scatter_gather", quant, variant), qwen35_moe_group_scatter_gather_lowp,
                 replace=replace)
    for quant, variant in (("generic", "bf16_lanes"), ("w4_paro", "qwen35_lowp")):
        register(KernelKey(backend, "moe_gather_packed_hidden", quant, variant), qwen35_moe_gather_packed_hidden_lowp,
                 replace=replace)
    register(KernelKey(backend, "moe_group_compact", "generic", "active_experts"), qwen35_moe_group_compact_active,
             replace=replace)
    register(KernelKey(backend, "moe_group_compact", "generic", "active_experts_source_rows"),
             qwen35_moe_group_compact_active_source_rows, replace=replace)
    register(KernelKey(backend, "moe_mmq_tile_map", "generic", "tile32"), qwen35_moe_mmq32_tile_map, replace=replace)
    register(KernelKey(backend, "moe_mmq_tile_map", "generic", "tile64"), qwen35_moe_mmq64_tile_map, replace=replace)
    for quant, variant in (("generic", "tile16"), ("w4_paro", "qwen35")):
        register(KernelKey(backend, "moe_wmma_tile_map", quant, variant), qwen35_moe_wmma_tile_map, replace=replace)
    register(KernelKey(backend, "moe_group_prefix", "generic", "active_experts"), qwen35_moe_group_prefix_active,
             replace=replace)
    register(KernelKey(backend, "moe_group_compact", "generic", "active_experts_parallel"),
             qwen35_moe_group_compact_active_parallel, replace=replace)
    register(KernelKey(backend, "moe_group_compact", "generic", "active_experts_i32_parallel"),
             qwen35_moe_group_compact_active_i32_parallel, replace=replace)
    register(KernelKey(backend, "moe_group_compact", "generic", "active_experts_source_rows_parallel"),
             qwen35_moe_group_compact_active_source_rows_parallel, replace=replace)
    register(KernelKey(backend, "moe_group_scatter", "w4_paro", "qwen35"), qwen35_moe_group_scatter, replace=replace)
    register(KernelKey(backend, "moe_lane_to_compact", "generic", "sorted_lanes"), moe_lane_to_compact, replace=replace)
