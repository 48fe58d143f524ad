"""Host logic of the drop-in boundary: kernel registry semantics, quant plugin
records, GGUF layout helpers and wrapper validation.  CPU only, no kernels run.

The expectations restate hipEngine's own unit tests for these surfaces
(tests/test_unit_kernel_registry.py:25-154, tests/test_unit_model_quant_and_imports.py:65-95,
tests/test_unit_gguf_quant_layout.py:22-39, tests/test_gpu_gguf_q4_k_gemv.py:206-223).
"""

from __future__ import annotations

import subprocess
import sys
from pathlib import Path

import pytest

from hipengine_amd import quant
from hipengine_amd.kernels import registry as R
from hipengine_amd.kernels.registry import KernelKey
from hipengine_amd.quant import GGMLQuantizationType as T

ROOT = Path(__file__).resolve().parents[1]


@pytest.fixture()
def clean_registry():
    saved = R.snapshot_registry_for_tests()
    R.clear_registry_for_tests()
    yield
    R.restore_registry_for_tests(saved)


def test_kernel_key_validation_and_display():
    with pytest.raises(ValueError):
        KernelKey("", "linear", "fp16")
    with pytest.raises(ValueError):
        KernelKey("hip_gfx950", "linear", "")
    assert "variant='v'" in KernelKey("b", "l", "q", "v").display()
    assert KernelKey("a", "l", "q") < KernelKey("b", "l", "q")


def test_registry_exact_duplicate_and_fallback_order(clean_registry):
    def exact(): return "exact"
    def novar(): return "novar"
    def fp16(): return "fp16"
    def cpu(): return "cpu"

    R.register(KernelKey("cpu_reference", "linear", "fp16"), cpu)
    assert R.resolve(backend="hip_gfx950", layer="linear", quant="gguf_q4_k", variant="v")() == "cpu"
    R.register(KernelKey("hip_gfx950", "linear", "fp16"), fp16)
    assert R.resolve(backend="hip_gfx950", layer="linear", quant="gguf_q4_k", variant="v")() == "fp16"
    R.register(KernelKey("hip_gfx950", "linear", "gguf_q4_k"), novar)
    assert R.resolve(backend="hip_gfx950", layer="linear", quant="gguf_q4_k", variant="v")() == "novar"
    R.register(KernelKey("hip_gfx950", "linear", "gguf_q4_k", "v"), exact)
    assert R.resolve(backend="hip_gfx950", layer="linear", quant="gguf_q4_k", variant="v")() == "exact"
    with pytest.raises(R.DuplicateKernelError):
        R.register(KernelKey("hip_gfx950", "linear", "gguf_q4_k", "v"), exact)
    R.register(KernelKey("hip_gfx950", "linear", "gguf_q4_k", "v"), novar, replace=True)
    assert R.resolve(backend="hip_gfx950", layer="linear", quant="gguf_q4_k", variant="v")() == "novar"
    assert R.is_registered(KernelKey("hip_gfx950", "linear", "gguf_q4_k", "v"))
    assert not R.is_registered(KernelKey("hip_gfx950", "linear", "gguf_q4_k", "other"))   # exact only
    assert R.can_resolve(backend="hip_gfx950", layer="linear", quant="gguf_q4_k", variant="other")


def test_registry_missing_error_generation_and_cache_invalidation(clean_registry):
    g0 = R.generation()
    with pytest.raises(R.MissingKernelError) as info:
        R.resolve(backend="hip_gfx950", layer="linear", quant="gguf_q4_k", variant="v")
    assert info.value.requested == KernelKey("hip_gfx950", "linear", "gguf_q4_k", "v")
    assert [k.backend for k in info.value.attempted] == ["hip_gfx950"] * 4 + ["cpu_reference"] * 4
    assert R.resolve(backend="x", layer="l", quant="q", missing="none") is None
    def a(): return "a"
    def b(): return "b"
    R.register(KernelKey("hip_gfx950", "linear", "fp16"), a)
    assert R.generation() > g0
    assert R.resolve(backend="hip_gfx950", layer="linear", quant="gguf_q4_k")() == "a"      # memoized fallback
    R.register(KernelKey("hip_gfx950", "linear", "gguf_q4_k"), b)
    assert R.resolve(backend="hip_gfx950", layer="linear", quant="gguf_q4_k")() == "b"      # memo dropped
    R.unregister(KernelKey("hip_gfx950", "linear", "gguf_q4_k"))
    assert R.resolve(backend="hip_gfx950", layer="linear", quant="gguf_q4_k")() == "a"
    snap = R.snapshot_registry_for_tests()
    R.clear_registry_for_tests()
    assert R.registered_keys() == ()
    R.restore_registry_for_tests(snap)
    assert R.registered_keys() == tuple(sorted(snap))


def test_backend_registers_the_documented_keys(clean_registry):
    from hipengine_amd.kernels import hip_gfx950

    hip_gfx950.register_backend_kernels(replace=True)
    keys = set(R.registered_keys())
    for q in ("gguf_q4_k", "gguf_q6_k", "gguf_q8_0"):
        for v in ("q8_1_fused_gemv_f32_f32_out", "q8_1_fused_gemv_bf16_bf16_out", "q8_1_fused_prefill_bf16_f32_out"):
            assert KernelKey("hip_gfx950", "linear", q, v) in keys
    assert KernelKey("hip_gfx950", "linear", "gguf_q4_k", "q8_1_dp4a_vdr_bf16_f32_out") in keys
    assert KernelKey("hip_gfx950", "activation_quant", "q8_1_ds4", "bf16") in keys
    for key in (KernelKey("hip_gfx950", "linear", "gguf_q4_k", "mmq32_vdr_dense_bf16_f32_out"),
                KernelKey("hip_gfx950", "linear", "gguf_q6_k", "mmq32_q8_1_d4s4_f32_bf16_f32_out"),
                KernelKey("hip_gfx950", "linear", "gguf_q4_k", "selected_gemv_bf16_bf16_out"),
                KernelKey("hip_gfx950", "moe_linear", "gguf_q4_k",
                          "selected_dual_q8_1_ds4_mmq32_prefill_compact32_bf16_bf16_out"),
                KernelKey("hip_gfx950", "moe_group_compact", "generic", "active_experts_source_rows"),
                KernelKey("hip_gfx950", "moe_mmq_tile_map", "generic", "tile32"),
                KernelKey("hip_gfx950", "router_select", "fp32"),
                KernelKey("hip_gfx950", "argmax", "f32", "rows_i32"),
                KernelKey("hip_gfx950", "embedding", "gguf_q5_k", "lookup_bf16_out"),
                KernelKey("hip_gfx950", "embedding", "gguf_q6_k", "lookup_bf16_out"),
                KernelKey("hip_gfx950", "linear", "gguf_q4_k", "dual_silu_gemv_bf16_bf16_out"),
                KernelKey("hip_gfx950", "linear", "gguf_q6_k", "gemv_bf16_residual_bf16_out")):
        assert key in keys
    assert not any(k.backend == "cpu_reference" for k in keys)            # the package ships no CPU path
    assert hip_gfx950.GGUF_CONSUMER_LAYERS >= {"linear", "moe_linear"}
    fn = R.resolve(backend="hip_gfx950", layer="linear", quant="gguf_q4_k", variant="q8_1_fused_gemv_f32_f32_out")
    assert fn.__name__ == "gguf_q4_k_q8_1_fused_gemv_f32_f32_out"


def test_every_raw_row_of_the_dispatch_surface_resolves_to_this_backend(clean_registry):
    """hipEngine's dispatcher resolves, for a raw-layout weight, ("linear", weight quant, "gemv_<act>_<out>_out") and
    rewrites gemv_ to prefill_ for rows > 1 (loading/qwen35_gguf_consumer_surface.py:134-144,527-530); with
    missing="error" nothing may fall through to another backend.  The MoE consumers and call kinds of
    loading/gguf_selected_contract.py:31-54 resolve too."""
    from hipengine_amd.kernels import hip_gfx950

    hip_gfx950.register_backend_kernels(replace=True)
    raw_rows = (("bf16", "bf16"), ("bf16", "fp16"), ("bf16", "f32"), ("f32", "f32"))
    for q in ("gguf_q4_k", "gguf_q5_k", "gguf_q6_k", "gguf_q8_0"):
        for act, out in raw_rows:
            for family in ("gemv", "prefill"):
                variant = f"{family}_{act}_{out}_out"
                assert R.is_registered(KernelKey("hip_gfx950", "linear", q, variant))
                fn = R.resolve(backend="hip_gfx950", layer="linear", quant=q, variant=variant, missing="error")
                assert fn.__name__ == f"{q}_{variant}"
        assert R.resolve(backend="hip_gfx950", layer="linear", quant=q, variant="dual_gemv_bf16_bf16_out",
                         missing="error").__name__ == f"{q}_dual_gemv_bf16_bf16_out"
    for layer, q, variant in (
            ("linear", "gguf_q4_k", "selected_gemv_bf16_bf16_out"),
            ("linear", "gguf_q4_k", "selected_dual_gemv_bf16_bf16_out"),
            ("linear", "gguf_q4_k", "selected_dual_silu_gemv_bf16_bf16_out"),
            ("linear", "gguf_q4_k", "selected_dual_gemv_q8_1_dp4a_bf16_bf16_out"),
            ("moe_linear", "gguf_q4_k", "selected_gemv_decode_bf16_bf16_out"),
            ("moe_linear", "gguf_q4_k", "selected_dual_silu_gemv_decode_bf16_bf16_out"),
            ("moe_linear", "gguf_q4_k", "selected_weighted_down_gemv_decode_bf16_bf16_out"),
            ("moe_linear", "gguf_q6_k", "selected_weighted_down_gemv_decode_bf16_bf16_out"),
            ("moe_linear", "gguf_q4_k", "selected_grouped_prefill_compact_rowbatch8_bf16_bf16_out"),
            ("moe_group_count", "generic", "selected_experts"), ("moe_group_prefix", "w4_paro", "qwen35"),
            ("moe_group_scatter_gather", "generic", "bf16_lane_rows"), ("moe_gather_packed_hidden", "generic", "bf16_lanes")):
        assert R.is_registered(KernelKey("hip_gfx950", layer, q, variant)), (layer, q, variant)
    # a prefill wrapper checks its arguments like hipEngine's before it touches the library
    fn = R.resolve(backend="hip_gfx950", layer="linear", quant="gguf_q4_k", variant="prefill_bf16_bf16_out")
    with pytest.raises(ValueError, match="divisible"):
        fn(16, 16, 16, 40, 100, 64)
    with pytest.raises(ValueError, match="threads"):
        fn(16, 16, 16, 40, 256, 64, threads=7)


def test_quant_plugin_records():
    p = quant.resolve_quant("gguf_q4_k")
    assert (p.weight_storage, p.activation_preprocess, p.compute_dtype, p.scale_granularity, p.calibration_artifact,
            p.kernel_family) == ("gguf_block_q4_k", "none", "fp32_accum", "block256_subblock32_scale_min", "gguf",
                                 "gguf_q4_k_gemv")
    p6, p8 = quant.resolve_quant("gguf_q6_k"), quant.resolve_quant("gguf_q8_0")
    assert (p6.weight_storage, p6.scale_granularity, p6.kernel_family) == ("gguf_block_q6_k", "block256_subblock16_scale", "gguf_k_gemv")
    assert (p8.weight_storage, p8.scale_granularity, p8.kernel_family) == ("gguf_block_q8_0", "block32_scale", "gguf_k_gemv")
    assert isinstance(p, quant.QuantPlugin)
    with pytest.raises(quant.DuplicateQuantError):
        quant.register_quant(quant.GGUFQ4KQuant())
    with pytest.raises(quant.MissingQuantError, match="gguf_q4_k"):
        quant.resolve_quant("nope")
    with pytest.raises(ValueError):
        quant.register_quant(quant.GGUFQ4KQuant(name=""))
    assert [q.name for q in quant.registered_quants()] == sorted(q.name for q in quant.registered_quants())


def test_gguf_layout_table_and_byte_shapes():
    assert (quant.quant_layout(T.Q8_0).block_size, quant.quant_layout(T.Q8_0).type_size) == (32, 34)
    assert (quant.quant_layout(T.Q4_K).block_size, quant.quant_layout(T.Q4_K).type_size) == (256, 144)
    assert quant.quant_layout(T.Q5_K).type_size == 176
    assert quant.quant_layout(T.Q6_K).type_size == 210
    assert quant.quant_layout(T.BF16).type_size == 2
    assert quant.quant_layout(12).name == "Q4_K" and quant.quant_layout(T.Q4_K).is_block_quantized
    assert quant.nbytes_for_shape((3, 64), T.Q8_0) == 3 * 2 * 34
    assert quant.nbytes_for_shape((17408, 5120), T.Q4_K) == 50_135_040
    assert quant.nbytes_for_shape((5120, 17408), T.Q6_K) == 73_113_600
    assert quant.quant_shape_to_byte_shape((3, 64), T.Q8_0) == (3, 68)
    assert quant.quant_shape_from_byte_shape((3, 68), T.Q8_0) == (3, 64)
    assert quant.quant_shape_to_byte_shape((2, 5), T.F32) == (2, 5)
    with pytest.raises(ValueError, match="row size 63"):
        quant.quant_shape_to_byte_shape((3, 63), T.Q8_0)
    with pytest.raises(ValueError):
        quant.nbytes_for_shape((3, 63), T.Q8_0)
    with pytest.raises(ValueError):
        quant.quant_shape_from_byte_shape((3, 67), T.Q8_0)
    with pytest.raises(KeyError):
        quant.quant_layout(999)
    assert quant.GGUF_Q8_1_MMQ_DS4_BYTES == 144 and quant.GGUF_Q4_K_BLOCK_BYTES == 144 and quant.QK_K == 256


def test_wrappers_validate_before_touching_the_library():
    from hipengine_amd.kernels.hip_gfx950.quant import gguf_q8_1_gemv as G
    from hipengine_amd.kernels.hip_gfx950.quant import gguf_quantize as Q

    fn = G.FUSED[("q4_k", "bf16", "bf16")]
    with pytest.raises(ValueError, match="divisible"):
        fn(1, 1, 1, 1, 100, 8)
    with pytest.raises(ValueError, match="threads"):
        fn(1, 1, 1, 1, 256, 8, threads=96)
    with pytest.raises(ValueError, match="rows"):
        fn(1, 1, 1, 0, 256, 8)
    with pytest.raises(ValueError, match="pointer"):
        fn(0, 1, 1, 1, 256, 8)
    with pytest.raises(ValueError, match="divisible"):
        Q.gguf_q8_1_mmq_ds4_pack_bf16(1, 1, 1, 192)
    assert Q.q8_1_workspace_nbytes(2, 5120) == 2 * 160 * 36
    assert Q.ds4_workspace_nbytes(2048, 5120) == 2048 * 40 * 144


class _RecordingFunction:
    """Stands in for a configured C function: records its arguments, returns a chosen hipError_t."""

    def __init__(self, code=0):
        self.code, self.calls, self.argtypes, self.restype = code, [], None, None

    def __call__(self, *args):
        self.calls.append(args)
        return self.code


class _RecordingLibrary:
    def __init__(self, code=0):
        self._code, self.functions = code, {}

    def __getattr__(self, name):
        if name.startswith("hipengine_"):
            return self.functions.setdefault(name, _RecordingFunction(self._code))
        raise AttributeError(name)


def test_validation_flag_and_lean_launcher_reach_the_c_function_with_the_c_signature():
    """The launch path of a decode loop: with validation on the wrapper refuses bad shapes before the library is
    touched; with it off the same call goes straight to the C function (whose own checks remain); the lean
    launcher is that C function with its argument types set once."""
    from hipengine_amd.kernels.hip_gfx950 import _launch
    from hipengine_amd.kernels.hip_gfx950.quant import gguf_q8_1_gemv as G

    lib = _RecordingLibrary()
    fn = G.FUSED[("q4_k", "f32", "f32")]
    symbol = "hipengine_gguf_q4_k_q8_1_fused_gemv_f32_f32_out"
    fn(16, 32, 48, 1, 5120, 17408, library=lib)
    assert lib.functions[symbol].calls == [(16, 32, 48, 1, 5120, 17408, 128, 0)]
    assert len(lib.functions[symbol].argtypes) == 8
    with pytest.raises(ValueError):
        fn(16, 32, 48, 1, 100, 8, library=lib)
    assert len(lib.functions[symbol].calls) == 1                     # refused before the library was touched
    assert _launch.VALIDATE is True
    try:
        _launch.set_validation(False)
        fn(16, 32, 48, 1, 100, 8, library=lib)                       # not checked here: the C entry point's job
        assert lib.functions[symbol].calls[-1] == (16, 32, 48, 1, 100, 8, 128, 0)
    finally:
        _launch.set_validation(True)
    assert _launch.VALIDATE is True
    lean = G.lean_fused("q4_k", "f32", "f32", library=lib)
    assert lean is lib.functions[symbol]                             # the configured function itself
    assert lean(16, 32, 48, 1, 5120, 17408, 128, 0) == 0
    # a non-zero hipError_t from the C function surfaces as an error of the wrapper
    bad = _RecordingLibrary(code=1)
    with pytest.raises(Exception) as err:
        fn(16, 32, 48, 1, 5120, 17408, library=bad)
    assert "1" in str(err.value) or "invalid" in str(err.value).lower()


def test_host_package_is_torch_free():
    """Importing the package, the wrappers and bench.py's harness must not import torch."""
    code = ("import sys; sys.path.insert(0, %r); import hipengine_amd, hipengine_amd.quant, "
            "hipengine_amd.kernels.hip_gfx950 as b; b.register_backend_kernels(); "
            "import hipengine_amd.core.hip, hipengine_amd.core.memory, hipengine_amd.core.build, hipengine_amd.synthetic; "
            "assert 'torch' not in sys.modules, 'torch was imported'; "
            "import hipengine_amd.core.hip as h; assert not h.is_default_runtime_loaded()") % str(ROOT)
    subprocess.run([sys.executable, "-c", code], check=True)


def test_product_package_never_imports_the_oracle():
    for path in (ROOT / "hipengine_amd").rglob("*.py"):
        text = path.read_text()
        assert "import oracle" not in text and "from oracle" not in text, path


def test_build_plan_is_stable_and_names_the_artifact():
    from hipengine_amd.core import build

    a = build.plan_hip_build(compiler_version="test")
    b = build.plan_hip_build(compiler_version="test")
    assert a.key == b.key and len(a.key) == 64
    assert a.output.name == "libhipengine_gfx950.so"
    assert {s.name for s in a.sources} >= {"gguf_gemv.hip", "gguf_quantize.hip", "gguf_verify.hip"}
    assert "--offload-arch=gfx950" in a.flags and "-mcumode" not in a.flags
    assert build.plan_hip_build(compiler_version="other").key != a.key
    assert a.commands[-1][-1].endswith("libhipengine_gfx950.so")


def test_moe_wrappers_validate_before_touching_the_device():
    """Argument errors are raised on the host, before any library call (hipEngine's wrappers do the same)."""
    from hipengine_amd.kernels.hip_gfx950.moe import group_scatter as GS
    from hipengine_amd.kernels.hip_gfx950.quant import gguf_moe as M

    with pytest.raises(ValueError, match="num_experts"):
        GS.qwen35_moe_mmq32_tile_map(1, 1, 1, 1, 0)
    with pytest.raises(ValueError, match="num_experts"):
        GS.qwen35_moe_group_compact_active_source_rows(1, 1, 1, 1, 1, 1, 1, 1, 8, 4096, 8)
    with pytest.raises(ValueError, match="tile_capacity"):
        GS.qwen35_moe_mmq32_tile_map(1, 1, 1, 1, 8, tile_capacity=-1)
    from hipengine_amd.kernels.hip_gfx950.moe import router as RT
    with pytest.raises(ValueError, match="top_k must be <= 16"):
        RT.qwen35_router_select(1, 1, 1, 4, 256, 256, 17)
    with pytest.raises(ValueError, match="top_k must be <= num_experts"):
        RT.qwen35_router_select(1, 1, 1, 4, 256, 4, 8)
    with pytest.raises(ValueError, match="num_experts must be <= logits_stride"):
        RT.qwen35_router_select(1, 1, 1, 4, 128, 256, 8)
    with pytest.raises(ValueError, match="threads"):
        RT.qwen35_router_select(1, 1, 1, 4, 256, 256, 8, threads=100)
    with pytest.raises(ValueError, match="multiple of x_rows"):
        M.gguf_q4_k_selected_gemv_bf16_bf16_out(1, 1, 1, 1, 3, 8, 4, 256, 32)
    with pytest.raises(ValueError, match="divisible"):
        M.gguf_q4_k_selected_gemv_bf16_bf16_out(1, 1, 1, 1, 1, 8, 4, 200, 32)
    with pytest.raises(ValueError, match="non-null"):
        M.gguf_q4_k_selected_gemv_bf16_bf16_out(0, 1, 1, 1, 1, 8, 4, 256, 32)
    with pytest.raises(ValueError, match="x_rows \\* top_k"):
        M.gguf_selected_gemv("gguf_q4_k", M.SEL_DOWN_SUM, 1, 1, 1, 1, 2, 9, 4, 256, 32, routing_weights_ptr=1, top_k=4)
    with pytest.raises(ValueError, match="up to in_features 4096"):
        M.gguf_selected_gemv("gguf_q8_0", M.SEL_DUAL_SILU, 1, 1, 1, 1, 1, 8, 4, 4352, 32, qweight_b_ptr=1)
    with pytest.raises(ValueError, match="quant must be"):
        M.gguf_selected_gemv("gguf_q3_k", M.SEL_SINGLE, 1, 1, 1, 1, 1, 8, 4, 256, 32)
    single, silu = M.SELECTED_K["q6_k"]
    with pytest.raises(ValueError, match="multiple of x_rows"):
        single(1, 1, 1, 1, 3, 8, 4, 256, 32)
    with pytest.raises(ValueError, match="non-null"):
        silu(1, 0, 1, 1, 1, 8, 8, 4, 256, 32)
    from hipengine_amd.kernels.hip_gfx950.quant import gguf_q8_1_gemv as G
    with pytest.raises(TypeError, match="2 weight and 2 output pointers"):
        G.gguf_q8_0_dp4a_dual_split_rowtile4_gemv_f32_f32_out(1, 1, 1, 1, 1, 4, 256, 8)
    with pytest.raises(ValueError, match="divisible"):
        G.gguf_q8_0_dp4a_triple_split_rowtile4_gemv_bf16_bf16_out(1, 1, 1, 1, 1, 1, 1, 4, 100, 8, 8, 8)
    with pytest.raises(ValueError, match="hidden must be divisible"):
        from hipengine_amd.kernels.hip_gfx950.quant import gguf_quantize as Q
        Q.gguf_q8_1_mmq_gather_ds4_pack_bf16(1, 1, 1, 8, 192, 1, 8)
    with pytest.raises(ValueError, match="num_experts"):
        GS.moe_group_compact_index(1, 1, 1, 1, 1, 1, 1, 1, 1, 8, 4096, 8)
    with pytest.raises(ValueError, match="multiples of 32"):
        M.gguf_q4_k_grouped_mmq(1, 1, 1, 1, 1, 1, 8, 8, 256, 40, 4, 32)
    with pytest.raises(ValueError, match="multiple of 32"):
        M.gguf_q4_k_grouped_mmq(1, 1, 1, 1, 1, 1, 8, 8, 256, 64, 4, 40)
    with pytest.raises(ValueError, match="multiples of 32"):
        M.gguf_q5_k_grouped_mmq(1, 1, 1, 1, 1, 1, 8, 8, 256, 40, 4, 32)
    with pytest.raises(ValueError, match="multiple of 128"):
        M.gguf_q6_k_grouped_mmq(1, 1, 1, 1, 1, 1, 8, 8, 256, 64, 4, 64)
    with pytest.raises(ValueError, match="divisible by the GGUF block size"):
        M.gguf_q6_k_grouped_mmq(1, 1, 1, 1, 1, 1, 8, 8, 384, 64, 4, 128)
    with pytest.raises(ValueError, match="non-null"):
        M.gguf_q6_k_grouped_mmq(1, 1, 1, 0, 1, 1, 8, 8, 256, 64, 4, 128)
    with pytest.raises(ValueError, match="tile_rows"):
        GS.moe_tile_map(1, 1, 1, 1, 8, tile_rows=48)
    with pytest.raises(ValueError, match="total_lanes must be positive"):
        GS.qwen35_moe_group_scatter(1, 1, 1, 1, 1, 1, 1, 0, 8)
    with pytest.raises(ValueError, match="non-null"):
        GS.qwen35_moe_group_scatter(1, 0, 1, 1, 1, 1, 1, 16, 8)          # weights asked for, no pointer
    with pytest.raises(ValueError, match="num_experts"):
        GS.qwen35_moe_group_prefix_active(1, 1, 1, 1, 0)
    with pytest.raises(ValueError, match="tile_capacity"):
        GS.qwen35_moe_wmma_tile_map(1, 1, 1, 1, 8, tile_capacity=-2)
    from hipengine_amd.kernels.hip_gfx950.fused import paro_combine as PC
    with pytest.raises(ValueError, match="features must be positive"):
        PC.shared_gate_combine_residual_rmsnorm_gguf_bf16_out(1, 1, 1, 1, 1, 1, 1, 4, 0, 1)
    with pytest.raises(ValueError, match="rows_per_token must be positive"):
        PC.weighted_sum_shared_gate_combine_residual_rmsnorm_gguf_bf16_out(1, 1, 1, 1, 1, 1, 1, 1, 4, 0, 64, 1)
    with pytest.raises(ValueError, match="non-null"):
        PC.moe_gather_tail_rmsnorm_bf16(1, 0, 1, 1, 1, 1, 1, 1, 1, 4, 8, 64, 32, 1)
    with pytest.raises(ValueError, match="inter"):
        M.moe_silu_mul_d4s4_pack(1, 1, 4, 100)


def test_gguf_container_round_trip_and_errors(tmp_path):
    """GGUF intake: a container written with the synthetic writer comes back with the same metadata, logical and
    byte shapes and payload bytes (raw block rows as the kernels take them); malformed files raise as hipEngine's
    scanner does (hipengine/loading/gguf.py:185-268)."""
    import struct

    import numpy as np

    from hipengine_amd.loading import gguf as GG
    from hipengine_amd.quant.gguf import GGMLQuantizationType as T

    rng = np.random.default_rng(0)
    q4 = rng.integers(0, 256, size=(6, 512 // 256 * 144), dtype=np.uint8)
    q6 = rng.integers(0, 256, size=(2, 3, 256 // 256 * 210), dtype=np.uint8)      # [experts, rows, bytes]
    f32 = rng.standard_normal((5,)).astype(np.float32)
    bf16 = rng.integers(0, 65536, size=(4, 8), dtype=np.uint16)
    meta = {"general.architecture": "qwen35", "general.file_type": 15, "qwen35.block_count": 2,
            "tokenizer.ggml.tokens": ["a", "bc", ""], "qwen35.rope.freq_base": 1000000.0, "flag": True,
            "qwen35.dims": [1, 2, 3], "big": 2**40, "neg": -7}
    path = GG.write_gguf(tmp_path / "m.gguf", meta, [
        ("blk.0.ffn_gate.weight", T.Q4_K, (6, 512), q4), ("blk.0.ffn_down_exps.weight", T.Q6_K, (2, 3, 256), q6),
        ("output_norm.weight", T.F32, (5,), f32), ("token_embd.weight", T.BF16, (4, 8), bf16)], alignment=64)
    reader = GG.GGUFReader(path)
    info = reader.info
    assert info.version == 3 and info.alignment == 64 and info.tensor_count == 4
    assert info.architecture == "qwen35" and info.file_type == 15
    assert info.metadata["tokenizer.ggml.tokens"] == ["a", "bc", ""] and info.metadata["flag"] is True
    assert info.metadata["qwen35.dims"] == [1, 2, 3] and info.metadata["big"] == 2**40 and info.metadata["neg"] == -7
    assert info.tensor_data_offset % 64 == 0
    t = reader.tensor_info("blk.0.ffn_gate.weight")
    assert t.shape == (6, 512) and t.ggml_shape == (512, 6) and t.byte_shape == (6, 288) and t.nbytes == 6 * 288
    assert t.ggml_type == 12 and t.ggml_type_name == "Q4_K" and t.n_elements == 6 * 512 and t.data_offset % 64 == 0
    assert np.array_equal(reader.tensor_data("blk.0.ffn_gate.weight"), q4)
    e = reader.tensor_info("blk.0.ffn_down_exps.weight")
    assert e.shape == (2, 3, 256) and e.byte_shape == (2, 3, 210)
    assert np.array_equal(reader.tensor_data("blk.0.ffn_down_exps.weight"), q6)
    assert np.array_equal(reader.tensor_data("output_norm.weight"), f32)
    assert reader.tensor_data("token_embd.weight").dtype == np.uint16
    assert np.array_equal(reader.tensor_data("token_embd.weight"), bf16)
    assert info.total_tensor_nbytes == q4.nbytes + q6.nbytes + f32.nbytes + bf16.nbytes
    assert info.names_with_prefix("blk.0.") == ("blk.0.ffn_gate.weight", "blk.0.ffn_down_exps.weight")
    assert [x.name for x in info.require(["output_norm.weight", "token_embd.weight"])] == ["output_norm.weight", "token_embd.weight"]
    with pytest.raises(GG.MissingGGUFTensorError, match="missing required GGUF tensors: nope"):
        info.require(["output_norm.weight", "nope"])
    with pytest.raises(GG.MissingGGUFTensorError):
        reader.tensor_info("absent")

    raw = path.read_bytes()
    bad = tmp_path / "bad.gguf"
    bad.write_bytes(b"GGUX" + raw[4:])
    with pytest.raises(GG.GGUFFormatError, match="magic"):
        GG.scan_gguf(bad)
    bad.write_bytes(raw[:4] + struct.pack("<I", 9) + raw[8:])
    with pytest.raises(GG.GGUFFormatError, match="unsupported GGUF version 9"):
        GG.scan_gguf(bad)
    bad.write_bytes(raw[: info.tensor_data_offset + 100])          # payload cut short
    with pytest.raises(GG.GGUFFormatError, match="falls outside file size"):
        GG.scan_gguf(bad)
    bad.write_bytes(raw[:40])                                        # header cut short
    with pytest.raises(EOFError):
        GG.scan_gguf(bad)
    with pytest.raises(ValueError, match="stored bytes"):
        GG.write_gguf(tmp_path / "x.gguf", {}, [("w", T.Q4_K, (6, 512), q4[:5])])
    v2 = GG.write_gguf(tmp_path / "v2.gguf", {"general.architecture": "x"}, [("w", T.Q8_0, (3, 64), np.zeros((3, 68), np.uint8))],
                       version=2)
    assert GG.scan_gguf(v2).version == 2 and GG.scan_gguf(v2).alignment == 32
    assert GG.scan_gguf(v2).tensor("w").byte_shape == (3, 68)


def test_gguf_reader_on_a_container_packed_without_this_package(tmp_path):
    """tests/golden/tiny_v3.gguf is packed field by field with `struct` (tests/golden/make_tiny_gguf.py), not by
    this package's writer; content and expectations are those of hipEngine's reader test
    (tests/test_unit_gguf_reader.py:54-142): reversed ggml dimensions, 32-byte alignment of the payload, string and
    float arrays, F32 / BF16 / Q8_0 payloads."""
    from pathlib import Path

    import numpy as np

    from hipengine_amd.loading import gguf as GG
    from oracle import gguf_oracle as O

    golden = Path(__file__).parent / "golden" / "tiny_v3.gguf"
    info = GG.scan_gguf(golden)
    assert info.version == 3 and info.alignment == 32 and info.architecture == "toy" and info.file_type == 7
    assert info.metadata["toy.context_length"] == 16
    assert info.metadata["tokenizer.ggml.tokens"] == ["a", "b"]
    assert info.metadata["tokenizer.ggml.scores"] == pytest.approx([0.25, -0.5])
    assert info.tensor_count == 3 and info.names_with_prefix("dense") == ("dense.weight",)
    assert info.tensor_data_offset == 448                       # 435 header bytes rounded up to 32
    dense, bf16, q8 = info.require(["dense.weight", "bf16.weight", "q8.weight"])
    assert dense.shape == (2, 3) and dense.ggml_shape == (3, 2) and dense.ggml_type_name == "F32" and dense.nbytes == 24
    assert bf16.byte_shape == (2,) and bf16.nbytes == 4
    assert q8.shape == (1, 32) and q8.byte_shape == (1, 34) and q8.nbytes == 34
    assert (dense.data_offset, bf16.data_offset, q8.data_offset) == (448, 480, 512)
    reader = GG.GGUFReader(golden)
    assert np.array_equal(reader.tensor_data("dense.weight"), np.arange(6, dtype=np.float32).reshape(2, 3))
    assert np.array_equal(O.bf16_bits_to_f32(np.asarray(reader.tensor_data("bf16.weight"))), np.float32([1.0, -2.5]))
    assert np.array_equal(O.dequantize(np.asarray(reader.tensor_data("q8.weight")), O.GGML_Q8_0)[0],
                          np.arange(-16, 16, dtype=np.float32) * 2.0)
    with pytest.raises(GG.MissingGGUFTensorError, match="missing required GGUF tensors: absent"):
        info.require(["dense.weight", "absent"])
    # the committed file is what the generator writes
    script = golden.with_name("make_tiny_gguf.py").read_text().replace('with_name("tiny_v3.gguf")', f'with_name("{tmp_path.name}.gguf")')
    probe = golden.with_name(f"{tmp_path.name}.gguf")
    try:
        namespace = {"__file__": str(golden.with_name("make_tiny_gguf.py")), "__name__": "make_tiny_gguf"}
        exec(compile(script, "make_tiny_gguf.py", "exec"), namespace)
        namespace["main"]()
        assert probe.read_bytes() == golden.read_bytes()
    finally:
        probe.unlink(missing_ok=True)


def test_bench_refuses_more_than_one_gpu_and_fails_loudly_without_one():
    """bench.py is a one-GPU measurement: --gpus above 1 exits with a message that says so, and without a HIP
    device it stops with an error instead of timing anything else."""
    import subprocess
    import sys
    from pathlib import Path

    root = Path(__file__).resolve().parents[1]
    two = subprocess.run([sys.executable, str(root / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert two.returncode != 0 and "one GPU" in (two.stderr + two.stdout)
    try:
        from hipengine_amd.core.hip import get_hip_runtime
        has_gpu = get_hip_runtime().device_count() > 0
    except Exception:
        has_gpu = False
    if not has_gpu:
        one = subprocess.run([sys.executable, str(root / "bench.py"), "--steps", "2", "--warmup", "1"], capture_output=True,
                             text=True, timeout=120)
        assert one.returncode != 0 and "metric" not in one.stdout
