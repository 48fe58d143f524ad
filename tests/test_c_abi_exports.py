"""The C-ABI library loads and exports every function include/*.h declares.
CPU only: nothing is launched."""

from __future__ import annotations

import ctypes
import re
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
HEADER = ROOT / "include" / "hipengine_gfx950.h"
TUNING_HEADER = ROOT / "include" / "hipengine_gfx950_tuning.h"
LIB = ROOT / "hipengine_amd" / "lib" / "libhipengine_gfx950.so"


def declared_functions() -> list[str]:
    text = subprocess.run(["gcc", "-E", "-P", str(TUNING_HEADER)], check=True, capture_output=True, text=True).stdout   # includes HEADER
    names = re.findall(r"\bint\s+(hipengine_[a-z0-9_]+)\s*\(", text)
    assert len(names) >= 30
    return sorted(set(names))


@pytest.fixture(scope="module")
def library() -> ctypes.CDLL:
    if not LIB.exists():
        from hipengine_amd.core.build import build_hip

        build_hip(load=False)
    return ctypes.CDLL(str(LIB))


def test_header_compiles_as_c_and_cpp(tmp_path):
    src = tmp_path / "t.c"
    src.write_text(f'#include "{HEADER}"\n#include "{TUNING_HEADER}"\nint main(void) {{ return 0; }}\n')
    subprocess.run(["gcc", "-std=c11", "-Wall", "-Werror", "-fsyntax-only", str(src)], check=True)
    subprocess.run(["g++", "-std=c++17", "-Wall", "-Werror", "-fsyntax-only", "-x", "c++", str(src)], check=True)


def test_every_declared_function_is_exported(library):
    missing = [n for n in declared_functions() if not hasattr(library, n)]
    assert not missing, f"declared in the header but not exported: {missing}"


def test_every_exported_entry_point_is_declared():
    out = subprocess.run(["nm", "-D", "--defined-only", str(LIB)], check=True, capture_output=True, text=True).stdout
    exported = {line.split()[-1] for line in out.splitlines() if " T " in line and "hipengine_" in line.split()[-1]
                and not line.split()[-1].startswith("_Z")}
    undeclared = sorted(exported - set(declared_functions()))
    assert not undeclared, f"exported but not declared in the header: {undeclared}"


def test_abi_version_and_host_only_entry_points(library):
    assert library.hipengine_gfx950_abi_version() == 2
    plan = (ctypes.c_int32 * 5)()
    fn = library.hipengine_gfx950_gguf_gemv_default_plan
    fn.argtypes = [ctypes.c_int32, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.POINTER(ctypes.c_int32)]
    assert fn(12, 1, 5120, 17408, plan) == 0 and plan[0] == 1
    assert fn(12, 1, 100, 17408, plan) == 1          # hipErrorInvalidValue
    assert fn(99, 1, 5120, 17408, plan) == 1
    form = (ctypes.c_int32 * 2)()
    ff = library.hipengine_gfx950_gguf_gemv_default_form
    ff.argtypes = [ctypes.c_int32, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.POINTER(ctypes.c_int32)]
    picks = {}
    for name, (qt, rows, k, n) in {"c1": (12, 1, 5120, 17408), "c1_b8": (12, 8, 5120, 17408), "down_b1": (14, 1, 17408, 5120),
                                   "down_b8": (14, 8, 17408, 5120), "head_b4": (14, 4, 5120, 151936), "o_b4": (8, 4, 5120, 5120),
                                   "q4_long_b8": (12, 8, 17408, 5120), "q5_b2": (13, 2, 5120, 4096), "short_k": (12, 1, 512, 64),
                                   "odd_blocks_b8": (14, 8, 256 * 17, 5120), "o_q4_b1": (12, 1, 5120, 5120), "o_q4_b2": (12, 2, 5120, 5120),
                                   "k_q4_b1": (12, 1, 5120, 1024)}.items():
        assert ff(qt, rows, k, n, form) == 0
        picks[name] = (form[0], form[1])
    # 0 row-strided, 1 run, 2 stream, 3 slab, 4 phased slab, 5 direct slab; second field: batch rows of the first launch
    assert picks == {"c1": (2, 1), "c1_b8": (3, 8), "down_b1": (2, 1), "down_b8": (5, 8), "head_b4": (4, 4), "o_b4": (4, 4),
                     "q4_long_b8": (5, 8), "q5_b2": (2, 2), "short_k": picks["short_k"], "odd_blocks_b8": (2, 8), "o_q4_b1": (2, 1), "o_q4_b2": (2, 2), "k_q4_b1": (2, 1)}
    assert picks["short_k"][0] in (0, 1)
    assert ff(12, 1, 100, 64, form) == 1
    # argument checks come before any HIP call: null pointers and bad sizes are refused on a host without a GPU
    ps = library.hipengine_gfx950_gguf_q8_1_fused_gemv_pslab_tuned
    ps.argtypes = [ctypes.c_int32, ctypes.c_void_p, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32,
                   ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32,
                   ctypes.c_void_p]
    assert ps(14, None, 0, None, None, 0, 8, 5120, 5120, 0, 0, 0, None) == 1
    assert ps(14, 16, 0, 16, 16, 0, 9, 5120, 5120, 0, 0, 0, None) == 1        # more than 8 batch rows
    assert ps(14, 16, 0, 16, 16, 0, 8, 256 * 17, 5120, 0, 0, 0, None) == 1    # odd block count: not this form
    assert ps(14, 16, 0, 18, 16, 0, 8, 5120, 5120, 0, 0, 0, None) == 1        # weights not 4-byte aligned
    assert ps(14, 16, 0, 16, 16, 0, 8, 5120, 5120, 13, 1, 0, None) == 1       # more than 12 waves
    ds = library.hipengine_gfx950_gguf_q8_1_fused_gemv_dslab_tuned
    ds.argtypes = [ctypes.c_int32, ctypes.c_void_p, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32,
                   ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32,
                   ctypes.c_int32, ctypes.c_void_p]
    assert ds(14, None, 0, None, None, 0, 8, 5120, 5120, 0, 0, 0, 0, None) == 1
    assert ds(13, 16, 0, 16, 16, 0, 8, 5120, 5120, 0, 0, 0, 0, None) == 1      # Q5_K: not this form
    assert ds(14, 16, 0, 16, 16, 0, 8, 5120, 5120, 0, 0, 0, 3, None) == 1      # K parts: 1, 2 or 4
    assert ds(14, 16, 0, 17, 16, 0, 8, 5120, 5120, 0, 0, 0, 0, None) == 1      # weights not 2-byte aligned
    # the one-call prefill refuses what its MMQ would refuse before it packs anything: nothing is enqueued or written
    pf = library.hipengine_gfx950_gguf_prefill_bf16
    pf.argtypes = [ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64,
                   ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p]
    big = 1 << 30
    assert pf(12, 16, 16, 16, 0, 64, 1024, 33, 16, big, None) == 1             # Q4_K: out_features % 32
    assert pf(13, 16, 16, 16, 0, 64, 1024, 40, 16, big, None) == 1             # Q5_K likewise
    assert pf(14, 16, None, 16, 0, 64, 1024, 40, 16, big, None) == 1           # no weights
    assert pf(14, 16, 16, None, 0, 64, 1024, 40, 16, big, None) == 1           # no output
    assert pf(14, 16, 16, 16, 7, 64, 1024, 40, 16, big, None) == 1             # output kind
    assert pf(8, 16, 16, 16, 0, 64, 1024, (1 << 24) + 1, 16, big, None) == 1   # out_features out of range


def test_form_picks_hold_their_invariants_over_many_shapes(library):
    """Host only: whatever the shape, the dispatcher names a form that exists, starts with 1..8 rows of the batch
    (never more than asked), streams batch 1-2 wherever a matrix gives every CU a group of blocks, and takes the direct
    slab form only for the types and row lengths it is built for."""
    import random

    ff = library.hipengine_gfx950_gguf_gemv_default_form
    ff.argtypes = [ctypes.c_int32, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.POINTER(ctypes.c_int32)]
    form = (ctypes.c_int32 * 2)()
    rng = random.Random(7)
    seen = set()
    shapes = [(qt, rows, 256 * nb, n) for qt in (8, 12, 13, 14) for rows in (1, 2, 3, 5, 8, 11, 64)
              for nb in (1, 2, 16, 17, 20, 24, 25, 68, 96) for n in (1, 33, 1024, 5120, 17408)]
    shapes += [(rng.choice((8, 12, 13, 14)), rng.randint(1, 40), 256 * rng.randint(1, 80), rng.randint(1, 200000))
               for _ in range(2000)]
    for qt, rows, k, n in shapes:
        assert ff(qt, rows, k, n, form) == 0, (qt, rows, k, n)
        kind, first = form[0], form[1]
        seen.add(kind)
        assert 0 <= kind <= 5 and 1 <= first <= min(rows, 8), (qt, rows, k, n, kind, first)
        if first <= 2 and k >= 4096 and n * (k // 256) >= 16 * 256:
            assert kind == 2, (qt, rows, k, n, kind, first)               # a group of 16 blocks per CU or more: the stream form
        if kind == 3:
            assert qt == 12 and k <= 6144                                 # (batch 1-2 only where a matrix is too small to stream)
        if kind == 5:
            assert qt in (8, 12, 14) and k > 6144 and first >= (5 if qt == 8 else 3)
            assert (k // 256) % 2 == 0, (qt, rows, k, n)                   # K parts of equal length only
        if kind == 4:
            assert k % 512 == 0, (qt, rows, k, n)                          # the phased slab takes K blocks in pairs
    assert seen == {0, 1, 2, 3, 4, 5}
    assert ff(12, 0, 5120, 64, form) == 1 and ff(12, 1, 5120, 0, form) == 1 and ff(12, 1, 5000, 64, form) == 1
