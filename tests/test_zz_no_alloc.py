"""The arg-max entry point that allocates nothing (`hipengine_gfx950_argmax_f32_rows_i32_noalloc`, stage
scratch held inside the library) against the entry point it is a variant of (`hipengine_argmax_f32_rows_i32`,
caller-owned scratch): same indices and values, bit for bit, on two calls in a row, the second with a smaller
input, so that whatever the first call left in the shared scratch would show.  Both go through the C ABI.
"""

from __future__ import annotations

import ctypes

import numpy as np
import pytest

from hipengine_amd.kernels.hip_gfx950.linear import lm_head as L

pytestmark = pytest.mark.gpu


def _reference(dev, logits: np.ndarray, threads: int):
    rows, vocab = logits.shape
    n = L.argmax_scratch_entries(rows, vocab, threads)
    dl, bv, bi = dev.put(logits), dev.empty(n * 4), dev.empty(n * 4)
    oi, ov = dev.empty(rows * 4), dev.empty(rows * 4)
    L.argmax_f32_rows_i32(dl.ptr, bv.ptr, bi.ptr, oi.ptr, ov.ptr, rows, vocab, threads=threads)
    got = dev.get(oi, np.int32, (rows,)).copy(), dev.get(ov, np.uint32, (rows,)).copy()
    dev.free(dl, bv, bi, oi, ov)
    return got


def _noalloc(dev, logits: np.ndarray, threads: int):
    rows, vocab = logits.shape
    dl, oi, ov = dev.put(logits), dev.empty(rows * 4), dev.empty(rows * 4)
    L.argmax_f32_rows_i32_noalloc(dl.ptr, oi.ptr, ov.ptr, rows, vocab, threads=threads)
    got = dev.get(oi, np.int32, (rows,)).copy(), dev.get(ov, np.uint32, (rows,)).copy()
    dev.free(dl, oi, ov)
    return got


def _logits(rng, rows: int, vocab: int) -> np.ndarray:
    x = rng.standard_normal((rows, vocab)).astype(np.float32)
    # equal maxima in every row: the lowest index must win, in both entry points
    for r in range(rows):
        hi = np.float32(x[r].max() + 1.0)
        x[r, [(7 * r + 11) % vocab, (vocab - 1 - r) % vocab]] = hi
    return x


def test_noalloc_argmax_matches_caller_scratch_twice(dev):
    rng = np.random.default_rng(20260401)
    # first call: the lm_head vocabulary at batch 8 (1192 pairs of scratch); second: smaller in both dimensions
    for rows, vocab, threads in ((8, 151936, 256), (3, 4099, 128)):
        x = _logits(rng, rows, vocab)
        want_i, want_v = _reference(dev, x, threads)
        got_i, got_v = _noalloc(dev, x, threads)
        assert np.array_equal(want_i, np.argmax(x, axis=1).astype(np.int32))
        assert np.array_equal(got_i, want_i)
        assert np.array_equal(got_v, want_v)


def test_noalloc_argmax_rejects_sizes_beyond_the_scratch(dev):
    x = dev.put(np.zeros(16, dtype=np.float32))
    out = dev.empty(4 * 65535)
    fn = dev.library.hipengine_gfx950_argmax_f32_rows_i32_noalloc
    fn.argtypes = [ctypes.c_void_p] * 3 + [ctypes.c_int64] * 3 + [ctypes.c_void_p]
    fn.restype = ctypes.c_int
    # 4096 rows x 17 blocks = 69632 pairs > 65536: refused before any launch (the pointers are never read)
    assert fn(x.ptr, out.ptr, None, 4096, 17 * 1024, 256, None) == 1
    with pytest.raises(ValueError, match="scratch"):
        L.argmax_f32_rows_i32_noalloc(x.ptr, out.ptr, None, 4096, 17 * 1024)
    dev.free(x, out)
