"""The attention entry point that allocates nothing (`trocm_sdpa_cached_noalloc`: split-K scratch in a
static device array) against `trocm_sdpa_cached` with a caller's workspace, through the C ABI: same
kernels, same arguments, so the outputs must agree; two calls in a row, the second with a smaller
input, so that whatever the first left in the shared scratch is seen by the second."""
import ctypes as C

import numpy as np
import pytest

import tract_amd as ta
from tract_amd import _lib
from tract_amd.runtime import DeviceTensor, Stream, Workspace
from tests.gpu_util import max_abs, rt  # noqa: F401

pytestmark = pytest.mark.gpu


def _caches(rng, fmt, B, Hkv, T, D, dtype):
    k = rng.standard_normal((B, Hkv, T, D), dtype=np.float32).astype(dtype)
    v = rng.standard_normal((B, Hkv, T, D), dtype=np.float32).astype(dtype)
    kc, vc = ta.InPlaceKvCache(2, storage_format=fmt), ta.InPlaceKvCache(2, storage_format=fmt)
    kc.push(k)
    vc.push(v)
    return kc, vc


def _both(rng, stream, fmt, dtype, B, Hq, Hkv, Sq, T, D, causal):
    kc, vc = _caches(rng, fmt, B, Hkv, T, D, dtype)
    q = DeviceTensor.from_numpy((rng.standard_normal((B, Hq, Sq, D), dtype=np.float32) / np.sqrt(D)).astype(dtype))
    code = ta.F16 if dtype == np.float16 else ta.F32
    ws = Workspace(B, Hq, Sq, D)
    want_t = DeviceTensor(q.shape, q.dtype)
    _lib.call("trocm_sdpa_cached", q.ptr, code, Hq, Sq, kc.handle, vc.handle, want_t.ptr, C.c_float(float("nan")), int(causal),
              ws.ptr, ws.nbytes, stream.handle)
    got_t = DeviceTensor(q.shape, q.dtype)
    _lib.call("trocm_sdpa_cached_noalloc", q.ptr, code, Hq, Sq, kc.handle, vc.handle, got_t.ptr, C.c_float(float("nan")),
              int(causal), stream.handle)
    stream.synchronize()
    return got_t.to_numpy(), want_t.to_numpy()


# (format, dtype, batch, q heads, kv heads, queries, tokens, head_dim, causal): a larger call, then a smaller one
PAIRS = [
    # split-K decode on the matrix cores: 4 splits with the in-kernel merge, then 16 splits (wide merge)
    [(None, np.float16, 8, 32, 8, 1, 4133, 128, True), (None, np.float16, 2, 32, 8, 1, 2050, 128, True)],
    # 16 heads per kv head: partials + merge launch; then one head per kv head on the vector-ALU kernel, f32
    [(None, np.float16, 2, 32, 2, 1, 3000, 128, False), (None, np.float32, 1, 8, 8, 1, 777, 64, False)],
    # quantised caches
    [(ta.Q8_0, np.float16, 4, 32, 8, 1, 4096, 128, True), (ta.Q4_0, np.float16, 1, 32, 8, 1, 1000, 128, True)],
    # prefill with the key range split over workgroups (f16 partials in the scratch), then a short one
    [(None, np.float16, 1, 32, 8, 256, 2048, 128, True), (None, np.float16, 1, 8, 2, 64, 192, 64, True)],
]


@pytest.mark.parametrize("pair", PAIRS, ids=["decode_f16", "decode_g16_then_f32", "decode_quant", "prefill"])
def test_noalloc_matches_the_workspace_entry_point(rt, pair):
    rng = np.random.default_rng(77)
    stream = Stream()
    for (fmt, dtype, B, Hq, Hkv, Sq, T, D, causal) in pair:
        got, want = _both(rng, stream, fmt, dtype, B, Hq, Hkv, Sq, T, D, causal)
        assert np.isfinite(got.astype(np.float32)).all()
        tol = 1e-3 if dtype == np.float32 else 2e-2   # the bar of the attention outputs
        assert max_abs(got, want) <= tol, (fmt, B, Hq, Sq, T, max_abs(got, want))
        # the same kernels in the same order: in practice the bits agree
        assert np.array_equal(got, want), (fmt, B, Hq, Sq, T, max_abs(got, want))


def test_noalloc_refuses_what_does_not_fit_and_a_null_stream(rt):
    rng = np.random.default_rng(5)
    stream = Stream()
    kc, vc = _caches(rng, None, 1, 8, 64, 128, np.float16)
    lib = _lib.load()
    Hq = 8 * 8192   # 65536 query heads: the records of a split would not fit the static scratch
    q = DeviceTensor((1, 8, 1, 128), np.float16)   # never read: the call is refused on its sizes
    out = DeviceTensor((1, 8, 1, 128), np.float16)
    rc = lib.trocm_sdpa_cached_noalloc(q.ptr, ta.F16, Hq, 1, kc.handle, vc.handle, out.ptr, C.c_float(1.0), 0, stream.handle)
    assert rc == 1 and b"static buffer" in lib.trocm_last_error()
    rc = lib.trocm_sdpa_cached_noalloc(q.ptr, ta.F16, 8, 1, kc.handle, vc.handle, out.ptr, C.c_float(1.0), 0, None)
    assert rc == 1 and b"stream is required" in lib.trocm_last_error()
    # and the entry point still works afterwards
    lib_rc = lib.trocm_sdpa_cached_noalloc(q.ptr, ta.F16, 8, 1, kc.handle, vc.handle, out.ptr, C.c_float(1.0), 0, stream.handle)
    assert lib_rc == 0
    stream.synchronize()
