"""Behaviour at the edges of the boundary: growth that does not stall the host, calls that fail before they change
anything, and rows that a mask hides entirely."""
import ctypes as C
import time

import numpy as np
import pytest

import tract_amd as ta
from oracle import oracle as orc
from tests import cases
from tests.gpu_util import max_abs, rt  # noqa: F401
from tract_amd._lib import call, load
from tract_amd.runtime import DeviceTensor, Stream, Workspace

pytestmark = pytest.mark.gpu
NAN = C.c_float(float("nan"))


def test_growing_append_then_attention_without_a_host_sync(rt):
    """A step that doubles the capacity, then attention over the grown caches, queued behind ~100 ms of other work
    on the same stream: the calls return while that work is still running (growth does not wait for the stream),
    and contents and outputs are what the synchronous order gives."""
    B, Hq, Hkv, D, T = 2, 32, 8, 128, 1024
    rng = np.random.default_rng(3)
    k = rng.standard_normal((B, Hkv, T, D), dtype=np.float32).astype(np.float16)
    v = rng.standard_normal((B, Hkv, T, D), dtype=np.float32).astype(np.float16)
    kn = rng.standard_normal((3, B, Hkv, 1, D), dtype=np.float32).astype(np.float16)
    vn = rng.standard_normal((3, B, Hkv, 1, D), dtype=np.float32).astype(np.float16)
    q = (rng.standard_normal((3, B, Hq, 1, D), dtype=np.float32) / np.sqrt(D)).astype(np.float16)
    stream = Stream()
    st = ta.InPlaceKvSdpa(axis=2, causal=True).state()
    st.k.push(k, stream=stream), st.v.push(v, stream=stream)
    dq, dk, dv = DeviceTensor.from_numpy(q), DeviceTensor.from_numpy(kn), DeviceTensor.from_numpy(vn)
    outs = DeviceTensor((3, B, Hq, 1, D), np.float16)
    ws = Workspace(B, Hq, 1, D)
    big = DeviceTensor((1 << 30,), np.uint8)   # 1 GiB, copied onto itself's other half many times: ~100 ms of queued work
    half = 1 << 29
    shape, st1 = (C.c_int64 * 1)(half // 16), (C.c_int64 * 1)(1)
    stream.synchronize()
    t0 = time.perf_counter()
    for _ in range(500):
        call("trocm_copy_nd", big.ptr, half, st1, big.ptr, 0, st1, shape, 1, 16, stream.handle)
    t_queued = time.perf_counter()
    row_q, row_kv = B * Hq * D * 2, B * Hkv * D * 2
    for s in range(3):   # the first step grows both caches 1024 -> 2048
        call("trocm_inplace_kv_sdpa_eval", C.c_void_p(dq.ptr.value + s * row_q), C.c_void_p(dk.ptr.value + s * row_kv),
             C.c_void_p(dv.ptr.value + s * row_kv), ta.F16, Hq, 1, None, st.k.handle, st.v.handle,
             C.c_void_p(outs.ptr.value + s * row_q), NAN, 1, ws.ptr, ws.nbytes, stream.handle)
    t_steps = time.perf_counter()
    stream.synchronize()
    t_done = time.perf_counter()
    assert st.k.capacity() == 2 * T and st.k.reallocs() == 1 and st.k.len() == T + 3
    # the three steps were issued in a fraction of the time the queue needed to drain
    assert (t_steps - t_queued) < 0.25 * (t_done - t_queued), (t_queued - t0, t_steps - t_queued, t_done - t_steps)
    kc, vc = k, v
    got = outs.to_numpy()
    for s in range(3):
        kc, vc = np.concatenate([kc, kn[s]], axis=2), np.concatenate([vc, vn[s]], axis=2)
        assert max_abs(got[s], orc.flash_sdpa(q[s], kc, vc, causal=True, threads=8)) <= 2e-2, f"step {s}"
    assert st.k.valid_contiguous().tobytes() == kc.tobytes()
    assert st.v.valid_contiguous().tobytes() == vc.tobytes()


@pytest.mark.parametrize("fmt", [None, ta.Q8_0])
def test_a_refused_step_changes_nothing_and_can_be_repeated(rt, fmt):
    B, Hq, Hkv, D, T = 1, 8, 2, 128, 100
    rng = np.random.default_rng(4)
    k = rng.standard_normal((B, Hkv, T, D), dtype=np.float32).astype(np.float16)
    st = ta.InPlaceKvSdpa(axis=2, causal=True, storage_format=fmt).state()
    st.k.push(k), st.v.push(k)
    lib = load()
    q = DeviceTensor.from_numpy((rng.standard_normal((B, Hq, 1, D), dtype=np.float32) / np.sqrt(D)).astype(np.float16))
    kn = DeviceTensor.from_numpy(rng.standard_normal((B, Hkv, 1, D), dtype=np.float32).astype(np.float16))
    out = DeviceTensor((B, Hq, 1, D), np.float16)
    ws = Workspace(B, Hq, 1, D)
    before = st.k.valid_contiguous().tobytes()
    bad = [
        dict(out=None),                       # NULL output
        dict(q=None),                         # NULL query
        dict(q_heads=7),                      # not a multiple of the kv heads
        dict(dtype=ta.F32) if fmt is None else dict(dtype=5),   # a dtype the cache does not hold / no dtype at all
    ]
    for change in bad:
        a = dict(q=q.ptr, out=out.ptr, q_heads=Hq, dtype=ta.F16)
        a.update(change)
        rc = lib.trocm_inplace_kv_sdpa_eval(a["q"], kn.ptr, kn.ptr, a["dtype"], a["q_heads"], 1, None, st.k.handle, st.v.handle,
                                            a["out"], NAN, 1, ws.ptr, ws.nbytes, None)
        assert rc == 1, change
        assert (st.k.len(), st.v.len()) == (T, T), f"{change}: the refused call appended"
    assert st.k.valid_contiguous().tobytes() == before
    call("trocm_inplace_kv_sdpa_eval", q.ptr, kn.ptr, kn.ptr, ta.F16, Hq, 1, None, st.k.handle, st.v.handle, out.ptr, NAN, 1,
         ws.ptr, ws.nbytes, None)
    assert (st.k.len(), st.v.len()) == (T + 1, T + 1)


def test_a_step_that_runs_out_of_pool_memory_can_be_repeated(rt):
    """K grows, V does not fit: the call fails with the token not appended; once there is room the same call
    brings V up to K's capacity and goes through."""
    B, Hq, Hkv, D, T = 1, 8, 2, 64, 1024
    plane = lambda pitch: B * Hkv * pitch * D * 2
    grown = plane(2048 + 64)    # capacity 2048 pads its rows by 1/32
    filler_tokens = 2400
    pool = ta.KvPool(2 * plane(T) + plane(filler_tokens + 80) + grown + 4096)
    rng = np.random.default_rng(5)
    k = rng.standard_normal((B, Hkv, T, D), dtype=np.float32).astype(np.float16)
    v = rng.standard_normal((B, Hkv, T, D), dtype=np.float32).astype(np.float16)
    kc, vc = ta.InPlaceKvCache(2, pool=pool), ta.InPlaceKvCache(2, pool=pool)
    kc.push(k), vc.push(v)
    filler = ta.InPlaceKvCache(2, pool=pool)
    filler.push(np.zeros((B, Hkv, filler_tokens, D), np.float16))
    q = (rng.standard_normal((B, Hq, 1, D), dtype=np.float32) / np.sqrt(D)).astype(np.float16)
    kn = rng.standard_normal((B, Hkv, 1, D), dtype=np.float32).astype(np.float16)
    vn = rng.standard_normal((B, Hkv, 1, D), dtype=np.float32).astype(np.float16)
    dq, dk, dv = DeviceTensor.from_numpy(q), DeviceTensor.from_numpy(kn), DeviceTensor.from_numpy(vn)
    out = DeviceTensor((B, Hq, 1, D), np.float16)
    ws = Workspace(B, Hq, 1, D)
    lib = load()
    args = (dq.ptr, dk.ptr, dv.ptr, ta.F16, Hq, 1, None, kc.handle, vc.handle, out.ptr, NAN, 1, ws.ptr, ws.nbytes, None)
    assert lib.trocm_inplace_kv_sdpa_eval(*args) == 1
    assert b"pool exhausted" in lib.trocm_last_error()
    assert (kc.len(), vc.len()) == (T, T)
    assert (kc.capacity(), vc.capacity()) == (2 * T, T)   # K had grown before V failed
    assert lib.trocm_inplace_kv_sdpa_eval(*args) == 1      # still no room: still refused, still nothing appended
    assert (kc.len(), vc.len()) == (T, T)
    filler.close()
    call("trocm_inplace_kv_sdpa_eval", *args)
    assert (kc.len(), vc.len(), kc.capacity(), vc.capacity()) == (T + 1, T + 1, 2 * T, 2 * T)
    kk, vv = np.concatenate([k, kn], axis=2), np.concatenate([v, vn], axis=2)
    assert max_abs(out.to_numpy(), orc.flash_sdpa(q, kk, vv, causal=True)) <= 2e-2
    assert kc.valid_contiguous().tobytes() == kk.tobytes() and vc.valid_contiguous().tobytes() == vv.tobytes()
    kc.close(), vc.close(), pool.close()


@pytest.mark.parametrize("dt,B,Hq,Hkv,Sq,Sk,D", [
    (np.float16, 2, 32, 8, 1, 2052, 128),    # split-K decode on the matrix cores, in-kernel merge
    (np.float16, 1, 32, 8, 1, 4100, 128),    # ... 32 splits: the wide merge
    (np.float16, 2, 32, 2, 1, 1028, 128),    # ... 16 heads per kv head: the merge launch
    (np.float16, 2, 32, 8, 1, 2051, 128),    # odd length: the vector-ALU decode kernel (4 heads per kv head)
    (np.float32, 2, 8, 4, 1, 513, 64),       # f32: the vector-ALU decode kernel
    (np.float16, 1, 8, 2, 64, 256, 128),     # the MFMA prefill kernel
    (np.float32, 1, 4, 2, 5, 40, 32),        # the generic kernel
])
def test_a_row_masked_out_entirely_with_minus_infinity_yields_zeros(rt, dt, B, Hq, Hkv, Sq, Sk, D):
    """Whichever kernel the shape selects: a query row whose every key carries -inf comes back as zeros (the CPU
    op's tile skip leaves such a row of a decode call at its zero initialisation), and its neighbours are untouched."""
    rng = np.random.default_rng(Sk)
    q = (rng.standard_normal((B, Hq, Sq, D), dtype=np.float32) / np.sqrt(D)).astype(dt)
    k = rng.standard_normal((B, Hkv, Sk, D), dtype=np.float32).astype(dt)
    v = rng.standard_normal((B, Hkv, Sk, D), dtype=np.float32).astype(dt)
    mask = np.zeros((B, Hq, Sq, Sk), dt)
    mask[0, 1, 0, :] = -np.inf             # one head's (first) query of the first sequence
    mask[B - 1, Hq - 1, Sq - 1, :] = -np.inf
    mask[0, 2, 0, : Sk // 2] = -np.inf     # half hidden: an ordinary row
    got = ta.Sdpa(datum_type=dt).eval(q, k, v, mask).to_numpy()
    assert not np.isnan(got).any()
    assert not got[0, 1, 0].any() and not got[B - 1, Hq - 1, Sq - 1].any()
    want = cases.textbook_sdpa(q, k, v, np.where(np.isinf(mask), -1e30, mask.astype(np.float64)))
    keep = np.ones((B, Hq, Sq), bool)
    keep[0, 1, 0] = keep[B - 1, Hq - 1, Sq - 1] = False
    assert max_abs(got[keep], want[keep]) <= (1e-3 if dt == np.float32 else 2e-2)


def test_launch_floor_kernels_run_and_refuse_bad_shapes(rt):
    """The measurement aid: an empty kernel and a read-only streaming kernel on a given launch shape.  They write
    nothing (the buffer and the 4-byte sink stay as they were) and refuse shapes that are not launches."""
    src = DeviceTensor.from_numpy(np.arange(1 << 20, dtype=np.uint32))
    sink = DeviceTensor.from_numpy(np.array([7], dtype=np.uint32))
    for wg, th in ((1, 64), (256, 256), (2048, 256), (256, 1024)):
        call("trocm_launch_floor", 0, None, 0, wg, th, None, None)
        call("trocm_launch_floor", 1, src.ptr, 4 << 20, wg, th, sink.ptr, None)
    call("trocm_launch_floor", 1, src.ptr, 16 * 1000 + 16, 512, 256, None, None)   # a size that is no multiple of the grid
    ta.synchronize()
    assert sink.to_numpy()[0] == 7 and np.array_equal(src.to_numpy(), np.arange(1 << 20, dtype=np.uint32))
    lib = load()
    for args in ((2, src.ptr, 16, 1, 64, None, None), (1, None, 16, 1, 64, None, None), (1, src.ptr, 24, 1, 64, None, None),
                 (0, None, 0, 0, 64, None, None), (0, None, 0, 1, 96, None, None), (0, None, 0, 1, 2048, None, None)):
        assert lib.trocm_launch_floor(*args) == 1
        assert b"launch_floor" in lib.trocm_last_error() or b"null pointer" in lib.trocm_last_error()


def test_release_unused_frees_what_growth_left_behind(rt):
    """A cache that grows outside a pool leaves its old planes on a list guarded by an event; a host that never calls
    one of the library's synchronising entry points releases them with trocm_release_unused.  Contents stay."""
    B, H, D = 1, 2, 64
    rng = np.random.default_rng(9)
    c = ta.InPlaceKvCache(2)
    chunks = [rng.standard_normal((B, H, n, D), dtype=np.float32).astype(np.float16) for n in (16, 16, 40, 200)]
    for x in chunks:
        c.push(x)                       # 16 -> 32 -> 72 -> 272: three reallocations
        call("trocm_release_unused", 0)  # never waits: frees what the device has finished with
    call("trocm_release_unused", 1)      # waits for the rest
    call("trocm_release_unused", 1)      # nothing left: still fine
    assert c.reallocs() == 3
    assert c.valid_contiguous().tobytes() == np.concatenate(chunks, axis=2).tobytes()
