"""The C ABI is re-entrant across host threads: each thread gets a stream of its own (the
reference keeps one stream per host thread in thread-local storage, cuda/src/context.rs:37-43), its
own op states and workspaces, and its own last-error string (api/ffi/src/lib.rs:18-62).  Four
threads run different decode workloads at once; every result must equal, bit for bit, what the
same workload gives when it runs alone."""
import threading

import numpy as np
import pytest

import tract_amd
from oracle import oracle as orc
from tests.gpu_util import max_abs, rt  # noqa: F401

pytestmark = pytest.mark.gpu


def workload(kind, seed, steps=24):
    rng = np.random.default_rng(seed)
    B, Hq, Hkv, D, T0 = 2, 32, 8, 128, 700 + 37 * seed
    dt = np.float16
    fmt = {"f16": None, "q8": tract_amd.Q8_0, "q4": tract_amd.Q4_0, "window": None}[kind]
    if kind == "window":
        st = tract_amd.WindowKvSdpa(axis=2, window=512).state()
    else:
        st = tract_amd.InPlaceKvSdpa(axis=2, causal=True, storage_format=fmt).state()
    k = rng.standard_normal((B, Hkv, T0, D), dtype=np.float32).astype(dt)
    v = rng.standard_normal((B, Hkv, T0, D), dtype=np.float32).astype(dt)
    q = (rng.standard_normal((B, Hq, T0, D), dtype=np.float32) / np.sqrt(D)).astype(dt)
    outs = [st.eval([q, k, v]).to_numpy()]
    for _ in range(steps):
        q1 = (rng.standard_normal((B, Hq, 1, D), dtype=np.float32) / np.sqrt(D)).astype(dt)
        k1 = rng.standard_normal((B, Hkv, 1, D), dtype=np.float32).astype(dt)
        v1 = rng.standard_normal((B, Hkv, 1, D), dtype=np.float32).astype(dt)
        outs.append(st.eval([q1, k1, v1]).to_numpy())
    outs.append(st.k.valid_contiguous())
    return outs


def test_four_threads_at_once_equal_the_same_work_alone(rt):
    jobs = [("f16", 1), ("q8", 2), ("q4", 3), ("window", 4)]
    alone = [workload(kind, seed) for kind, seed in jobs]
    together, errors = [None] * len(jobs), []

    def run(i):
        try:
            for _ in range(3):   # several rounds, so that the threads overlap for a while
                together[i] = workload(*jobs[i])
        except Exception as e:  # noqa: BLE001
            errors.append((i, repr(e)))

    threads = [threading.Thread(target=run, args=(i,)) for i in range(len(jobs))]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not errors, errors
    for (kind, _), a, b in zip(jobs, alone, together):
        assert b is not None and len(a) == len(b), kind
        for x, y in zip(a, b):
            assert x.tobytes() == y.tobytes(), kind


def test_last_error_is_per_thread(rt):
    """Thread A fails, then thread B fails with another message, then A reads its error: still its own."""
    import ctypes as C
    from tract_amd._lib import load
    lib = load()
    seen = {}
    a_failed, b_failed = threading.Event(), threading.Event()

    def thread_a():
        assert lib.trocm_kv_cache_len(None, None) == 1
        a_failed.set()
        b_failed.wait(30)
        seen["a"] = lib.trocm_last_error()

    def thread_b():
        a_failed.wait(30)
        sz = C.c_size_t()
        assert lib.trocm_sdpa_workspace_bytes(-1, 1, 1, 64, C.byref(sz)) == 1
        seen["b"] = lib.trocm_last_error()
        b_failed.set()

    ta, tb = threading.Thread(target=thread_a), threading.Thread(target=thread_b)
    ta.start(), tb.start(), ta.join(60), tb.join(60)
    assert b"null pointer" in seen["a"] and b"negative" in seen["b"]
