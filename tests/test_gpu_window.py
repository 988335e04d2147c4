"""Sliding-window (ring buffer) KV cache and WindowKvSdpa on the GPU vs the oracle: buffer bytes,
len and cursor bit-exact; attention within the path's tolerance."""
import numpy as np
import pytest

import tract_amd
from oracle import oracle as orc
from tests import cases
from tests.gpu_util import max_abs, rt  # noqa: F401

pytestmark = pytest.mark.gpu


def test_window_holds_last_w_as_a_set(rt):
    # window_kv_cache.rs:342-362
    w = 4
    c = tract_amd.WindowKvCache(2, w)
    full = []
    for t in range(10):
        c.push(np.full((1, 1, 1, 1), float(t), np.float32))
        full.append(float(t))
        assert c.len() <= w
        assert sorted(c.valid_view().ravel().tolist()) == sorted(full[-w:])
    assert c.capacity() == w


def test_prefill_chunk_larger_than_window_keeps_last_w(rt):
    # window_kv_cache.rs:364-374
    c = tract_amd.WindowKvCache(2, 3)
    c.push(np.arange(7, dtype=np.float32).reshape(1, 1, 7, 1))
    assert c.valid_view().ravel().tolist() == [4.0, 5.0, 6.0]
    assert c.cursor() == 0 and c.len() == 3 and c.capacity() == 3


@pytest.mark.parametrize("dt", [np.float32, np.float16])
@pytest.mark.parametrize("w,chunks", [(5, [3, 4, 3, 0, 1, 1, 9, 2, 5, 5, 1]), (64, [1] * 70 + [33, 40, 64, 65, 1]),
                                      (33, [7, 7, 7, 7, 7, 100, 1, 32, 2])])
def test_ring_buffer_bytes_equal_the_oracle(rt, dt, w, chunks):
    rng = np.random.default_rng(w)
    B, H, D = 2, 3, 64
    g, o = tract_amd.WindowKvCache(2, w), orc.WindowKvCache(w)
    for n in chunks:
        x = rng.standard_normal((B, H, n, D)).astype(dt)
        g.push(x), o.push(x)
        assert (g.len(), g.cursor()) == (o.len(), o.cursor())
        if o.len():
            assert g.valid_view().tobytes() == o.valid_view().tobytes()
    assert g.capacity() == w and g.reallocs() == 0


def test_refusals(rt):
    c = tract_amd.WindowKvCache(2, 6)
    c.push(np.zeros((1, 2, 4, 32), np.float32))
    with pytest.raises(tract_amd.TractRocmError, match="sliding-window"):
        c.truncate(1)
    with pytest.raises(tract_amd.TractRocmError, match="fixed capacity"):
        c.reserve(100)
    with pytest.raises(tract_amd.TractRocmError, match="window must be > 0"):
        tract_amd.WindowKvCache(2, 0)


@pytest.mark.parametrize("fmt", ["q8_0", "q4_0"])
def test_quantised_ring_buffer_blocks_equal_the_oracle(rt, fmt):
    code = {"q8_0": tract_amd.Q8_0, "q4_0": tract_amd.Q4_0}[fmt]
    ofmt = {"q8_0": orc.FMT_Q8_0, "q4_0": orc.FMT_Q4_0}[fmt]
    rng = np.random.default_rng(9)
    w, B, H, D = 7, 1, 2, 64
    g = tract_amd.WindowKvCache(2, w, storage_format=code)
    o = orc.WindowKvCache(w)
    for n in [3, 3, 3, 1, 12, 2]:
        x = rng.standard_normal((B, H, n, D)).astype(np.float32)
        g.push(x)
        blocks = orc.quant(ofmt, x.reshape(-1, 32)).reshape(B, H, n, -1)   # canonical block bytes per token row
        o.push(blocks)
        assert g.valid_view().tobytes() == o.valid_view().tobytes()


def test_window_sdpa_decode_matches_last_w_in_model(rt):
    # window_kv_cache.rs:468-527: b=1, h=2, d=16, w=5, 15 steps, values base + sin(0.013 i)
    b, h, d, w = 1, 2, 16, 5
    st = tract_amd.WindowKvSdpa(axis=2, window=w, scale=None).state()

    def mk(base):
        return (base + np.sin(np.arange(b * h * d, dtype=np.float32) * np.float32(0.013))).astype(np.float32).reshape(b, h, 1, d)

    kf, vf = [], []
    for t in range(15):
        qi, ki, vi = mk(9.0 + t * 0.1), mk(1.0 + t * 0.07), mk(5.0 - t * 0.05)
        o_model = st.eval([qi, ki, vi]).to_numpy()
        kf.append(ki), vf.append(vi)
        n = min(len(kf), w)
        o_ref = cases.textbook_sdpa(qi, np.concatenate(kf[-n:], 2), np.concatenate(vf[-n:], 2))
        assert max_abs(o_model, o_ref) <= 1e-3, t


@pytest.mark.parametrize("dt,fmt,tol", [(np.float16, None, 2e-2), (np.float32, None, 1e-3), (np.float16, "q8_0", 2e-2)])
def test_window_sdpa_llm_shape_long_run(rt, dt, fmt, tol):
    """GQA decode (32 q / 8 kv heads, d=128) with a 300-slot window: a 200-token prompt chunk, a
    150-token chunk that wraps, then single tokens across two more wrap-arounds; every step
    equals the oracle's windowed op (ring buffer + attend-all) and attention over the last w."""
    code = {None: None, "q8_0": tract_amd.Q8_0}[fmt]
    rng = np.random.default_rng(21)
    B, Hq, Hkv, D, w = 2, 32, 8, 128, 300
    st = tract_amd.WindowKvSdpa(axis=2, window=w, storage_format=code).state()
    ok, ov = orc.WindowKvCache(w), orc.WindowKvCache(w)
    kf, vf = [], []
    for step, S in enumerate([200, 150] + [1] * 12 + [299] + [1] * 3):
        q = (rng.standard_normal((B, Hq, S, D)) / np.sqrt(D)).astype(dt)
        k = rng.standard_normal((B, Hkv, S, D)).astype(dt)
        v = rng.standard_normal((B, Hkv, S, D)).astype(dt)
        got = st.eval([q, k, v]).to_numpy()
        ok.push(k), ov.push(v)
        kf.append(k), vf.append(v)
        assert (st.k.len(), st.k.cursor()) == (ok.len(), ok.cursor())
        if fmt is None:
            assert st.k.valid_view().tobytes() == ok.valid_view().tobytes()
            want = orc.flash_sdpa(q, ok.valid_view(), ov.valid_view(), threads=8)
            assert max_abs(got, want) <= tol, step
        n = ok.len()
        last = cases.textbook_sdpa(q, np.concatenate(kf, 2)[:, :, -n:], np.concatenate(vf, 2)[:, :, -n:])
        assert max_abs(got, last) <= (tol if fmt is None else 6e-2), step


def test_window_state_freeze_is_a_deep_copy(rt):
    rng = np.random.default_rng(2)
    st = tract_amd.WindowKvSdpa(axis=2, window=4).state()
    mk = lambda: rng.standard_normal((1, 2, 1, 32)).astype(np.float32)  # noqa: E731
    for _ in range(6):
        st.eval([mk(), mk(), mk()])
    fr = st.freeze()
    before = fr.k.valid_view().copy()
    st.eval([mk(), mk(), mk()])
    assert fr.k.valid_view().tobytes() == before.tobytes() and fr.k.cursor() == 2 and st.k.cursor() == 3
    q, k, v = mk(), mk(), mk()
    a = fr.unfreeze().eval([q, k, v]).to_numpy()
    b = fr.eval([q, k, v]).to_numpy()
    assert a.tobytes() == b.tobytes()
