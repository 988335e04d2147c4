"""In-place KV cache on the GPU vs the oracle and vs numpy.concatenate — bit-exact.
Mirrors the reference's tests: inplace_kv_cache.rs:366-418 (concat equivalence, O(log T)
reallocs), dyn_kv_cache.rs:499-527, freeze/save/load :898-942, truncate :112-119."""
import numpy as np
import pytest

import tract_amd
from oracle import oracle as orc
from tests.gpu_util import rt  # noqa: F401

pytestmark = pytest.mark.gpu


def _chunks(rng, shape, axis, lens, dt):
    out = []
    for n in lens:
        s = list(shape)
        s[axis] = n
        out.append((rng.standard_normal(s) * 4).astype(dt))
    return out


@pytest.mark.parametrize("dt", [np.float32, np.float16])
@pytest.mark.parametrize("shape,axis", [((1, 4, 0, 8), 2), ((2, 3, 0, 16), 2), ((2, 0, 5), 1), ((1, 32, 0, 64), 2),
                                        ((3, 8, 0, 128), 2)])
def test_push_matches_concat_and_oracle(rt, dt, shape, axis):
    rng = np.random.default_rng(0)
    lens = [3, 1, 1, 0, 7, 1, 2, 30, 1, 64]
    chunks = _chunks(rng, shape, axis, lens, dt)
    dev, ref = tract_amd.InPlaceKvCache(axis), orc.InPlaceKvCache(axis)
    for i, ch in enumerate(chunks):
        dev.push(ch)
        ref.push(ch)
        assert (dev.len(), dev.capacity(), dev.reallocs()) == (ref.len(), ref.capacity(), ref.reallocs())
        if dev.len():
            got = dev.valid_contiguous()
            assert got.tobytes() == ref.valid_contiguous().tobytes()
            assert got.tobytes() == np.concatenate(chunks[: i + 1], axis=axis).tobytes()


def test_single_token_decode_growth(rt):
    # cfg1 shape: [1,32,1,64] f32 grown token by token 0 -> 256
    rng = np.random.default_rng(1)
    dev, ref = tract_amd.InPlaceKvCache(2), orc.InPlaceKvCache(2)
    toks = rng.standard_normal((256, 1, 32, 1, 64)).astype(np.float32)
    for t in range(256):
        dev.push(toks[t])
        ref.push(toks[t])
        assert (dev.len(), dev.capacity(), dev.reallocs()) == (ref.len(), ref.capacity(), ref.reallocs())
    assert dev.reallocs() == 8 and dev.capacity() == 256
    assert dev.valid_contiguous().tobytes() == np.concatenate(list(toks), axis=2).tobytes()


def test_strided_source_view(rt):
    # K projected as [B,S,H,D] and viewed as [B,H,S,D] (a fused Move axis op)
    rng = np.random.default_rng(2)
    B, S, H, D = 2, 5, 4, 32
    for dt in (np.float16, np.float32):
        x = rng.standard_normal((B, S, H, D)).astype(dt)
        dev = tract_amd.InPlaceKvCache(2)
        t = tract_amd.DeviceTensor.from_numpy(x)
        view = tract_amd.DeviceTensor((B, H, S, D), dt, ptr=t.ptr.value, owner=t)
        dev.push(view, strides=(S * H * D, D, H * D, 1))
        dev.push(view, strides=(S * H * D, D, H * D, 1))
        want = np.concatenate([x.transpose(0, 2, 1, 3)] * 2, axis=2)
        assert dev.valid_contiguous().tobytes() == np.ascontiguousarray(want).tobytes()


def test_reserve_then_append_in_place(rt):
    rng = np.random.default_rng(3)
    x = rng.standard_normal((2, 2, 100, 64)).astype(np.float16)
    dev = tract_amd.InPlaceKvCache(2)
    dev.reserve(512, like=(x.shape, x.dtype))
    assert dev.capacity() == 512 and dev.len() == 0
    dev.push(x)
    for t in range(50):
        dev.push(x[:, :, t:t + 1])
    assert dev.capacity() == 512 and dev.reallocs() == 0 and dev.len() == 150
    assert dev.valid_contiguous().tobytes() == np.concatenate([x, x[:, :, :50]], axis=2).tobytes()


def test_truncate_clone_save_load(rt):
    rng = np.random.default_rng(4)
    x = rng.standard_normal((1, 2, 20, 32)).astype(np.float32)
    st = tract_amd.DynKeyValueCache("k", 2).state()
    with pytest.raises(tract_amd.TractRocmError, match="zero-len"):
        st.truncate(0)
    with pytest.raises(tract_amd.TractRocmError, match="never initialized"):
        st.save_to([])
    st.eval(x)
    assert st.resolve_symbols() == 20
    frozen = st.freeze()
    st.truncate(7)
    assert st.resolve_symbols() == 7
    saved = []
    st.save_to(saved)
    assert saved[0].tobytes() == x[:, :, :7].tobytes()
    with pytest.raises(tract_amd.TractRocmError):
        st.truncate(8)
    st.eval(x[:, :, :3])  # appends after the rollback point
    assert st.kv_cache.valid_contiguous().tobytes() == np.concatenate([x[:, :, :7], x[:, :, :3]], axis=2).tobytes()
    # the frozen copy is independent
    assert frozen.kv_cache.valid_contiguous().tobytes() == x.tobytes()
    st2 = tract_amd.DynKeyValueCache("k", 2).state()
    st2.load_from(saved)
    assert st2.resolve_symbols() == 7 and st2.kv_cache.valid_contiguous().tobytes() == saved[0].tobytes()


def test_error_paths(rt):
    c = tract_amd.InPlaceKvCache(2)
    c.push(np.zeros((1, 2, 3, 8), np.float32))
    with pytest.raises(tract_amd.TractRocmError, match="rank mismatch"):
        c.push(np.zeros((1, 3, 8), np.float32))
    with pytest.raises(tract_amd.TractRocmError, match="does not match"):
        c.push(np.zeros((1, 2, 3, 8), np.float16))
    with pytest.raises(tract_amd.TractRocmError):
        tract_amd.InPlaceKvCache(1).push(np.zeros((1, 2, 3, 8), np.float32))


def test_copy_nd_general(rt):
    """DeviceContext::copy_nd: arbitrary strides, ranks 1..6, all element sizes."""
    import ctypes as C
    from tract_amd._lib import call
    rng = np.random.default_rng(5)
    for es, dt in ((1, np.uint8), (2, np.uint16), (4, np.uint32), (8, np.uint64)):
        src = rng.integers(0, 255, size=(3, 4, 5, 6, 2, 2)).astype(dt)
        # transpose + slice expressed through strides
        view = src.transpose(2, 0, 5, 1, 4, 3)[1:, :, :, 1:3]
        shape = view.shape
        sst = [s // es for s in view.strides]
        off = view.__array_interface__["data"][0] - src.__array_interface__["data"][0]
        d_src = tract_amd.DeviceTensor.from_numpy(src)
        d_dst = tract_amd.DeviceTensor(shape, dt)
        dst_strides = d_dst.strides()
        I = C.c_int64 * 6
        call("trocm_copy_nd", d_dst.ptr, 0, I(*dst_strides), d_src.ptr, off, I(*sst), I(*shape), 6, es, None)
        assert np.array_equal(d_dst.to_numpy(), view)
    # broadcast source (stride 0) and rank 1
    src = np.arange(7, dtype=np.float32)
    d_src = tract_amd.DeviceTensor.from_numpy(src)
    d_dst = tract_amd.DeviceTensor((4, 7), np.float32)
    I2 = C.c_int64 * 2
    call("trocm_copy_nd", d_dst.ptr, 0, I2(7, 1), d_src.ptr, 0, I2(0, 1), I2(4, 7), 2, 4, None)
    assert np.array_equal(d_dst.to_numpy(), np.broadcast_to(src, (4, 7)))


def test_pool_backed_caches_share_one_allocation(rt):
    """cfg5's memory arrangement: per-sequence capacity-doubling caches carved from one device
    allocation; growth exchanges planes inside the pool; exhaustion is an error, not a fault."""
    rng = np.random.default_rng(6)
    H, D = 2, 64
    pool = tract_amd.KvPool(4 << 20)
    base, total = pool.stats()["base"], pool.stats()["bytes_total"]
    caches, refs = [], []
    for i in range(6):
        c, r = tract_amd.InPlaceKvCache(2, pool=pool), orc.InPlaceKvCache(2)
        x = rng.standard_normal((1, H, 3 + 5 * i, D)).astype(np.float16)
        c.push(x), r.push(x)
        caches.append(c), refs.append(r)
    for step in range(70):  # single-token growth: every cache doubles several times inside the pool
        for c, r in zip(caches, refs):
            x = rng.standard_normal((1, H, 1, D)).astype(np.float16)
            c.push(x), r.push(x)
    for c, r in zip(caches, refs):
        assert (c.len(), c.capacity(), c.reallocs()) == (r.len(), r.capacity(), r.reallocs())
        assert c.valid_contiguous().tobytes() == r.valid_contiguous().tobytes()
        ptr, _, cap = c.raw()
        assert base <= ptr and ptr + H * cap * D * 2 <= base + total
    used = pool.stats()["bytes_in_use"]
    assert used >= sum(H * c.capacity() * D * 2 for c in caches)
    # a quantised cache in the same pool
    qc = tract_amd.InPlaceKvCache(2, storage_format=tract_amd.Q4_0, pool=pool)
    x = rng.standard_normal((1, H, 40, D)).astype(np.float16)
    qc.push(x)
    assert qc.valid_contiguous().tobytes() == orc.quant(orc.FMT_Q4_0, x).tobytes()
    # exhaustion
    big = tract_amd.InPlaceKvCache(2, pool=pool)
    with pytest.raises(tract_amd.TractRocmError, match="pool exhausted"):
        big.push(np.zeros((1, H, 40000, D), np.float16))
    with pytest.raises(tract_amd.TractRocmError, match="live caches"):
        pool.close()
    for c in caches + [qc, big]:
        c.close()
    assert pool.stats()["bytes_in_use"] == 0 and pool.stats()["largest_free"] == total
    pool.close()
