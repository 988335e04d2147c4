"""save_dat / load_dat of cache states: NNEF tensor files written from device caches and loaded back,
bit-exact, quantised caches without dequantisation."""
import numpy as np
import pytest

import tract_amd
from oracle import oracle as orc
from tests.gpu_util import max_abs, rt  # noqa: F401

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dt", [np.float32, np.float16])
def test_plain_cache_round_trip(rt, dt):
    rng = np.random.default_rng(0)
    x = rng.standard_normal((2, 4, 37, 64)).astype(dt)
    c = tract_amd.InPlaceKvCache(2)
    c.push(x[:, :, :20]), c.push(x[:, :, 20:])
    data = c.save_dat()
    assert data == orc.dat_write_plain(x)                       # what tract's write_tensor would write
    d = tract_amd.InPlaceKvCache(2)
    d.load_dat(data)
    assert d.len() == 37 and d.valid_contiguous().tobytes() == x.tobytes()
    d.load_dat(data)                                            # load_dat appends
    assert d.len() == 74 and d.valid_contiguous()[:, :, 37:].tobytes() == x.tobytes()


@pytest.mark.parametrize("fmt,ofmt,item", [("q4_0", "FMT_Q4_0", 0x3040), ("q8_0", "FMT_Q8_0", 0x3081)])
def test_quantised_cache_round_trip_without_dequantising(rt, fmt, ofmt, item):
    code = {"q4_0": tract_amd.Q4_0, "q8_0": tract_amd.Q8_0}[fmt]
    rng = np.random.default_rng(3)
    B, H, T, D = 2, 3, 45, 128
    x = rng.standard_normal((B, H, T, D)).astype(np.float16)
    x[:, :, :, 5] *= 20
    c = tract_amd.InPlaceKvCache(2, storage_format=code)
    c.push(x[:, :, :7]), c.push(x[:, :, 7:])
    blocks = c.valid_contiguous()
    assert blocks.tobytes() == orc.quant(getattr(orc, ofmt), x).tobytes()
    data = c.save_dat()
    h = orc.dat_header_fields(data)
    assert h["item_type"] == item and h["item_type_vendor"] == 0x5452 and h["dims"] == (B * H * T, D)
    if fmt == "q4_0":
        assert data == orc.dat_write_block_quant(0x3040, blocks.tobytes(), (B, H, T, D))
    d = tract_amd.InPlaceKvCache(2, storage_format=code)
    d.load_dat(data, like=((B, H, 0, D), np.float16))
    assert d.len() == T and d.valid_contiguous().tobytes() == blocks.tobytes()   # same blocks: nothing was requantised
    # growth while importing, then more tokens through the ordinary quantising append
    d.load_dat(data)
    more = rng.standard_normal((B, H, 3, D)).astype(np.float16)
    d.push(more)
    got = d.valid_contiguous()
    assert d.len() == 2 * T + 3 and d.reallocs() >= 1
    assert got[:, :, T:2 * T].tobytes() == blocks.tobytes()
    assert got[:, :, 2 * T:].tobytes() == orc.quant(getattr(orc, ofmt), more).tobytes()


def test_attention_state_reload_gives_identical_outputs(rt):
    rng = np.random.default_rng(5)
    B, Hq, Hkv, D = 1, 8, 2, 128
    st = tract_amd.InPlaceKvSdpa(axis=2, causal=True, storage_format=tract_amd.Q8_0).state()
    k = rng.standard_normal((B, Hkv, 300, D)).astype(np.float16)
    v = rng.standard_normal((B, Hkv, 300, D)).astype(np.float16)
    q = (rng.standard_normal((B, Hq, 300, D)) / np.sqrt(D)).astype(np.float16)
    st.eval([q, k, v])
    files = [st.k.save_dat(), st.v.save_dat()]
    st2 = tract_amd.InPlaceKvSdpa(axis=2, causal=True, storage_format=tract_amd.Q8_0).state()
    st2.k.load_dat(files[0], like=(k.shape, k.dtype)), st2.v.load_dat(files[1], like=(v.shape, v.dtype))
    q1 = (rng.standard_normal((B, Hq, 1, D)) / np.sqrt(D)).astype(np.float16)
    k1 = rng.standard_normal((B, Hkv, 1, D)).astype(np.float16)
    a = st.eval([q1, k1, k1]).to_numpy()
    b = st2.eval([q1, k1, k1]).to_numpy()
    assert a.tobytes() == b.tobytes()


def test_import_refusals(rt):
    c = tract_amd.InPlaceKvCache(2)
    c.push(np.zeros((1, 1, 2, 32), np.float32))
    q = tract_amd.InPlaceKvCache(2, storage_format=tract_amd.Q4_0)
    q.push(np.zeros((1, 1, 2, 32), np.float32))
    with pytest.raises(tract_amd.TractRocmError, match="differs from the cache"):
        tract_amd.InPlaceKvCache(2, storage_format=tract_amd.Q8_0).load_dat(q.save_dat(), like=((1, 1, 0, 32), np.float32))
    with pytest.raises(tract_amd.TractRocmError, match="needs `like"):
        tract_amd.InPlaceKvCache(2, storage_format=tract_amd.Q4_0).load_dat(q.save_dat())
    with pytest.raises(tract_amd.TractRocmError, match="plain"):
        from tract_amd._lib import call
        call("trocm_kv_import_blocks", c.handle, tract_amd.DeviceTensor.from_numpy(np.zeros(18, np.uint8)).ptr, 1, None)
