"""Q8_0 / Q4_0 quantisation on append: stored blocks must be bit-identical to the
oracle's (tract's CPU block quantisers), for f16 and f32 sources, including outlier
channels, ties, zeros, denormal-range scales and special values."""
import numpy as np
import pytest

import tract_amd
from oracle import oracle as orc
from tests import cases
from tests.gpu_util import rt  # noqa: F401

pytestmark = pytest.mark.gpu

FMTS = [(tract_amd.Q8_0, orc.FMT_Q8_0, tract_amd.Q8_0_FORMAT), (tract_amd.Q4_0, orc.FMT_Q4_0, tract_amd.Q4_0_FORMAT)]


def _nasty(rng, n_blocks, dt):
    x = rng.standard_normal((n_blocks, 32)).astype(np.float32)
    x *= rng.choice([1e-7, 1e-4, 1.0, 20.0, 3000.0], size=(n_blocks, 1)).astype(np.float32)
    x[0] = 0
    x[1, :] = 1.0            # all ties
    x[2, 0], x[2, 1] = -3.0, 3.0  # tie on |v|: first wins
    x[3, 5] = np.nan
    x[4, 7] = np.inf
    x[5, :] = np.float32(6e-8)  # f16 subnormal scale range
    x[6] = np.arange(32) - 16
    x[7] = -(np.arange(32) - 15.5)
    # equal magnitudes of both signs: the first element decides the sign of the scale
    x[8, 0], x[8, 1] = 3.0, -3.0
    x[9] = -0.0
    x[10] = np.nan
    x[11, 3], x[11, 9] = np.inf, -np.inf
    x[12, 3], x[12, 9] = -np.inf, np.inf
    m = np.abs(x[13]).max()
    x[13, 31] = -m if x[13][np.abs(x[13]).argmax()] > 0 else m
    x[14, 20], x[14, 2] = -5000.0, 5000.0
    x[15, 0], x[15, 4], x[15, 9] = np.nan, -7000.0, 7000.0
    x[16, 1:] = np.nan                                   # one number among NaN
    x[17, :] = -2.5
    x[18, 0], x[18, 1], x[18, 2] = 1.0, 900.0, 3.0          # a signalling NaN beside the block's largest value:
    x.view(np.uint32)[18, 3] = 0x7FA00000                     # ignored like any NaN, and it must not take its neighbours along
    x[19, 5], x[19, 6], x[19, 7] = -700.0, 2.0, 1.0
    x.view(np.uint32)[19, 4] = 0xFFA00001
    return x.astype(dt)


@pytest.mark.parametrize("dt", [np.float32, np.float16])
@pytest.mark.parametrize("dev_fmt,orc_fmt,bq", FMTS)
def test_block_quant_op_bit_exact(rt, dt, dev_fmt, orc_fmt, bq):
    rng = np.random.default_rng(10)
    with np.errstate(over="ignore", invalid="ignore"):
        x = _nasty(rng, 4096, dt)
    got = bq.quant_f16(x) if dt == np.float16 else bq.quant_f32(x)
    want = orc.quant(orc_fmt, x).reshape(-1)
    bb = bq.block_bytes()
    bad = np.nonzero((got.reshape(-1, bb) != want.reshape(-1, bb)).any(axis=1))[0]
    assert bad.size == 0, f"blocks differ: {bad[:10]}"
    # dequantisation in both output types is bit-exact too
    for odt, fn in ((np.float32, bq.dequant_f32), (np.float16, bq.dequant_f16)):
        g, w = fn(want), orc.dequant(orc_fmt, want, odt).reshape(-1)
        ok = (g.view(np.uint16 if odt == np.float16 else np.uint32) == w.view(np.uint16 if odt == np.float16 else np.uint32)) | (np.isnan(g) & np.isnan(w))
        assert ok.all()


@pytest.mark.parametrize("dt", [np.float32, np.float16])
@pytest.mark.parametrize("dev_fmt,orc_fmt,bq", FMTS)
def test_simulate_precision_loss_bit_exact(rt, dt, dev_fmt, orc_fmt, bq):
    """BlockQuant::simulate_precision_loss (block_quant/mod.rs:130-154): one pass on the device gives the bits of
    quantising and dequantising in the tensor's own type, on a rank-3 tensor blocked along its last axis."""
    rng = np.random.default_rng(12)
    with np.errstate(over="ignore", invalid="ignore"):
        x = _nasty(rng, 6 * 50 * 4, dt).reshape(6, 50, 128)
        got = bq.simulate_precision_loss(x, 2)
        want = orc.simulate_precision_loss(orc_fmt, x)
    assert got.shape == x.shape and got.dtype == x.dtype
    u = np.uint16 if dt == np.float16 else np.uint32
    ok = (got.view(u) == want.view(u)) | (np.isnan(got) & np.isnan(want))
    assert ok.all(), np.argwhere(~ok)[:5]
    # the reference's own round trips (q4_0.rs:505-535): small integers survive Q4_0 exactly
    if dev_fmt == tract_amd.Q4_0:
        for head in ([1, 2, 3, 4], [-1, -2, -3, -4], [1234], [-1234]):
            y = np.zeros((1, 32), dtype=dt)
            y[0, : len(head)] = head
            assert np.array_equal(bq.simulate_precision_loss(y, 1), y)
    with pytest.raises(tract_amd.TractRocmError):
        bq.simulate_precision_loss(x, 1)                      # blocks run along the last axis only
    with pytest.raises(tract_amd.TractRocmError):
        bq.simulate_precision_loss(x[:, :, :48], 2)           # 48 is not a multiple of the block length


@pytest.mark.parametrize("dt", [np.float32, np.float16])
@pytest.mark.parametrize("dev_fmt,orc_fmt,bq", FMTS)
def test_quantised_cache_append_bit_exact(rt, dt, dev_fmt, orc_fmt, bq):
    """cfg4 shape (reduced): GQA [B,8,T,128], 1% outlier channels x20, appended in chunks
    with growth; export must equal quant(concat(chunks))."""
    B, H, D = 2, 8, 128
    rng = np.random.default_rng(cases.cfg_seed(4, "chan"))
    chan = rng.choice(H * D, size=10, replace=False)
    lens = [40, 1, 1, 17, 1, 64, 1]
    chunks = []
    for i, n in enumerate(lens):
        x = cases.seeded_normal(cases.cfg_seed(4, "k") + i, (B, H, n, D))
        xf = x.transpose(0, 2, 1, 3).reshape(B, n, H * D).copy()
        xf[:, :, chan] *= 20
        chunks.append(xf.reshape(B, n, H, D).transpose(0, 2, 1, 3).astype(dt))
    cache = tract_amd.InPlaceKvCache(2, storage_format=dev_fmt)
    ref = orc.InPlaceKvCache(2)
    for i, ch in enumerate(chunks):
        cache.push(ch)
        ref.push(orc.quant(orc_fmt, ch))  # the reference cache of canonical block rows
        assert (cache.len(), cache.capacity(), cache.reallocs()) == (ref.len(), ref.capacity(), ref.reallocs())
        got = cache.valid_contiguous()
        want = orc.quant(orc_fmt, np.concatenate(chunks[: i + 1], axis=2))
        assert got.shape == want.shape and got.tobytes() == want.tobytes()
        assert got.tobytes() == ref.valid_contiguous().tobytes()
    # truncate + clone keep the bytes
    cl = cache.clone()
    cache.truncate(50)
    assert cache.valid_contiguous().tobytes() == want[:, :, :50].tobytes()
    assert cl.valid_contiguous().tobytes() == want.tobytes()


def test_quantised_cache_strided_f16_source(rt):
    rng = np.random.default_rng(12)
    B, S, H, D = 2, 6, 4, 64
    x = rng.standard_normal((B, S, H, D)).astype(np.float16)
    t = tract_amd.DeviceTensor.from_numpy(x)
    view = tract_amd.DeviceTensor((B, H, S, D), np.float16, ptr=t.ptr.value, owner=t)
    for dev_fmt, orc_fmt, _ in FMTS:
        cache = tract_amd.InPlaceKvCache(2, storage_format=dev_fmt)
        cache.push(view, strides=(S * H * D, D, H * D, 1))
        want = orc.quant(orc_fmt, np.ascontiguousarray(x.transpose(0, 2, 1, 3)))
        assert cache.valid_contiguous().tobytes() == want.tobytes()


def test_quant_rejects_bad_head_dim(rt):
    c = tract_amd.InPlaceKvCache(2, storage_format=tract_amd.Q4_0)
    with pytest.raises(tract_amd.TractRocmError, match="head_dim"):
        c.push(np.zeros((1, 1, 2, 48), np.float16))
