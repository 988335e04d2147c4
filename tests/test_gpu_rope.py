"""ApplyRope / RotateHalf / Cast on the GPU vs the oracle: bit-exact (each is a fixed sequence of
correctly rounded IEEE operations)."""
import numpy as np
import pytest

import tract_amd
from oracle import oracle as orc
from tests.gpu_util import rt  # noqa: F401

pytestmark = pytest.mark.gpu


def _tables(shape, dt):
    m = int(np.prod(shape))
    return (np.cos(np.arange(m, dtype=np.float32)).reshape(shape).astype(dt),
            np.sin(np.arange(m, dtype=np.float32)).reshape(shape).astype(dt))


# the shapes of the reference's GPU test (cuda/src/kernels/nn/apply_rope.rs:200-209), cos/sin of the input's shape
@pytest.mark.parametrize("shape", [(2, 1, 2, 2), (2, 4, 4), (2, 1, 512, 10), (8, 8), (1, 10, 512, 24), (3, 10, 512, 24)])
@pytest.mark.parametrize("dt", [np.float32, np.float16])
def test_apply_rope_reference_cases(rt, shape, dt):
    n = int(np.prod(shape))
    x = (np.arange(n, dtype=np.float32) / np.float32(1000.0)).reshape(shape).astype(dt)
    cos, sin = _tables(shape, dt)
    got = tract_amd.ApplyRope().eval(x, cos, sin).to_numpy()
    want = orc.apply_rope(x, cos, sin)
    assert got.dtype == dt and got.tobytes() == want.tobytes()


@pytest.mark.parametrize("shape,cs_shape", [((8, 32, 1, 128), (8, 1, 1, 128)), ((1, 32, 512, 128), (512, 128)),
                                            ((2, 8, 77, 64), (1, 1, 77, 64)), ((4, 6, 128), (6, 128)),
                                            ((3, 5, 7, 2), (3, 1, 7, 2))])
@pytest.mark.parametrize("dt", [np.float32, np.float16])
def test_apply_rope_broadcast_tables(rt, shape, cs_shape, dt):
    """The LLM layouts: Q/K [B,H,S,D] against per-position tables [S,D] (prefill) or per-sequence
    positions [B,1,1,D] (one decode token each)."""
    rng = np.random.default_rng(sum(shape))
    x = rng.standard_normal(shape).astype(dt)
    ang = rng.uniform(-7, 7, cs_shape)
    cos, sin = np.cos(ang).astype(dt), np.sin(ang).astype(dt)
    got = tract_amd.ApplyRope().eval(x, cos, sin).to_numpy()
    assert got.tobytes() == orc.apply_rope(x, cos, sin).tobytes()


@pytest.mark.parametrize("shape", [(2, 2), (512, 512), (10, 512, 1024), (6,), (2, 3, 4, 10)])
@pytest.mark.parametrize("dt", [np.float32, np.float16])
def test_rotate_half(rt, shape, dt):
    # apply_rope.rs:270-277 shapes; RotateHalf twice == negation
    n = int(np.prod(shape))
    x = (np.arange(n, dtype=np.float32) % 2048).reshape(shape).astype(dt)
    op = tract_amd.RotateHalf()
    once = op.eval(x)
    assert once.to_numpy().tobytes() == orc.rotate_half(x).tobytes()
    assert np.array_equal(-op.eval(once).to_numpy(), x)


def test_rope_errors(rt):
    with pytest.raises(tract_amd.TractRocmError, match="divisible by 2"):
        tract_amd.RotateHalf().eval(np.zeros((2, 3), np.float32))
    with pytest.raises(tract_amd.TractRocmError, match="same shape"):
        tract_amd.ApplyRope().eval(np.zeros((2, 4), np.float32), np.zeros((2, 4), np.float32), np.zeros((1, 4), np.float32))
    with pytest.raises(tract_amd.TractRocmError, match="rank"):
        tract_amd.ApplyRope().eval(np.zeros((4,), np.float32), np.zeros((4,), np.float32), np.zeros((4,), np.float32))


@pytest.mark.parametrize("n", [0, 1, 5, 12, 4096, 1000003])
def test_cast_f32_f16_round_trip(rt, n):
    # cuda/src/kernels/array/cast.rs:111-131: f as f32 / 2 values; plus random values incl. subnormals and ties
    rng = np.random.default_rng(n)
    x = np.concatenate([np.arange(n // 2, dtype=np.float32) / 2, (rng.standard_normal(n - n // 2) * 10.0 ** rng.integers(-9, 5, n - n // 2)).astype(np.float32)])
    h = tract_amd.Cast(np.float16).eval(x)
    assert h.to_numpy().view(np.uint16).tobytes() == orc.f32_to_f16_bits(x).tobytes()
    back = tract_amd.Cast(np.float32).eval(h).to_numpy()
    assert back.tobytes() == orc.f16_bits_to_f32(orc.f32_to_f16_bits(x)).tobytes()
    same = tract_amd.Cast(np.float32).eval(x).to_numpy()
    assert same.tobytes() == x.tobytes()


def test_rope_then_cache_then_attention_matches_oracle(rt):
    """The layer order of an exported decoder: RoPE on Q and K_new, then the fused cache + attention."""
    rng = np.random.default_rng(11)
    B, Hq, Hkv, D, T0 = 2, 8, 2, 128, 70
    freq = 1.0 / (10000.0 ** (np.arange(D // 2) / (D // 2)))

    def tables(pos):
        a = np.outer(pos, freq)
        a = np.concatenate([a, a], -1)
        return np.cos(a).astype(np.float16), np.sin(a).astype(np.float16)

    st = tract_amd.InPlaceKvSdpa(axis=2, causal=True).state()
    rope = tract_amd.ApplyRope()
    ks, vs = [], []
    pos = 0
    for S in (T0, 1, 1, 1):
        q = (rng.standard_normal((B, Hq, S, D)) / np.sqrt(D)).astype(np.float16)
        k = rng.standard_normal((B, Hkv, S, D)).astype(np.float16)
        v = rng.standard_normal((B, Hkv, S, D)).astype(np.float16)
        c, s = tables(np.arange(pos, pos + S))
        qr, kr = rope.eval(q, c, s), rope.eval(k, c, s)
        out = st.eval([qr, kr, tract_amd.DeviceTensor.from_numpy(v)]).to_numpy()
        ks.append(orc.apply_rope(k, c, s))
        vs.append(v)
        want = orc.flash_sdpa(orc.apply_rope(q, c, s), np.concatenate(ks, 2), np.concatenate(vs, 2), causal=True)
        assert np.abs(out.astype(np.float32) - want.astype(np.float32)).max() <= 2e-2
        pos += S
    assert st.k.valid_contiguous().tobytes() == np.concatenate(ks, 2).tobytes()
