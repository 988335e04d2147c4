"""Pins for the oracle's RotateHalf / ApplyRope (transformers/src/ops/apply_rope.rs).

Each check is independent of the C restatement's formula: the reference's own unit test
(RotateHalf twice is a negation), numpy's concatenate form, and the rotation's closed forms
(a pair keeps its norm; rotating by a then b equals rotating by a + b)."""
import numpy as np
import pytest

from oracle import oracle as orc


@pytest.mark.parametrize("shape", [(2, 2), (512, 512), (10, 64, 128)])
def test_rotate_half_twice_is_negation(shape):
    # apply_rope.rs:257-277 (run_test_case): RotateHalf(RotateHalf(x)) == -x, values 0..len
    n = int(np.prod(shape))
    x = np.arange(n, dtype=np.float32).reshape(shape)
    back = orc.rotate_half(orc.rotate_half(x))
    assert np.array_equal(-back, x)


@pytest.mark.parametrize("dt", [np.float32, np.float16])
def test_rotate_half_is_concat_of_negated_upper_and_lower(dt):
    x = np.random.default_rng(0).standard_normal((3, 5, 8)).astype(dt)
    want = np.concatenate([-x[..., 4:], x[..., :4]], axis=-1)
    got = orc.rotate_half(x)
    assert got.dtype == dt and got.tobytes() == want.tobytes()
    # a dropped sign or swapped halves would pass neither of these
    assert np.array_equal(got[..., 0], -x[..., 4]) and np.array_equal(got[..., 7], x[..., 3])


@pytest.mark.parametrize("shape,cs_shape", [((2, 1, 2, 2), (2, 1, 2, 2)), ((2, 4, 4), (2, 4, 4)), ((8, 8), (8, 8)),
                                            ((1, 10, 16, 24), (16, 24)), ((3, 4, 5, 6), (1, 1, 5, 6)),
                                            ((3, 4, 5, 6), (3, 1, 5, 6))])
def test_apply_rope_f32_equals_numpy_expression_bitwise(shape, cs_shape):
    # inputs as in the reference's GPU test (cuda/src/kernels/nn/apply_rope.rs:156-170)
    n, m = int(np.prod(shape)), int(np.prod(cs_shape))
    x = (np.arange(n, dtype=np.float32) / np.float32(1000.0)).reshape(shape)
    cos = np.cos(np.arange(m, dtype=np.float32)).reshape(cs_shape)
    sin = np.sin(np.arange(m, dtype=np.float32)).reshape(cs_shape)
    h = shape[-1] // 2
    rot = np.concatenate([-x[..., h:], x[..., :h]], axis=-1)
    want = x * cos + rot * sin   # numpy f32: each operation rounded once, no fma
    assert orc.apply_rope(x, cos, sin).tobytes() == want.astype(np.float32).tobytes()


def test_apply_rope_f16_rounds_after_every_operation():
    rng = np.random.default_rng(3)
    x = rng.standard_normal((2, 3, 7, 16)).astype(np.float16)
    ang = rng.uniform(-3, 3, (7, 16)).astype(np.float32)
    cos, sin = np.cos(ang).astype(np.float16), np.sin(ang).astype(np.float16)
    rot = np.concatenate([-x[..., 8:], x[..., :8]], axis=-1)
    want = (x * cos).astype(np.float16) + (rot * sin).astype(np.float16)   # numpy float16 ops round each result
    got = orc.apply_rope(x, cos, sin)
    assert got.dtype == np.float16 and got.tobytes() == want.astype(np.float16).tobytes()
    # and it is NOT what a single rounding of the f32 expression gives everywhere
    single = (x.astype(np.float32) * cos.astype(np.float32) + rot.astype(np.float32) * sin.astype(np.float32)).astype(np.float16)
    assert (single != got).any()


def test_apply_rope_is_a_rotation_of_each_pair():
    rng = np.random.default_rng(5)
    S, D = 9, 32
    x = rng.standard_normal((2, 4, S, D)).astype(np.float32)
    freq = 1.0 / (10000.0 ** (np.arange(D // 2) / (D // 2)))

    def tables(pos):
        a = np.outer(pos, freq)
        a = np.concatenate([a, a], axis=-1)   # both halves carry the same angle
        return np.cos(a).astype(np.float32), np.sin(a).astype(np.float32)

    c1, s1 = tables(np.arange(S))
    y = orc.apply_rope(x, c1, s1)
    # pair (i, i + D/2) keeps its norm
    n_in = x[..., :D // 2] ** 2 + x[..., D // 2:] ** 2
    n_out = y[..., :D // 2] ** 2 + y[..., D // 2:] ** 2
    assert np.allclose(n_in, n_out, rtol=1e-5, atol=1e-6)
    # angles add
    c2, s2 = tables(np.arange(S) * 0.5 + 3)
    c12, s12 = tables(np.arange(S) * 1.5 + 3)
    assert np.allclose(orc.apply_rope(y, c2, s2), orc.apply_rope(x, c12, s12), rtol=1e-4, atol=1e-5)
    # position 0 is the identity
    assert np.array_equal(y[:, :, 0], x[:, :, 0])


def test_cast_is_ieee_round_to_nearest_even():
    # the oracle's conversions are pinned exhaustively elsewhere; here the two ties that tell
    # RNE from round-half-up, and the exact widening
    x = np.array([1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 65520.0, -0.0, 1e-8], dtype=np.float32)
    got = orc.f32_to_f16_bits(x).view(np.float16)
    with np.errstate(over="ignore"):
        assert got.tobytes() == x.astype(np.float16).tobytes()
    assert got[0] == np.float16(1.0) and got[1] == np.float16(1.0 + 2.0 ** -9) and np.isinf(got[2])
