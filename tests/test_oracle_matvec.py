"""Pins for the oracle's Q4_0 matrix-vector product (GgmlGemm's m <= 8 arm as the reference's own
test defines it, cuda/src/kernels/matmul/mod.rs:864-890: activations times the weights after
Q4_0.simulate_precision_loss).  The block (de)quantisers it builds on are pinned in
test_oracle_quant.py; here: a closed form on hand-built blocks, numpy's f64 product with the
dequantised weights, batch broadcasting, linearity."""
import numpy as np
import pytest

from oracle import oracle as orc

Q4 = 3


def hand_blocks(n, k, scale_of_row):
    """Row j: every block has scale scale_of_row(j) and nibbles i % 16 in ggml order (element i of the
    block has code i % 16, the table of q4_0.rs:722-739), so dequantised element i = (i % 16 - 8) * d."""
    nb = k // 32
    out = np.zeros((1, n, nb * 18), np.uint8)
    codes = np.arange(32) % 16
    packed = (codes[:16] | (codes[16:] << 4)).astype(np.uint8)
    for j in range(n):
        d = np.array([scale_of_row(j)], np.float16).view(np.uint8)
        for b in range(nb):
            out[0, j, b * 18:b * 18 + 2] = d
            out[0, j, b * 18 + 2:b * 18 + 18] = packed
    return out


def test_closed_form_on_hand_built_blocks():
    n, k = 4, 96
    blocks = hand_blocks(n, k, lambda j: [0.5, 0.25, 1.0, 2.0][j])
    ones = np.ones((1, 1, k), np.float32)
    # sum over a block of (i % 16 - 8) = 2 * (0 + ... + 15 - 128) = -16; three blocks per row
    want = np.array([0.5, 0.25, 1.0, 2.0], np.float32) * (-16.0) * 3
    assert np.array_equal(orc.q4_0_matvec(blocks, ones)[0, 0], want)
    # a one-hot activation picks one dequantised weight: element 37 = block 1, index 5 -> (5 - 8) * d
    e = np.zeros((1, 1, k), np.float32)
    e[0, 0, 37] = 1.0
    assert np.array_equal(orc.q4_0_matvec(blocks, e)[0, 0], np.array([0.5, 0.25, 1.0, 2.0], np.float32) * -3.0)
    # ... and index 21 of a block is a HIGH nibble (elements 16..31): (21 % 16 - 8) = -3 as well; 16 -> -8
    e[:] = 0
    e[0, 0, 16] = 1.0
    assert np.array_equal(orc.q4_0_matvec(blocks, e)[0, 0], np.array([0.5, 0.25, 1.0, 2.0], np.float32) * -8.0)


@pytest.mark.parametrize("dt", [np.float32, np.float16])
@pytest.mark.parametrize("wb,ab,m,n,k", [(1, 1, 1, 7, 64), (1, 3, 2, 5, 128), (2, 4, 8, 3, 96), (2, 2, 5, 9, 32)])
def test_equals_numpy_product_with_dequantised_weights(dt, wb, ab, m, n, k):
    rng = np.random.default_rng(n * k)
    w = rng.standard_normal((wb, n, k)).astype(dt)
    act = rng.standard_normal((ab, m, k)).astype(dt)
    blocks = orc.quant(Q4, w)
    wd = orc.dequant(Q4, blocks, dt).astype(np.float64)
    want = np.einsum("bmk,bnk->bmn", act.astype(np.float64), np.repeat(wd, ab // wb, axis=0))
    got = orc.q4_0_matvec(blocks, act)
    assert got.dtype == dt and got.shape == (ab, m, n)
    tol = 1e-5 if dt == np.float32 else 2e-3
    assert np.max(np.abs(got.astype(np.float64) - want) / (1 + np.abs(want))) <= tol


def test_weight_batch_is_shared_by_consecutive_activation_batches():
    rng = np.random.default_rng(3)
    w = rng.standard_normal((2, 4, 64)).astype(np.float32)
    act = rng.standard_normal((4, 1, 64)).astype(np.float32)
    blocks = orc.quant(Q4, w)
    got = orc.q4_0_matvec(blocks, act)
    for b in range(4):   # batch_ratio = act_batch / w_batch (mod.rs:502): activations 0,1 -> weights 0; 2,3 -> 1
        assert np.array_equal(got[b:b + 1], orc.q4_0_matvec(blocks[b // 2:b // 2 + 1], act[b:b + 1]))


def test_linearity_in_the_activations():
    rng = np.random.default_rng(4)
    blocks = orc.quant(Q4, rng.standard_normal((1, 6, 128)).astype(np.float32))
    a = rng.integers(-4, 5, (1, 1, 128)).astype(np.float32)
    b = rng.integers(-4, 5, (1, 1, 128)).astype(np.float32)
    lhs = orc.q4_0_matvec(blocks, a + 2 * b)
    rhs = orc.q4_0_matvec(blocks, a) + 2 * orc.q4_0_matvec(blocks, b)
    assert np.max(np.abs(lhs - rhs)) <= 1e-4
