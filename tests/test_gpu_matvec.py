"""Q4_0 weights x a few activation rows on the GPU (the matrix-vector arm of GgmlGemm,
cuda/src/kernels/matmul/mod.rs:575-627) vs the oracle and the f64 product with the dequantised
weights.  Tolerance: relative to 1 + |reference|, 1e-4 for f32 and 4e-3 for f16 activations (the
reference's own test allows Approximation::VeryApproximate, mod.rs:776-786)."""
import ctypes as C

import numpy as np
import pytest

import tract_amd
from oracle import oracle as orc
from tests.gpu_util import rt  # noqa: F401

pytestmark = pytest.mark.gpu
Q4 = 3


def rel_err(got, want):
    return float(np.max(np.abs(got.astype(np.float64) - want) / (1 + np.abs(want))))


def f64_product(blocks, act, dt):
    wd = orc.dequant(Q4, blocks, dt).astype(np.float64)
    return np.einsum("bmk,bnk->bmn", act.astype(np.float64), np.repeat(wd, act.shape[0] // wd.shape[0], axis=0))


# (b, m, k, n) of the reference's matrix-vector cases (mod.rs:709-724, with k rounded up to whole
# blocks) plus decoder shapes: ragged n, k that is not a multiple of 64 blocks, k beyond one LDS chunk
@pytest.mark.parametrize("dt", [np.float32, np.float16])
@pytest.mark.parametrize("wb,ab,m,n,k", [
    (1, 1, 1, 1, 32), (2, 2, 1, 2, 64), (2, 2, 2, 7, 128), (1, 4, 1, 1, 64), (1, 1, 5, 1, 32), (1, 2, 8, 2, 64),
    (1, 1, 1, 4096, 4096), (1, 1, 1, 1000, 2080), (1, 1, 3, 515, 4096), (1, 2, 4, 130, 1024), (1, 1, 6, 77, 2048),
    (1, 1, 7, 33, 992), (1, 1, 8, 200, 8192), (1, 1, 1, 64, 20480), (2, 4, 2, 50, 14336),
    (1, 1, 9, 40, 128), (1, 2, 21, 70, 256), (2, 2, 64, 33, 512),   # more than 8 rows: the matrix-matrix arm (f16) / groups of 8
    (1, 1, 9, 40, 96), (2, 4, 9, 129, 128), (1, 2, 130, 300, 1024), (1, 1, 257, 131, 2048), (1, 1, 512, 1024, 4096),
    (1, 1, 300, 14336, 256), (2, 2, 129, 8250, 128),   # enough 128 x 128 tiles for every compute unit (the shapes above run 128 x 64 tiles)
    # 4..16 f16 rows against 16 weight rows per matrix instruction: one staged chunk (2 and 4 sets of waves per
    # workgroup, more than 64 KB of LDS), k beyond one chunk, ragged n, batches that share weights
    (1, 1, 5, 2050, 256), (1, 1, 8, 2048, 4096), (1, 1, 6, 2100, 8320), (1, 1, 4, 12300, 128), (1, 1, 7, 12290, 384),
    (1, 1, 16, 40, 384), (2, 4, 12, 70, 256), (1, 1, 4, 2064, 512), (1, 2, 9, 129, 1024), (1, 1, 13, 3000, 2176), (1, 1, 16, 2049, 4096),
])
def test_matvec_matches_the_oracle(rt, dt, wb, ab, m, n, k):
    rng = np.random.default_rng(n + k + m)
    w = (rng.standard_normal((wb, n, k)) * 0.05).astype(np.float32)
    w[:, :, ::97] *= 8.0    # outliers: blocks with very different scales
    act = rng.standard_normal((ab, m, k)).astype(dt)
    blocks = orc.quant(Q4, w)
    wq = tract_amd.Q40Weights(blocks, wb, n, k)
    got = tract_amd.GgmlGemm().eval(act, wq).to_numpy()
    assert got.dtype == dt and got.shape == (ab, m, n)
    tol = 1e-4 if dt == np.float32 else 4e-3
    assert rel_err(got, f64_product(blocks, act, dt)) <= tol
    if n * k * ab * m <= 1 << 24:
        assert rel_err(got, orc.q4_0_matvec(blocks, act).astype(np.float64)) <= tol


# Weights whose rows are a multiple of 16 and whose features a multiple of 128 are held as tiles of 16 rows x 128
# features: one wave per row group and k share (1, 2, 4 or 8 shares by the matrix's size), activations whole in LDS or
# in chunks (8 rows of 14336 features, 16 of 8192), row groups that do not fill a workgroup's set, several rounds per
# workgroup (20000 rows x 128 features), batches that share weights, and more than 16 rows (the matrix-matrix kernel
# reading tiles; 17 rows of f32 in groups of 8).
TILED_SHAPES = [
    (1, 1, 1, 16, 128), (1, 1, 1, 48, 256), (2, 2, 1, 80, 384), (1, 2, 2, 1024, 4096), (1, 1, 3, 1024, 4096), (1, 3, 2, 4096, 1024), (1, 1, 1, 14336, 4096), (1, 1, 3, 4096, 14336),
    (1, 1, 8, 14336, 4096), (1, 1, 8, 4096, 14336), (1, 1, 16, 1040, 8192), (2, 4, 5, 272, 2176), (1, 1, 7, 20000, 128),
    (1, 1, 12, 6000 * 16, 256), (1, 1, 17, 160, 640), (1, 2, 40, 4112, 1152), (1, 1, 130, 2048, 4096),
    (1, 2, 200, 528, 384), (1, 1, 2100, 4112, 1152),   # the matrix-matrix kernel: 64 and 128 activation rows per workgroup, ragged edges
    (1, 1, 100, 1024, 768), (1, 1, 400, 8192, 512),      # ... with k split over 2 sets of waves (130 x 2048 x 4096 above: over 4)
    # ... sets of 4 waves and of 2 (64 rows of the weights per workgroup; the three small matrices above take sets of one
    # wave), k over 4, 2 and 1 of them
    (1, 1, 400, 4096, 512), (1, 1, 400, 4096, 768), (1, 1, 400, 4096, 384),
    (1, 1, 200, 4096, 512), (1, 1, 200, 4096, 768), (1, 1, 200, 4096, 384),
    # ... 25..32 rows: tiles of 32 activation rows
    (1, 1, 30, 4096, 512), (1, 2, 32, 14336, 256), (1, 1, 26, 32768, 128), (1, 1, 28, 50000, 256), (1, 1, 28, 50000, 128),
    (1, 1, 30, 14336, 512), (1, 1, 30, 4096, 1024),   # (the last: k over 8 sets of one wave, as 130 x 2048 x 4096 above)
]


@pytest.mark.parametrize("dt", [np.float32, np.float16])
@pytest.mark.parametrize("wb,ab,m,n,k", TILED_SHAPES)
def test_tiled_weights_match_the_f64_product(rt, monkeypatch, dt, wb, ab, m, n, k):
    rng = np.random.default_rng(n + k + m)
    w = (rng.standard_normal((wb, n, k)) * 0.05).astype(np.float32)
    w[:, :, ::97] *= 8.0
    act = rng.standard_normal((ab, m, k)).astype(dt)
    blocks = orc.quant(Q4, w)
    wq = tract_amd.Q40Weights(blocks, wb, n, k)
    assert np.array_equal(wq.blocks(), blocks)              # the tiles give the canonical bytes back
    got = tract_amd.GgmlGemm().eval(act, wq).to_numpy()
    assert got.dtype == dt and got.shape == (ab, m, n)
    tol = 1e-4 if dt == np.float32 else 4e-3
    want = f64_product(blocks, act, dt)
    assert rel_err(got, want) <= tol
    if n <= 3072 and m <= 2:
        # a small matrix keeps planes of codes and scales beside its tiles and runs one or two rows over those:
        # without them (the variable is read when the weights are created) the same call goes over the tiles
        monkeypatch.setenv("TROCM_Q4_ROWS_TOO", "0")
        only_tiles = tract_amd.Q40Weights(blocks, wb, n, k)
        monkeypatch.delenv("TROCM_Q4_ROWS_TOO")
        assert np.array_equal(only_tiles.blocks(), blocks)
        assert rel_err(tract_amd.GgmlGemm().eval(act, only_tiles).to_numpy(), want) <= tol


def test_tiles_and_planes_hold_the_same_weights(rt, monkeypatch):
    """The same matrix as tiles and (TROCM_Q4_TILED=0 at creation) as planes of codes and scales: equal exports, and
    products that agree to the tolerance of either."""
    rng = np.random.default_rng(5)
    n, k = 2048, 1024
    w = (rng.standard_normal((1, n, k)) * 0.05).astype(np.float32)
    blocks = orc.quant(Q4, w)
    tiles = tract_amd.Q40Weights(blocks, 1, n, k)
    monkeypatch.setenv("TROCM_Q4_TILED", "0")
    planes = tract_amd.Q40Weights(blocks, 1, n, k)
    monkeypatch.delenv("TROCM_Q4_TILED")
    assert np.array_equal(tiles.blocks(), planes.blocks())
    for dt, tol in ((np.float16, 4e-3), (np.float32, 1e-4)):
        for m in (1, 6, 24):
            act = rng.standard_normal((1, m, k)).astype(dt)
            a = tract_amd.GgmlGemm().eval(act, tiles).to_numpy()
            b = tract_amd.GgmlGemm().eval(act, planes).to_numpy()
            assert rel_err(a, b.astype(np.float64)) <= 2 * tol
            assert rel_err(a, f64_product(blocks, act, dt)) <= tol


@pytest.mark.parametrize("tiled", [1, 0])
@pytest.mark.parametrize("m,k", [(16, 3584), (8, 4096)])
def test_tall_matrix_of_repeated_rows(rt, monkeypatch, m, k, tiled):
    """65536 weight rows (the output matrix of a large vocabulary), built by repeating 512 quantised rows: every
    workgroup walks several row groups behind one staged copy of the activations, as tiles and as planes of codes
    and scales.  As planes, 16 rows of 3584 features leave the waves no LDS for their code buffers (the kernel that
    loads 64 bytes per row and transposes over the lane groups runs), 8 rows do.  Expected: the f64 product of the
    512 rows, repeated."""
    monkeypatch.setenv("TROCM_Q4_TILED", str(tiled))
    rng = np.random.default_rng(m + k)
    base_n, reps = 512, 128
    w = (rng.standard_normal((1, base_n, k)) * 0.05).astype(np.float32)
    w[:, :, ::97] *= 8.0
    act = rng.standard_normal((1, m, k)).astype(np.float16)
    base = orc.quant(Q4, w)
    blocks = np.ascontiguousarray(np.tile(base, (1, reps, 1)))
    wq = tract_amd.Q40Weights(blocks, 1, base_n * reps, k)
    got = tract_amd.GgmlGemm().eval(act, wq).to_numpy()
    want = np.tile(f64_product(base, act, np.float16), (1, 1, reps))
    assert got.shape == want.shape and rel_err(got, want) <= 4e-3
    assert np.array_equal(got[:, :, :base_n], got[:, :, -base_n:])


def test_closed_form_blocks(rt):
    """Nibbles i % 16 in every block (the table of q4_0.rs:722-739): sums of whole blocks and single
    elements are known exactly, low and high nibbles alike."""
    n, k = 4, 96
    scales = np.array([0.5, 0.25, 1.0, 2.0], np.float32)
    codes = np.arange(32) % 16
    packed = (codes[:16] | (codes[16:] << 4)).astype(np.uint8)
    blocks = np.zeros((1, n, 3 * 18), np.uint8)
    for j in range(n):
        for b in range(3):
            blocks[0, j, b * 18:b * 18 + 2] = np.array([scales[j]], np.float16).view(np.uint8)
            blocks[0, j, b * 18 + 2:b * 18 + 18] = packed
    wq = tract_amd.Q40Weights(blocks, 1, n, k)
    gemm = tract_amd.GgmlGemm()
    for dt in (np.float32, np.float16):
        assert np.array_equal(gemm.eval(np.ones((1, 1, k), dt), wq).to_numpy()[0, 0], (scales * -48.0).astype(dt))
        for pos, code in ((37, 5), (16, 0), (95, 15), (0, 0)):
            e = np.zeros((1, 1, k), dt)
            e[0, 0, pos] = 1
            assert np.array_equal(gemm.eval(e, wq).to_numpy()[0, 0], (scales * (code - 8)).astype(dt))


def test_weights_round_trip_and_quantize(rt):
    rng = np.random.default_rng(9)
    w = rng.standard_normal((2, 37, 160)).astype(np.float32)
    blocks = orc.quant(Q4, w)
    wq = tract_amd.Q40Weights(blocks, 2, 37, 160)
    assert np.array_equal(wq.blocks(), blocks)              # the canonical bytes come back unchanged
    wq2 = tract_amd.Q40Weights.quantize(w)                  # quantised on the device: same bytes as the oracle
    assert np.array_equal(wq2.blocks(), blocks)


def test_error_paths(rt):
    blocks = np.zeros((1, 4, 2 * 18), np.uint8)
    wq = tract_amd.Q40Weights(blocks, 1, 4, 64)
    with pytest.raises(tract_amd.TractRocmError, match="whole number of 32-element blocks"):
        tract_amd.Q40Weights(np.zeros(18, np.uint8), 1, 1, 40)
    with pytest.raises(tract_amd.TractRocmError, match="do not match"):
        tract_amd.GgmlGemm().eval(np.zeros((1, 1, 32), np.float32), wq)
    w2 = tract_amd.Q40Weights(np.zeros((2, 4, 2 * 18), np.uint8), 2, 4, 64)
    with pytest.raises(tract_amd.TractRocmError, match="not a multiple of the weights' batch"):
        tract_amd.GgmlGemm().eval(np.zeros((3, 1, 64), np.float32), w2)
    out = tract_amd.GgmlGemm().eval(np.zeros((0, 1, 64), np.float32).reshape(0, 1, 64), wq)
    assert out.shape == (0, 1, 4)
