"""Pins the oracle's KV-cache restatement: the valid region must be bit-identical to
numpy.concatenate (the reference's own test criterion, inplace_kv_cache.rs:366-404,
dyn_kv_cache.rs:499-527), capacities follow cap0 = first chunk, cap' = max(2cap, len+new)
(:61-80), and 1024 single pushes cost O(log T) reallocations (:406-418)."""
import os

import numpy as np
import pytest

from oracle import oracle as orc


def _chunks(rng, shape, axis, lens, dt):
    out = []
    for n in lens:
        s = list(shape)
        s[axis] = n
        out.append((rng.standard_normal(s) * 4).astype(dt))
    return out


@pytest.mark.parametrize("dt", [np.float32, np.float16, np.uint8])
@pytest.mark.parametrize("shape,axis", [((1, 4, 0, 8), 2), ((2, 3, 0, 16), 2), ((2, 0, 5), 1), ((0, 7), 0)])
def test_inplace_matches_concatenate(dt, shape, axis):
    rng = np.random.default_rng(0)
    lens = [3, 1, 1, 0, 7, 1, 2, 30, 1]
    chunks = _chunks(rng, shape, axis, lens, dt)
    c = orc.InPlaceKvCache(axis)
    cap = 0
    dyn = None
    for i, ch in enumerate(chunks):
        c.push(ch)
        dyn = orc.concat_append(dyn, ch, axis)
        n = sum(lens[: i + 1])
        if ch.shape[axis]:
            cap = ch.shape[axis] if cap == 0 else (cap if n <= cap else max(2 * cap, n))
        assert c.len() == n and c.capacity() == cap
        want = np.concatenate(chunks[: i + 1], axis=axis)
        assert c.valid_contiguous().tobytes() == want.tobytes()
        assert dyn.tobytes() == want.tobytes()


def test_realloc_count_is_logarithmic():
    c = orc.InPlaceKvCache(2)
    x = np.ones((1, 2, 1, 4), dtype=np.float32)
    for _ in range(1024):
        c.push(x)
    assert c.len() == 1024 and c.capacity() == 1024
    assert c.reallocs() == 10 and c.reallocs() <= 12  # 1,2,4,...,1024


def test_reference_gqa_fixture_cache_is_concat(golden_dir):
    z = np.load(os.path.join(golden_dir, "ref_sdpa", "simple-grouped-query-att-f32", "io.npz"))
    for i in (1, 2):
        past, out = z[f"input_{i}"], z[f"output_{i}"]
        new = out[:, :, 10:]
        c = orc.InPlaceKvCache(2)
        c.push(past)
        c.push(new)
        assert c.valid_contiguous().tobytes() == out.tobytes()
        assert orc.concat_append(past, new, 2).tobytes() == out.tobytes()
        assert np.array_equal(out[:, :, :10], past)
