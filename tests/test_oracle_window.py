"""Pins for the oracle's WindowKvCache (transformers/src/ops/window_kv_cache.rs)."""
import numpy as np

from oracle import oracle as orc
from tests import cases


def _tok(v, shape=(1, 1, 1, 1)):
    return np.full(shape, v, np.float32)


def test_window_holds_last_w_as_a_set():
    # window_kv_cache.rs:342-362
    w = 4
    c = orc.WindowKvCache(w)
    full = []
    for t in range(10):
        c.push(_tok(float(t)))
        full.append(float(t))
        assert c.len() <= w
        assert sorted(c.valid_view().ravel().tolist()) == sorted(full[-w:])
    assert c.capacity() == w


def test_prefill_chunk_larger_than_window_keeps_last_w():
    # window_kv_cache.rs:364-374; the slots are laid out [0, w) in order and the cursor resets (:119-126)
    c = orc.WindowKvCache(3)
    c.push(np.arange(7, dtype=np.float32).reshape(1, 1, 7, 1))
    assert c.valid_view().ravel().tolist() == [4.0, 5.0, 6.0]
    assert c.cursor() == 0 and c.len() == 3


def test_single_token_pushes_land_at_t_mod_w():
    w = 5
    c = orc.WindowKvCache(w)
    for t in range(23):
        c.push(_tok(float(t), (2, 3, 1, 4)))
        assert c.cursor() == (t + 1) % w
        view = c.valid_view()
        for slot in range(c.len()):
            newest_in_slot = max(u for u in range(t + 1) if u % w == slot)
            assert (view[:, :, slot] == newest_in_slot).all()


def test_wrap_around_push_splits_in_two():
    # hand-derived from :129-140: w=5, push 3 (slots 0..2, cursor 3), push 4: first = 2 go to slots 3,4,
    # the other 2 to slots 0,1, cursor = 2
    c = orc.WindowKvCache(5)
    c.push(np.arange(0, 3, dtype=np.float32).reshape(1, 1, 3, 1))
    assert c.valid_view().ravel().tolist() == [0, 1, 2] and c.cursor() == 3
    c.push(np.arange(3, 7, dtype=np.float32).reshape(1, 1, 4, 1))
    assert c.valid_view().ravel().tolist() == [5, 6, 2, 3, 4] and c.cursor() == 2 and c.len() == 5
    c.push(np.arange(7, 10, dtype=np.float32).reshape(1, 1, 3, 1))   # end == w: cursor wraps to 0
    assert c.valid_view().ravel().tolist() == [5, 6, 7, 8, 9] and c.cursor() == 0
    c.push(np.zeros((1, 1, 0, 1), np.float32))
    assert c.cursor() == 0 and c.len() == 5


def test_windowed_attention_matches_last_w_full():
    # window_kv_cache.rs:407-466: values base + sin(0.013 i), h=2, d=8, w=6, 20 steps
    h, d, w = 2, 8, 6

    def seq(base):
        return (base + np.sin(np.arange(h * d, dtype=np.float32) * np.float32(0.013))).astype(np.float32).reshape(1, h, 1, d)

    kc, vc = orc.WindowKvCache(w), orc.WindowKvCache(w)
    kfull, vfull = [], []
    for t in range(20):
        knew, vnew = seq(1.0 + t * 0.1), seq(5.0 - t * 0.07)
        kc.push(knew), vc.push(vnew)
        kfull.append(knew), vfull.append(vnew)
        q = seq(9.0 + t * 0.05)
        n = kc.len()
        o_win = orc.flash_sdpa(q, kc.valid_view(), vc.valid_view())
        o_ref = cases.textbook_sdpa(q, np.concatenate(kfull[-n:], 2), np.concatenate(vfull[-n:], 2))
        assert np.abs(o_win - o_ref).max() <= 1e-5
