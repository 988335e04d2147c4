"""Pins the oracle's attention restatement (FlashSdpaOp tile loop and the f64
textbook form) against: the five golden io.npz the reference holds, the literal
problems of its cross-backend suite with their closed-form answers, an independent
vectorised numpy implementation, and invariants a dropped term or wrong index breaks."""
import os

import numpy as np
import pytest

from oracle import oracle as orc
from tests import cases


def _load(golden_dir, name):
    return np.load(os.path.join(golden_dir, "ref_sdpa", name, "io.npz"))


@pytest.mark.parametrize("name,causal,scale", [("simple-causal-f32", True, None),
                                               ("simple-non-causal-f32", False, None),
                                               ("simple-scale-f32", False, 1.3)])
def test_reference_golden_f32(golden_dir, name, causal, scale):
    z = _load(golden_dir, name)
    x, want = z["input_0"], z["output_0"]
    got = orc.flash_sdpa(x, x, x, causal=causal, scale=scale)
    assert np.abs(got - want).max() < 1e-6
    assert np.abs(orc.naive_sdpa_f64(x, x, x, causal=causal, scale=scale) - want).max() < 1e-6


def test_reference_golden_mask(golden_dir):
    z = _load(golden_dir, "simple-mask-f32")
    raw = np.fromfile(os.path.join(golden_dir, "ref_sdpa", "simple-mask-f32", "v0.dat"), dtype=np.uint8)
    mask = raw[128:].view(np.float32).reshape(1, 2, 1)  # variable [2,1] unsqueezed at axis 0
    q, k, v, want = z["input_0"], z["input_1"], z["input_2"], z["output_0"]
    m = np.broadcast_to(mask, (1, 2, 2))
    assert np.abs(orc.flash_sdpa(q, k, v, mask=m) - want).max() < 1e-6
    assert np.abs(orc.naive_sdpa_f64(q, k, v, mask=m) - want).max() < 1e-6


def test_reference_golden_f16(golden_dir):
    z = _load(golden_dir, "simple-f16")
    x = z["input_0"].astype(np.float16)
    got = orc.flash_sdpa(x, x, x).astype(np.float32)
    assert np.abs(got - z["output_0"]).max() < 1e-3


@pytest.mark.parametrize("name", sorted(cases.sdpa_literal_cases()))
def test_literal_suite_cases(name):
    q, k, v, mask, scale, causal = cases.sdpa_literal_cases()[name]
    want = cases.textbook_sdpa(q, k, v, mask, scale, causal)
    tol = 1e-3 if q.dtype == np.float16 else 1e-6
    got = orc.flash_sdpa(q, k, v, mask=mask, causal=causal, scale=scale)
    assert got.dtype == q.dtype and got.shape == want.shape
    assert np.abs(got.astype(np.float64) - want).max() < tol
    assert np.abs(orc.naive_sdpa_f64(q, k, v, mask, causal, scale) - want).max() < 1e-12


def test_closed_form_answers():
    c = cases.sdpa_literal_cases()
    # causal_with_s_and_p_0: Sq=2, Sk=3, V=[0,0,1]: row r averages V[0..=p+r], p=1 -> [0, 1/3]
    q, k, v, *_ = c["causal_with_s_and_p_0"]
    assert np.allclose(orc.flash_sdpa(q, k, v, causal=True)[0, :, 0], [0.0, 1 / 3], atol=1e-7)
    # gqa_f32_0: two kv heads, V = [0],[1] -> outputs 0 and 1 (kv head = q head / group)
    q, k, v, *_ = c["gqa_f32_0"]
    assert np.array_equal(orc.flash_sdpa(q, k, v)[0, :, 0, 0], [0.0, 1.0])
    # mask_0: row 1 has logits [0,-1] over V=[2,0] -> 2/(1+e^-1)
    q, k, v, m, *_ = c["mask_0"]
    got = orc.flash_sdpa(q, k, v, mask=m)[0, :, 0]
    assert np.allclose(got, [1.0, 2 / (1 + np.exp(-1.0))], atol=1e-6)


@pytest.mark.parametrize("B,Hq,Hkv,Sq,Sk,D,causal", [
    (1, 2, 2, 16, 24, 8, False),      # flash_sdpa.rs:359-405
    (1, 4, 2, 1, 33, 8, True),        # flash_sdpa.rs:407-435
    (2, 8, 2, 70, 70, 16, True),      # several 32x32 tiles, causal diagonal inside tiles
    (1, 4, 1, 5, 133, 64, True),      # bottom-right aligned causal, q_len < kv_len
    (2, 6, 3, 40, 97, 32, False),
])
def test_flash_matches_independent_numpy(B, Hq, Hkv, Sq, Sk, D, causal):
    rng = np.random.default_rng(7)
    q = rng.standard_normal((B, Hq, Sq, D), dtype=np.float32)
    k = rng.standard_normal((B, Hkv, Sk, D), dtype=np.float32)
    v = rng.standard_normal((B, Hkv, Sk, D), dtype=np.float32)
    want = cases.textbook_sdpa(q, k, v, causal=causal)
    assert np.abs(orc.flash_sdpa(q, k, v, causal=causal) - want).max() < 1e-5
    assert np.abs(orc.flash_sdpa(q, k, v, causal=causal, threads=4) - want).max() < 1e-5
    assert np.abs(orc.naive_sdpa_f64(q, k, v, causal=causal) - want).max() < 1e-12
    # f16 eval path: whole-tensor casts, result rounded to f16 (flash_sdpa.rs:407-435: < 5e-3)
    got16 = orc.flash_sdpa(q.astype(np.float16), k.astype(np.float16), v.astype(np.float16), causal=causal)
    assert got16.dtype == np.float16 and np.abs(got16.astype(np.float64) - want).max() < 2e-2


def test_mask_with_padding_columns_and_broadcast():
    rng = np.random.default_rng(8)
    B, Hq, Hkv, Sq, Sk, D = 2, 4, 2, 3, 80, 16
    q = rng.standard_normal((B, Hq, Sq, D), dtype=np.float32)
    k = rng.standard_normal((B, Hkv, Sk, D), dtype=np.float32)
    v = rng.standard_normal((B, Hkv, Sk, D), dtype=np.float32)
    lens = [50, 80]
    mask = np.zeros((B, 1, Sq, Sk), dtype=np.float32)
    for b, n in enumerate(lens):
        mask[b, :, :, n:] = np.finfo(np.float32).min  # finite minimum, like Sdpa's causal mask
    got = orc.flash_sdpa(q, k, v, mask=mask)
    for b, n in enumerate(lens):
        want = cases.textbook_sdpa(q[b:b + 1], k[b:b + 1, :, :n], v[b:b + 1, :, :n])
        assert np.abs(got[b:b + 1] - want).max() < 1e-5


def test_invariants():
    rng = np.random.default_rng(9)
    B, Hq, Hkv, Sk, D = 1, 8, 2, 75, 16
    k = rng.standard_normal((B, Hkv, Sk, D), dtype=np.float32)
    v = rng.standard_normal((B, Hkv, Sk, D), dtype=np.float32)
    # all-equal logits (q = 0) -> output is the mean of the visible V rows
    q0 = np.zeros((B, Hq, 1, D), dtype=np.float32)
    got = orc.flash_sdpa(q0, k, v)
    assert np.abs(got[0, :, 0] - np.repeat(v.mean(axis=2)[0], 4, axis=0)).max() < 1e-6
    # q heads of one group with identical Q give identical outputs; groups differ
    q = np.repeat(rng.standard_normal((B, 1, 1, D), dtype=np.float32), Hq, axis=1)
    got = orc.flash_sdpa(q, k, v)
    assert np.array_equal(got[0, 0], got[0, 3]) and not np.array_equal(got[0, 0], got[0, 4])
    # decode step t of a causal run == row t of the one-shot causal prefill
    S = 40
    qs = rng.standard_normal((B, Hq, S, D), dtype=np.float32)
    full = orc.flash_sdpa(qs, k[:, :, :S], v[:, :, :S], causal=True)
    for t in (0, 1, 31, 32, 39):
        step = orc.flash_sdpa(qs[:, :, t:t + 1], k[:, :, :t + 1], v[:, :, :t + 1], causal=True)
        assert np.abs(step[:, :, 0] - full[:, :, t]).max() < 2e-6
    # scale default is 1/sqrt(D)
    a = orc.flash_sdpa(qs, k, v)
    b = orc.flash_sdpa(qs, k, v, scale=1 / np.sqrt(D))
    assert np.abs(a - b).max() < 1e-6
    # view over a capacity buffer == dense (InPlaceKvSdpa's zero-copy path)
    cap = 128
    kb = np.full((B, Hkv, cap, D), np.nan, dtype=np.float32)
    vb = np.full((B, Hkv, cap, D), np.nan, dtype=np.float32)
    kb[:, :, :Sk], vb[:, :, :Sk] = k, v
    assert np.array_equal(orc.flash_sdpa_view(qs, kb, vb, Sk), a)


# ------------------------------------------------------------------ StreamedSdpaOp (streamed_sdpa.rs:164-272)
def _streamed_f64(q, k, v, mask, causal, scale):
    """The operator's definition, vectorised in f64: its own mask rules and a row that sees nothing is zero."""
    q, k, v = (np.asarray(a, dtype=np.float64) for a in (q, k, v))
    B, Hq, Sq, D = q.shape
    Hkv, Sk = k.shape[1], k.shape[2]
    g = Hq // Hkv
    sc = (1.0 / D) ** 0.5 if scale is None else scale
    s = np.einsum("bhqd,bhkd->bhqk", q, np.repeat(k, g, axis=1)) * sc
    if mask is not None:
        s = s + np.asarray(mask, dtype=np.float64)[None, None]
    elif causal:
        s = np.where(np.arange(Sk)[None, :] > np.arange(Sq)[:, None], -np.inf, s)
    mx = s.max(axis=-1, keepdims=True)
    with np.errstate(invalid="ignore"):
        p = np.where(np.isfinite(s), np.exp(s - np.where(np.isfinite(mx), mx, 0.0)), 0.0)
    l = p.sum(axis=-1, keepdims=True)
    p = np.where(l > 0, p / np.where(l > 0, l, 1.0), 0.0)
    return np.einsum("bhqk,bhkd->bhqd", p, np.repeat(v, g, axis=1))


@pytest.mark.parametrize("B,Hq,Hkv,Sq,Sk,D,causal,with_mask,scale", [
    (2, 4, 2, 9, 9, 16, True, False, None),      # square causal
    (1, 6, 2, 5, 23, 8, True, False, 0.7),       # kv_len > q_len: the diagonal starts at the FIRST key
    (1, 2, 1, 17, 6, 8, True, False, None),      # kv_len < q_len: late queries see every key
    (2, 3, 3, 7, 13, 32, False, False, None),
    (1, 4, 2, 6, 11, 16, True, True, None),      # a mask overrides the causal flag
    (1, 2, 2, 1, 40, 64, False, True, 1.1),
])
def test_streamed_sdpa_vs_f64_definition(B, Hq, Hkv, Sq, Sk, D, causal, with_mask, scale):
    rng = np.random.default_rng(B * 1000 + Sq * 10 + Sk)
    q, k, v = (rng.standard_normal(sh).astype(np.float32) for sh in ((B, Hq, Sq, D), (B, Hkv, Sk, D), (B, Hkv, Sk, D)))
    mask = None
    if with_mask:
        mask = rng.standard_normal((Sq, Sk)).astype(np.float32)
        mask[rng.random((Sq, Sk)) < 0.3] = -np.inf
        mask[Sq // 2, :] = -np.inf               # a row that sees nothing
    want = _streamed_f64(q, k, v, mask, causal, scale)
    for bk in (1, 5, 64, 1000):                  # block_k changes the order of the sums only
        got = orc.streamed_sdpa(q, k, v, mask=mask, causal=causal, scale=scale, block_k=bk)
        assert got.shape == q.shape and got.dtype == np.float32
        assert np.abs(got - want).max() < 2e-6, bk
    if with_mask:
        assert not got[:, :, Sq // 2].any()
    if causal and not with_mask and Sk > Sq:     # keys past the q_len-th are invisible to every query
        trunc = orc.streamed_sdpa(q, k[:, :, :Sq], v[:, :, :Sq], causal=True, scale=scale)
        assert np.abs(got - trunc).max() < 1e-6
    if causal and not with_mask and Sk == Sq:    # where the two operators' rules coincide, so do they
        assert np.abs(got - orc.flash_sdpa(q, k, v, causal=True, scale=scale)).max() < 2e-6


def test_streamed_sdpa_rank3_f16_and_first_key_only():
    rng = np.random.default_rng(3)
    q, k, v = (rng.standard_normal(sh).astype(np.float16) for sh in ((2, 1, 32), (2, 9, 32), (2, 9, 32)))
    got = orc.streamed_sdpa(q, k, v, causal=True)
    assert got.shape == q.shape and got.dtype == np.float16
    assert np.array_equal(got[:, 0], v[:, 0])    # one query, causal: it sees key 0 alone (streamed_sdpa.rs:218)
