"""Pins the oracle's KIVI-style affine quantisers (oracle/kivi_oracle.c) before anything is compared to them:
the data and assertions of the reference's own unit tests (kv_quant.rs:446-560, quant_dyn_kv_cache.rs:728-778),
byte strings derived by hand from the formulas, an independent vectorised numpy form, and the structural facts
(sink tokens and the partial key block stay f32, a key block freezes at its 32nd token)."""
import numpy as np
import pytest

from oracle import oracle as orc


def lcg(seed, inc=1):
    """The generator of the reference's tests (kv_quant.rs:511-516, quant_dyn_kv_cache.rs:737-741)."""
    st = seed
    while True:
        st = (st * 6364136223846793005 + inc) & 0xFFFFFFFFFFFFFFFF
        yield np.float32(np.float32(st >> 40) / np.float32(1 << 24)) - np.float32(0.5)


def take(gen, *shape):
    return np.array([next(gen) for _ in range(int(np.prod(shape)))], np.float32).reshape(shape)


def round_half_away(v):
    t = np.trunc(v)
    return t + np.where(np.abs(v - t) >= 0.5, np.sign(v), 0).astype(np.float32)


def np_affine(x, bits, axis):
    """Independent statement: (codes, lo, scale) of groups along `axis` (f32 arithmetic throughout)."""
    lv = np.float32((1 << bits) - 1)
    lo = x.min(axis=axis, keepdims=True)
    hi = x.max(axis=axis, keepdims=True)
    scale = np.where(hi > lo, (hi - lo) / lv, np.float32(1)).astype(np.float32)
    codes = np.clip(round_half_away(((x - lo) / scale).astype(np.float32)), 0, lv).astype(np.uint8)
    return codes, lo.astype(np.float32), scale


# ---- hand-derived bytes ------------------------------------------------------------------------------------
def test_per_token_bytes_by_hand():
    # [0,1,2,3]: lo 0, scale 3/255 -> codes 0, 85, 170, 255; at 4 bits scale 0.2 -> 0, 5, 10, 15 -> bytes 0x50 0xFA
    row = np.array([0, 1, 2, 3], np.float32)
    s8 = orc.KiviStore(orc.KIVI_PER_TOKEN, 4, 8, 0)
    s8.push_token(row)
    st = s8.state()
    assert st["packed"].tolist() == [[0, 85, 170, 255]]
    assert st["lo"].tolist() == [0.0] and st["scale"][0] == np.float32(3) / np.float32(255)
    s4 = orc.KiviStore(orc.KIVI_PER_TOKEN, 4, 4, 0)
    s4.push_token(row)
    st = s4.state()
    assert st["packed"].tolist() == [[0x50, 0xFA]] and st["scale"][0] == np.float32(0.2)
    # a constant row: hi == lo -> scale 1, every code 0, dequantises to lo
    s = orc.KiviStore(orc.KIVI_PER_TOKEN, 4, 8, 0)
    s.push_token(np.full(4, 2.5, np.float32))
    assert s.state()["scale"].tolist() == [1.0] and s.state()["packed"].tolist() == [[0, 0, 0, 0]]
    assert s.dequant_all().tolist() == [[2.5] * 4]
    # odd head size at 4 bits: the last byte's high nibble is 0 (quant_dyn_kv_cache.rs:69-72)
    s = orc.KiviStore(orc.KIVI_PER_TOKEN, 3, 4, 0)
    s.push_token(np.array([0, 15, 15], np.float32))
    assert s.state()["packed"].tolist() == [[0xF0, 0x0F]]


def test_rounding_is_half_away_and_clamped():
    # lo 0, hi 255 at 8 bits: scale 1, so the code is round(x): 0.5 -> 1, 1.5 -> 2, 2.5 -> 3 (half away, not half even)
    row = np.array([0, 0.5, 1.5, 2.5, 254.5, 255], np.float32)
    s = orc.KiviStore(orc.KIVI_PER_TOKEN, 6, 8, 0)
    s.push_token(row)
    assert s.state()["packed"].tolist() == [[0, 1, 2, 3, 255, 255]]


def test_nan_and_inf_rows_by_hand():
    # NaN is ignored by min / max and its code is 0 (NaN as u8); +inf makes scale inf: finite / inf = 0, inf / inf = NaN -> 0
    s = orc.KiviStore(orc.KIVI_PER_TOKEN, 4, 8, 0)
    s.push_token(np.array([np.nan, 1, 3, 1.5], np.float32))
    st = s.state()
    assert st["lo"].tolist() == [1.0] and st["packed"].tolist() == [[0, 0, 255, 64]]   # (1.5 - 1) / (2 / 255) = 63.75 -> 64
    s = orc.KiviStore(orc.KIVI_PER_TOKEN, 3, 8, 0)
    s.push_token(np.array([np.inf, 1, 2], np.float32))
    st = s.state()
    assert st["lo"].tolist() == [1.0] and np.isinf(st["scale"][0]) and st["packed"].tolist() == [[0, 0, 0]]
    s = orc.KiviStore(orc.KIVI_PER_TOKEN, 2, 8, 0)
    s.push_token(np.array([np.nan, np.nan], np.float32))       # lo = +inf, hi = -inf: scale 1, codes 0
    st = s.state()
    assert np.isposinf(st["lo"][0]) and st["scale"].tolist() == [1.0] and st["packed"].tolist() == [[0, 0]]


def test_signalling_nan_is_ignored_like_a_quiet_one():
    # f32::min / f32::max return the other operand for ANY NaN (core::f32: "handles all NaNs the same way"); C's fminf /
    # fmaxf answer NaN for a signalling one, after which the running minimum would forget what it had seen
    row = np.array([-60.0, 0.0, 50.0, 1.0], np.float32)
    row.view(np.uint32)[1] = 0x7FA00000
    s = orc.KiviStore(orc.KIVI_PER_TOKEN, 4, 8, 0)
    s.push_token(row)
    st = s.state()
    assert st["lo"].tolist() == [-60.0] and st["scale"][0] == np.float32(np.float32(110.0) / np.float32(255.0))
    assert st["packed"].tolist() == [[0, 0, 255, 141]]          # 61 / (110 / 255) = 141.4
    blk = np.zeros((32, 1), np.float32)
    blk[3, 0], blk[5, 0] = 70.0, -80.0
    blk.view(np.uint32)[4, 0] = 0xFFA00001
    s = orc.KiviStore(orc.KIVI_BLOCK_CHANNEL, 1, 8, 0)
    for r in blk:
        s.push_token(r)
    st = s.state()
    assert st["lo"].reshape(-1).tolist() == [-80.0] and st["scale"].reshape(-1)[0] == np.float32(np.float32(150.0) / np.float32(255.0))


def test_running_channel_by_hand():
    # kv_quant.rs:200-222 with one channel: lo follows the minimum, scale only grows, old codes are kept and
    # read back with the CURRENT parameters (:224-234)
    s = orc.KiviStore(orc.KIVI_RUNNING_CHANNEL, 1, 8, 0)
    want = []
    for val, code, lo, scale in [(1.0, 0, 1.0, 1.0), (3.0, 2, 1.0, 1.0), (511.0, 255, 1.0, 2.0), (-1.0, 0, -1.0, 2.0)]:
        s.push_token(np.array([val], np.float32))
        want.append(code)
        st = s.state()
        assert st["packed"][:, 0].tolist() == want and st["lo"].tolist() == [lo] and st["scale"].tolist() == [scale]
    assert s.dequant_all()[:, 0].tolist() == [-1.0, 3.0, 509.0, -1.0]
    assert s.memory_bytes() == 4 * 1 + 1 * 8


def test_sinks_and_partial_block_stay_f32_and_blocks_freeze_at_32():
    rng = np.random.default_rng(5)
    d = 16
    rows = rng.standard_normal((4 + 32 + 32 + 7, d)).astype(np.float32)
    for layout in (orc.KIVI_BLOCK_CHANNEL, orc.KIVI_PER_TOKEN):
        s = orc.KiviStore(layout, d, 8)
        for t, r in enumerate(rows):
            s.push_token(r)
            st = s.state()
            assert st["sink"].shape[0] == min(t + 1, 4)
            if layout == orc.KIVI_BLOCK_CHANNEL:
                q = max(t + 1 - 4, 0)
                assert st["packed"].shape[0] == q // 32 * 32 and st["residual"].shape[0] == q % 32
                assert st["lo"].size == q // 32 * d
            else:
                assert st["packed"].shape[0] == max(t + 1 - 4, 0) and st["residual"].shape[0] == 0
        st = s.state()
        deq = s.dequant_all()
        assert st["sink"].tobytes() == rows[:4].tobytes() and deq[:4].tobytes() == rows[:4].tobytes()
        if layout == orc.KIVI_BLOCK_CHANNEL:
            assert st["residual"].tobytes() == rows[68:].tobytes() and deq[68:].tobytes() == rows[68:].tobytes()
            # a frozen block does not change when later tokens arrive
            before = deq[4:68].copy()
            for r in rng.standard_normal((40, d)).astype(np.float32) * 50:
                s.push_token(r)
            assert s.dequant_all()[4:68].tobytes() == before.tobytes()


# ---- independent numpy form ----------------------------------------------------------------------------------
@pytest.mark.parametrize("bits", [4, 8])
def test_stores_match_numpy_closed_form(bits):
    rng = np.random.default_rng(bits)
    d = 32
    rows = (rng.standard_normal((4 + 96, d)) * rng.choice([0.1, 1, 20], d)).astype(np.float32)
    v = orc.KiviStore(orc.KIVI_PER_TOKEN, d, bits)
    k = orc.KiviStore(orc.KIVI_BLOCK_CHANNEL, d, bits)
    for r in rows:
        v.push_token(r)
        k.push_token(r)
    body = rows[4:]

    def packed(codes):
        return codes if bits == 8 else (codes[:, 0::2] | (codes[:, 1::2] << 4)).astype(np.uint8)

    codes, lo, scale = np_affine(body, bits, axis=1)
    st = v.state()
    assert st["packed"].tobytes() == packed(codes).tobytes()
    assert st["lo"].tobytes() == lo.tobytes() and st["scale"].tobytes() == scale.tobytes()
    want = (lo + (codes.astype(np.float32) * scale).astype(np.float32)).astype(np.float32)
    assert v.dequant_all()[4:].tobytes() == want.tobytes()

    blocks = body.reshape(3, 32, d)
    codes, lo, scale = np_affine(blocks, bits, axis=1)
    st = k.state()
    assert st["packed"].tobytes() == packed(codes.reshape(96, d)).tobytes()
    assert st["lo"].tobytes() == lo.tobytes() and st["scale"].tobytes() == scale.tobytes()
    want = (lo + (codes.astype(np.float32) * scale).astype(np.float32)).astype(np.float32).reshape(96, d)
    assert k.dequant_all()[4:].tobytes() == want.tobytes()
    # quant_dequant is the same arithmetic in one call (kv_quant.rs:73-98)
    assert orc.kivi_quant_dequant(body, bits, True).tobytes() == v.dequant_all()[4:].tobytes()
    assert orc.kivi_quant_dequant(blocks[1], bits, False).tobytes() == k.dequant_all()[36:68].tobytes()


# ---- the reference's own unit tests ----------------------------------------------------------------------------
def test_ref_error_decreases_with_bits():                      # kv_quant.rs:454-478
    x = np.array([[0, 1, 2, 3], [-1, 0.5, 4, 9], [2, 2, 2, 2.1]], np.float32)
    e4, e8, e16 = (np.abs(x - orc.kivi_quant_dequant(x, b, False)).max() for b in (4, 8, 16))
    assert e8 < e4 and e16 < e8 and e16 < 1e-3
    q = orc.kivi_quant_dequant(x, 8, False)
    for j in range(4):
        step = (x[:, j].max() - x[:, j].min()) / 255
        assert (np.abs(x[:, j] - q[:, j]) <= step / 2 + 1e-6).all()


def test_ref_per_channel_beats_per_row_on_outlier_channel():   # kv_quant.rs:483-505
    x = np.array([[100, 0.10, -0.20, 0.05], [-90, 0.02, 0.30, -0.08], [120, -0.15, 0.10, 0.20],
                  [-110, 0.07, -0.05, 0.12]], np.float32)
    pc = np.abs(x - orc.kivi_quant_dequant(x, 4, False))[:, 1:].max()
    pt = np.abs(x - orc.kivi_quant_dequant(x, 4, True))[:, 1:].max()
    assert pc < pt * 0.2


def test_ref_attention_near_lossless_at_8bit():                # kv_quant.rs:508-540
    s, d = 12, 16
    q, k, v = take(lcg(1), s, d)[0], take(lcg(2), s, d), take(lcg(3), s, d)

    def attn(k, v):
        sc = (k @ q) / np.sqrt(np.float32(d))
        p = np.exp(sc - sc.max())
        return (p / p.sum()) @ v

    full = attn(k, v)

    def dev(bits):
        o = attn(orc.kivi_quant_dequant(k, bits, False), orc.kivi_quant_dequant(v, bits, True))
        return np.linalg.norm(o - full) / max(np.linalg.norm(full), 1e-9)

    d4, d8, d12 = dev(4), dev(8), dev(12)
    assert d8 < d4 and d12 < d8 and d8 < 0.02


def test_ref_packed_u8_saves_memory():                         # kv_quant.rs:543-565
    t, d = 512, 64
    gen = lcg(42, 1442695040888963407)
    kc, vc = orc.KiviStore(orc.KIVI_RUNNING_CHANNEL, d, 8, 0), orc.KiviStore(orc.KIVI_PER_TOKEN, d, 8, 0)
    for _ in range(t):
        kc.push_token(take(gen, d))
        vc.push_token(take(gen, d))
    assert kc.memory_bytes() == t * d + d * 8 and vc.memory_bytes() == t * d + t * 8
    assert t * d * 4 * 2 / (kc.memory_bytes() + vc.memory_bytes()) > 3.0


def close_enough_super(a, b):
    """Tensor::close_enough with Approximation::SuperApproximate (data/src/tensor.rs:77): atol 0.1, rtol 0.05,
    at most 0.01 % outliers."""
    bad = np.abs(a - b) > 0.1 + 0.05 * np.abs(b)
    return bad.sum() <= 0.0001 * a.size


def test_ref_block_per_channel_key_consistent_over_growing_range():   # quant_dyn_kv_cache.rs:758-778
    d = 16
    kc = orc.KiviStore(orc.KIVI_BLOCK_CHANNEL, d, 8)
    rows = np.array([[t * 2.0 if c == 0 else np.sin(np.float32((t * 7 + c) * 0.013)) * 0.1 for c in range(d)]
                     for t in range(80)], np.float32)
    for r in rows:
        kc.push_token(r)
    assert kc.len() == 80
    assert np.abs(kc.dequant_all() - rows).max() < 1.0
    # the bound the block scheme implies: half a step of each block's range (block ranges of channel 0 are 62)
    assert np.abs(kc.dequant_all() - rows).max() <= 62 / 255 / 2 + 1e-5


def test_ref_quant_cache_accumulates_near_lossless_int8():     # quant_dyn_kv_cache.rs:728-756
    for per_channel in (False, True):
        gen = lcg(3)
        cache = orc.KiviCache(per_channel, 8)
        acc = None
        for _ in range(40):
            step = take(gen, 1, 2, 1, 8)
            cache.ingest(step)
            acc = step if acc is None else orc.concat_append(acc, step, 2)
            out = cache.dequantized()
            assert out.shape == acc.shape and close_enough_super(out, acc)
            # far tighter than the reference asks: half a quantisation step of data in [-0.5, 0.5)
            assert np.abs(out - acc).max() <= 1.0 / 255 / 2 + 1e-6


def test_ref_quantized_kv_sdpa_near_f32_attention():           # kv_quant.rs:568-650
    b, h, d = 1, 2, 16
    kc, vc = orc.KiviCache(True, running=True), orc.KiviCache(False, running=True)
    kf = vf = None

    def mk(base):
        return (np.float32(base) + np.sin(np.arange(b * h * d, dtype=np.float32) * np.float32(0.013))).astype(np.float32).reshape(b, h, 1, d)

    for t in range(10):
        qi, ki, vi = mk(9.0 + t * 0.1), mk(1.0 + t * 0.07), mk(5.0 - t * 0.05)
        kc.ingest(ki)
        vc.ingest(vi)
        got = orc.flash_sdpa(qi, kc.dequantized(), vc.dequantized(), causal=False)
        kf = ki if kf is None else orc.concat_append(kf, ki, 2)
        vf = vi if vf is None else orc.concat_append(vf, vi, 2)
        want = orc.naive_sdpa_f64(qi, kf, vf, causal=False).astype(np.float32)
        assert close_enough_super(got, want), t


def test_codes_by_a_product_equal_codes_by_the_division_away_from_the_boundaries():
    """The device codes (x - lo) * RN(1 / scale) instead of (x - lo) / scale and falls back to the division when the
    product's fraction is within 2^-13 of one half.  Here in numpy: on quotients placed on and a few floats beside the
    boundaries k + 1/2 and on random ones, for power-of-two and other scales, the two codes agree wherever the rule does
    not ask for the fallback, and without the rule they would differ somewhere (so the rule is needed)."""
    rng = np.random.default_rng(8)
    half = np.float32(0.49999997)
    differ = checked = 0
    for lv in (255, 15):
        scales = np.concatenate([[1.0, 3.0, 0.75, 1e-3, 7.0, 2.0 ** -20], rng.uniform(1e-3, 50.0, 200)]).astype(np.float32)
        for s in scales:
            sc = np.float32(np.float32(lv) * s / np.float32(lv))
            ks = rng.integers(0, lv, 256).astype(np.float32)
            vals = ((ks + np.float32(0.5)) * sc).astype(np.float32)
            for j in range(vals.size):
                steps = (j % 7) - 3
                for _ in range(abs(steps)):
                    vals[j] = np.nextafter(vals[j], np.float32(np.inf if steps > 0 else 0.0), dtype=np.float32)
            vals = np.concatenate([vals, rng.uniform(0, lv * float(sc), 256).astype(np.float32)])
            q = (vals / sc).astype(np.float32)
            exact = np.clip(np.trunc((q + np.copysign(half, q)).astype(np.float32)), 0, lv)
            q0 = (vals * np.float32(np.float32(1.0) / sc)).astype(np.float32)
            fast = np.clip(np.trunc((q0 + half).astype(np.float32)), 0, lv)
            near = np.abs((q0 - np.floor(q0)).astype(np.float32) - np.float32(0.5))
            safe = near >= np.float32(2.0 ** -13)
            assert (fast[safe] == exact[safe]).all(), (lv, s)
            differ += int((fast != exact).sum())
            checked += int(safe.sum())
    assert differ > 0 and checked > 50000
