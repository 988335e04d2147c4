"""Pins the oracle's f16 conversions and Q4_0 / Q8_0 / Q8_1 block quantisers against
facts that do not come from the oracle itself: numpy's IEEE half type, the
known-answer tests the reference holds (linalg/src/frame/block_quant/q4_0.rs:505-535,
589-593, 722-739; q8_1.rs:348-401) and byte strings derived by hand from the cited
lines."""
import numpy as np
import pytest

from oracle import oracle as orc


# ------------------------------------------------------------------ f16 conversions
def test_f16_to_f32_exhaustive_vs_numpy():
    bits = np.arange(65536, dtype=np.uint16)
    got = orc.f16_bits_to_f32(bits)
    want = bits.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))
    assert np.isnan(got[nan]).all()


def test_f32_to_f16_vs_numpy_rne():
    rng = np.random.default_rng(1)
    # every half value, the midpoints between neighbours (ties), and random bit patterns
    halves = np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32)
    halves = halves[np.isfinite(halves)]
    srt = np.sort(halves)
    mids = ((srt[:-1].astype(np.float64) + srt[1:].astype(np.float64)) / 2).astype(np.float32)
    rnd = rng.integers(0, 2**32, size=400000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    big = np.array([65504.0, 65519.99, 65520.0, 65536.0, 1e9, -1e9, 5.96e-8, 2.98e-8, 2.9802322e-8,
                    2.9802326e-8, 0.0, -0.0, np.inf, -np.inf], dtype=np.float32)
    x = np.concatenate([halves, mids, np.nextafter(mids, np.float32(np.inf)),
                        np.nextafter(mids, np.float32(-np.inf)), rnd, big])
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = orc.f32_to_f16_bits(x)
    nan = np.isnan(x)
    assert np.array_equal(got[~nan], want[~nan])
    assert np.isnan(got[nan].view(np.float16)).all()


# ------------------------------------------------------------------ Q4_0
def _cycle(fmt, x):
    return orc.dequant(fmt, orc.quant(fmt, x), x.dtype.type)


@pytest.mark.parametrize("dt", [np.float32, np.float16])
@pytest.mark.parametrize("head", [[1, 2, 3, 4], [-1, -2, -3, -4], [1234], [-1234]])
def test_q4_0_reference_round_trips(dt, head):
    # q4_0.rs:505-535: loop_q4f32_pos/neg, loop_q4f16_pos/neg, loop_q4_big_pos/neg
    x = np.zeros(32, dtype=dt)
    x[: len(head)] = head
    assert np.array_equal(_cycle(orc.FMT_Q4_0, x), x)


@pytest.mark.parametrize("dt", [np.float32, np.float16])
@pytest.mark.parametrize("fmt", [orc.FMT_Q4_0, orc.FMT_Q8_0])
def test_simulate_precision_loss_is_quant_then_dequant_in_the_tensors_type(fmt, dt):
    # block_quant/mod.rs:130-154; the reference's matmul tests build their expected values with it
    # (test-rt/suite-unit/src/matmul_q40.rs:119-126).  Checked here against the round trip spelled out per block
    # with the formulas of q4_0.rs:27-45,82-95 and q8_1.rs:36-63 in numpy.
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((3, 7, 64)) * 4).astype(dt)
    got = orc.simulate_precision_loss(fmt, x)
    assert got.shape == x.shape and got.dtype == x.dtype
    xb = x.astype(np.float32).reshape(-1, 32)
    first_max = np.abs(xb).argmax(axis=1)                                  # first index of the largest magnitude
    mx = xb[np.arange(len(xb)), first_max]
    if fmt == orc.FMT_Q4_0:
        d = (mx / np.float32(-8)).astype(np.float32)
        r = np.where(d == 0, np.float32(0), np.float32(1) / d).astype(np.float32)
        codes = np.minimum((xb * r[:, None] + np.float32(8.5)).astype(np.float32).astype(np.int8), 15).astype(np.float32) - 8
    else:
        d = (mx / np.float32(127)).astype(np.float32)
        r = np.where(d == 0, np.float32(0), np.float32(1) / d).astype(np.float32)
        t = (xb * r[:, None]).astype(np.float32)
        codes = np.trunc(t + np.copysign(np.float32(0.5), t)).astype(np.float32)   # f32::round: half away from zero
    d16 = d.astype(np.float16).astype(np.float32)
    want = (codes * d16[:, None]).astype(np.float32).astype(dt).reshape(x.shape)
    assert np.array_equal(got, want)


def test_q4_0_ramp_extracts_exactly():
    # q4_0.rs:589-593: ((i % 14) - 6) survives quant/dequant after .round()
    x = np.array([(i % 14) - 6 for i in range(64)], dtype=np.float32)
    assert np.array_equal(np.round(_cycle(orc.FMT_Q4_0, x)), x)


def test_q4_0_hand_derived_bytes():
    # [1,2,3,4,0..]: max=4 -> scale=-0.5 -> d=f16(-0.5)=0xB800; r=-2;
    # codes trunc(x*r+8.5) = 6,4,2,0 then 8; byte j = code(j) | code(j+16)<<4
    x = np.zeros(32, dtype=np.float32)
    x[:4] = [1, 2, 3, 4]
    want = bytes([0x00, 0xB8, 0x86, 0x84, 0x82, 0x80] + [0x88] * 12)
    assert orc.quant(orc.FMT_Q4_0, x).tobytes() == want
    # negative twin: scale=+0.5 -> d=0x3800, same code bytes
    want_neg = bytes([0x00, 0x38, 0x86, 0x84, 0x82, 0x80] + [0x88] * 12)
    assert orc.quant(orc.FMT_Q4_0, -x).tobytes() == want_neg
    # all-zero block: max=+0.0, scale = 0.0 / -8.0 = -0.0 (IEEE) -> d=0x8000, every code 8
    assert orc.quant(orc.FMT_Q4_0, np.zeros(32, np.float32)).tobytes() == bytes([0, 0x80] + [0x88] * 16)
    # Q8: 0.0 / 127.0 = +0.0 -> d=0x0000, codes 0
    assert orc.quant(orc.FMT_Q8_0, np.zeros(32, np.float32)).tobytes() == bytes(34)


def test_q4_0_nibble_order_and_dequant_table():
    # q4_0.rs:722-739 (pack_prequantized test): nibble i%16 at logical position i,
    # scales {0.5,0.25,1,2}: dequant must be exactly (q-8)*s.  Blocks are built by
    # hand here in the canonical layout (d, then byte j = q[j] | q[j+16]<<4).
    scales = [0.5, 0.25, 1.0, 2.0]
    raw = bytearray()
    want = []
    for s in scales:
        q = [i % 16 for i in range(32)]
        raw += np.float16(s).tobytes()
        raw += bytes(q[j] | (q[j + 16] << 4) for j in range(16))
        want += [(v - 8) * s for v in q]
    got = orc.dequant(orc.FMT_Q4_0, np.frombuffer(bytes(raw), dtype=np.uint8))
    assert np.array_equal(got, np.array(want, dtype=np.float32))


def test_q4_0_high_element_goes_to_high_nibble():
    # element 16 is the only non-zero: it must land in the HIGH nibble of byte 0.
    x = np.zeros(32, dtype=np.float32)
    x[16] = 8.0  # max=8 -> scale=-1 -> code(8) = trunc(-8+8.5)=0; zeros -> 8
    b = orc.quant(orc.FMT_Q4_0, x)
    assert b[2] == 0x08 and all(v == 0x88 for v in b[3:])
    x = np.zeros(32, dtype=np.float32)
    x[0] = 8.0
    b = orc.quant(orc.FMT_Q4_0, x)
    assert b[2] == 0x80 and all(v == 0x88 for v in b[3:])


def test_q4_0_first_strict_max_wins_and_clamp_15():
    # ties on |v| keep the FIRST element (amax < |v| is strict, q4_0.rs:29-34):
    # [-3, 3, ...]: max=-3 -> scale=0.375 -> +3 codes trunc(8+8.5)=16 -> min 15.
    x = np.zeros(32, dtype=np.float32)
    x[0], x[1] = -3.0, 3.0
    b = orc.quant(orc.FMT_Q4_0, x)
    assert b[:2].tobytes() == np.float16(0.375).tobytes()
    assert b[2] & 0xF == 0 and b[3] & 0xF == 15


def test_q4_0_special_values():
    # NaN never wins the max and codes to 0 (Rust `as i8` of NaN); inf -> scale inf
    x = np.zeros(32, dtype=np.float32)
    x[0], x[1] = np.nan, 2.0
    b = orc.quant(orc.FMT_Q4_0, x)
    assert b[:2].tobytes() == np.float16(-0.25).tobytes()
    assert b[2] & 0xF == 0  # NaN*r+8.5 = NaN -> 0


# ------------------------------------------------------------------ Q8_0 / Q8_1
def test_q8_hand_derived_bytes():
    # q8_1.rs:20-48: [1,2,3,4,0..]: scale=f32(4/127) -> d=0x2808; r=1/scale=31.75;
    # codes round_half_away(x*31.75) = 32, 64 (63.5 away from zero), 95, 127
    x = np.zeros(32, dtype=np.float32)
    x[:4] = [1, 2, 3, 4]
    q = orc.quant(orc.FMT_Q8_0, x)
    assert q[:2].tobytes() == bytes([0x08, 0x28])
    assert q[2:6].view(np.int8).tolist() == [32, 64, 95, 127] and not q[6:].any()
    # negative twin: the sign lives in the scale (signed max), codes identical
    q = orc.quant(orc.FMT_Q8_0, -x)
    assert q[:2].tobytes() == bytes([0x08, 0xA8])
    assert q[2:6].view(np.int8).tolist() == [32, 64, 95, 127]
    # Q8_1 = same d and codes with the block sum in between (sum=10 -> f16 0x4900)
    q1 = orc.quant(orc.FMT_Q8_1, x)
    assert q1[:2].tobytes() == bytes([0x08, 0x28]) and q1[2:4].tobytes() == np.float16(10).tobytes()
    assert q1[4:8].view(np.int8).tolist() == [32, 64, 95, 127]


def test_q8_0_is_q8_1_without_sum():
    rng = np.random.default_rng(3)
    for dt in (np.float32, np.float16):
        x = (rng.standard_normal(32 * 50) * 3).astype(dt)
        a = orc.quant(orc.FMT_Q8_0, x).reshape(-1, 34)
        b = orc.quant(orc.FMT_Q8_1, x).reshape(-1, 36)
        assert np.array_equal(a[:, :2], b[:, :2]) and np.array_equal(a[:, 2:], b[:, 4:])


def test_q8_1_f16_sum_is_serial_in_f16():
    # q8_1.rs:30-36 with T=f16: 2048 + 1 + 1 ... stays 2048 in f16 serial adds
    x = np.ones(32, dtype=np.float16)
    x[0] = 2048
    s = orc.quant(orc.FMT_Q8_1, x)[2:4].view(np.float16)[0]
    assert s == np.float16(2048)
    s32 = orc.quant(orc.FMT_Q8_1, x.astype(np.float32))[2:4].view(np.float16)[0]
    assert s32 == np.float16(2048 + 31)  # f32 sum 2079 -> f16 RNE = 2080
    assert float(s32) == 2080.0


@pytest.mark.parametrize("dt", [np.float32, np.float16])
def test_q8_round_trip_tolerance(dt):
    # q8_1.rs:348-401 style: |x - dq(q(x))| <= |scale|/2 (+ f16 rounding of the scale)
    rng = np.random.default_rng(4)
    x = rng.standard_normal((64, 32)).astype(dt)
    y = _cycle(orc.FMT_Q8_0, x).astype(np.float32)
    amax = np.abs(x.astype(np.float32)).max(axis=1, keepdims=True)
    assert (np.abs(y - x.astype(np.float32)) <= amax / 127 * 0.5 + amax * 2e-3).all()


@pytest.mark.parametrize("fmt", [orc.FMT_Q4_0, orc.FMT_Q8_0])
def test_codes_match_closed_form_numpy(fmt):
    """Independent vectorised numpy-f32 derivation of the stored bytes."""
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((200, 32)) * rng.choice([1e-3, 1, 20], size=(200, 1))).astype(np.float32)
    idx = np.abs(x).argmax(axis=1)  # first index of the largest |v|
    mx = x[np.arange(200), idx]
    div = np.float32(-8.0) if fmt == orc.FMT_Q4_0 else np.float32(127.0)
    scale = (mx / div).astype(np.float32)
    with np.errstate(divide="ignore"):
        r = np.where(scale == 0, np.float32(0), np.float32(1) / scale).astype(np.float32)
    got = orc.quant(fmt, x)
    assert np.array_equal(got[:, :2].copy().view(np.float16)[:, 0], scale.astype(np.float16))
    if fmt == orc.FMT_Q4_0:
        t = ((x * r[:, None]).astype(np.float32) + np.float32(8.5)).astype(np.float32)
        codes = np.minimum(np.trunc(t).astype(np.int32), 15).astype(np.uint8)
        want = codes[:, :16] | (codes[:, 16:] << 4)
        assert np.array_equal(got[:, 2:], want)
    else:
        p = (x * r[:, None]).astype(np.float32)
        codes = (np.sign(p) * np.floor(np.abs(p) + np.float32(0.5))).astype(np.int8)
        assert np.array_equal(got[:, 2:].view(np.int8), codes)


def test_f16_dequant_rounds_product_to_f16():
    # q4_0.rs:82-95 with T=f16: (nibble-8)*d rounded to f16
    raw = np.float16(0.1).tobytes() + bytes([0x0F] * 16)  # low nibble 15 -> 7*d, high 0 -> -8*d
    got = orc.dequant(orc.FMT_Q4_0, np.frombuffer(raw, dtype=np.uint8), np.float16)
    d = np.float32(np.float16(0.1))
    assert got[0] == np.float16(np.float32(7) * d) and got[16] == np.float16(np.float32(-8) * d)


def test_round_half_away_as_one_addition_and_a_truncation():
    """The quantising kernels round with trunc(x + copysign(0.49999997, x)) (three instructions); this is f32::round
    for every float.  Checked here on every mantissa of the exponents 2^-2 .. 2^8 (the range of the codes) and on
    the ties, huge values, infinities and NaN; the exponents up to 2^24 were compared the same way when it was written."""
    h = np.nextafter(np.float32(0.5), np.float32(0))
    assert h == np.float32(0.49999997)

    def dev(x):
        return np.trunc((x + np.copysign(h, x)).astype(np.float32))

    for e in range(-2, 9):
        base = np.float32(2.0 ** e).view(np.uint32)
        x = np.arange(base, base + (1 << 23), dtype=np.uint32).view(np.float32)
        want = np.floor(x.astype(np.float64) + 0.5)
        assert np.array_equal(dev(x).astype(np.float64), want)
        assert np.array_equal(dev(-x).astype(np.float64), -want)
    ties = np.arange(0, 300, dtype=np.float32) + np.float32(0.5)
    assert np.array_equal(dev(ties), ties + np.float32(0.5)) and np.array_equal(dev(-ties), -ties - np.float32(0.5))
    assert dev(np.float32(0.49999997)) == 0 and dev(np.float32(-0.49999997)) == 0
    big = np.array([2.0 ** 23 + 1, 2.0 ** 24, 3e38, np.inf, -np.inf], np.float32)
    assert np.array_equal(dev(big), big) and np.isnan(dev(np.float32(np.nan)))
