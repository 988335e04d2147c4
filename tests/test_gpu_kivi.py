"""KIVI-style quantised caches on the GPU against the oracle (oracle/kivi_oracle.c): stored codes, parameters,
sink and partial-block rows and the dequantised cache bit-exact; the fused QuantizedKvSdpa within the path's
attention tolerance (1e-3 in f32, 2e-2 in f16).  The reference's own unit tests are replayed on the device ops."""
import ctypes as C

import numpy as np
import pytest

import tract_amd
from tract_amd import kivi
from oracle import oracle as orc
from tests.gpu_util import max_abs, rt  # noqa: F401
from tests.test_oracle_kivi import close_enough_super, lcg, take

pytestmark = pytest.mark.gpu


def same_state(gpu: dict, cpu: dict, where=""):
    for key in ("sink", "packed", "residual"):
        assert gpu[key].shape == cpu[key].shape, (where, key, gpu[key].shape, cpu[key].shape)
        assert gpu[key].tobytes() == cpu[key].tobytes(), (where, key)
    for key in ("lo", "scale"):
        # numerically equal (a zero `lo` may differ in sign: the CPU op leaves min(+0, -0) to the platform)
        g, c = gpu[key].reshape(-1), cpu[key].reshape(-1)
        assert g.shape == c.shape, (where, key)
        assert np.array_equal(g, c, equal_nan=True), (where, key)


@pytest.mark.parametrize("dt", [np.float32, np.float16])
@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("per_channel", [False, True])
def test_quantized_dyn_kv_cache_state_and_output_equal_the_oracle(rt, dt, bits, per_channel):
    rng = np.random.default_rng(bits + 10 * per_channel)
    B, H, D = 2, 3, 64
    op = tract_amd.QuantizedDynKeyValueCache("kv0", 2, bits, per_channel)
    st = op.state()
    ref = orc.KiviCache(per_channel, bits)
    outliers = rng.choice([1.0, 1.0, 1.0, 20.0], D)
    for step, n in enumerate([1, 2, 3, 1, 30, 1, 1, 64, 5, 100, 1, 27, 32, 1]):
        x = (rng.standard_normal((B, H, n, D)) * outliers).astype(dt)
        out = st.eval(x).to_numpy()
        ref.ingest(x)
        want = ref.dequantized().astype(dt)            # cast_to_dt(input_dt): round to nearest even
        assert out.shape == want.shape and out.dtype == dt
        assert out.tobytes() == want.tobytes(), f"step {step}"
        same_state(st.cache.state(), ref.state(), f"step {step}")
        assert st.resolve_symbols() == ref.length
    c = st.cache.counts()
    assert c["n_sink"] == 4 and c["row_bytes"] == D * bits // 8
    if per_channel:
        assert c["n_rows"] == (ref.length - 4) // 32 * 32 and c["n_res"] == (ref.length - 4) % 32


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("per_channel", [False, True])
def test_quotients_on_and_beside_the_rounding_boundaries(rt, bits, per_channel):
    """Values whose quotient (x - lo) / scale is exactly k + 1/2, or one to three floats beside it, for scales that are
    and are not powers of two, and scales outside the range where a reciprocal may stand in for the division: the codes
    must be the ones the division gives (the device codes most elements by a product and falls back near a boundary)."""
    rng = np.random.default_rng(bits)
    D, lv = 128, (1 << bits) - 1
    n_groups = 64
    scales = np.concatenate([[1.0, 3.0, 0.75, 1e-3, 7.0, 2.0 ** -20, 1e30, 1e-38, 3e-41, 1e38 / lv],
                             rng.uniform(1e-3, 50.0, n_groups - 10)]).astype(np.float32)
    # a group: lo = 0, hi = lv * s (so that scale = RN(hi / lv), close to s), 126 more values at and around the boundaries
    groups = np.zeros((n_groups, D), np.float32)
    for gi, s in enumerate(scales):
        hi = np.float32(lv) * s
        sc = np.float32(hi / np.float32(lv)) if np.isfinite(hi) and hi > 0 else np.float32(1.0)
        ks = rng.integers(0, lv, D - 2).astype(np.float32)
        with np.errstate(over="ignore", invalid="ignore"):
            vals = ((ks + np.float32(0.5)) * sc).astype(np.float32)
            for j in range(D - 2):
                steps = (j % 7) - 3
                for _ in range(abs(steps)):
                    vals[j] = np.nextafter(vals[j], np.float32(np.inf if steps > 0 else 0.0), dtype=np.float32)
            vals = np.clip(np.nan_to_num(vals, nan=0.0, posinf=float(hi), neginf=0.0), 0.0, hi)
        groups[gi, 0], groups[gi, 1], groups[gi, 2:] = 0.0, hi, vals
    if per_channel:     # a group is a channel over one 32-token block: blocks [32, D] with D groups side by side
        n_blocks = n_groups * D // (32 * D) * 4
        x = np.zeros((1, 1, 4 + 32 * n_blocks, D), np.float32)
        flat = groups.reshape(-1)
        for b in range(n_blocks):
            for c in range(D):
                g = groups[(b * D + c) % n_groups]
                x[0, 0, 4 + 32 * b:4 + 32 * (b + 1), c] = np.concatenate([g[:2], g[2 + (b * 30) % 96:2 + (b * 30) % 96 + 30]])
    else:               # a group is a token
        x = np.concatenate([np.zeros((4, D), np.float32), groups]).reshape(1, 1, 4 + n_groups, D)
    st = tract_amd.QuantizedDynKeyValueCache("kv", 2, bits, per_channel).state()
    ref = orc.KiviCache(per_channel, bits)
    out = st.eval(x).to_numpy()
    ref.ingest(x)
    same_state(st.cache.state(), ref.state(), f"bits={bits} per_channel={per_channel}")
    assert out.tobytes() == ref.dequantized().tobytes()


@pytest.mark.parametrize("D", [8, 16, 3, 130])
def test_odd_head_sizes_and_tiny_caches(rt, D):
    rng = np.random.default_rng(D)
    for per_channel in (False, True):
        for bits in (4, 8):
            st = tract_amd.QuantizedDynKeyValueCache("c", 2, bits, per_channel).state()
            ref = orc.KiviCache(per_channel, bits)
            for n in (1, 1, 1, 1, 1, 31, 1, 40):
                x = rng.standard_normal((1, 2, n, D)).astype(np.float32)
                out = st.eval(x).to_numpy()
                ref.ingest(x)
                assert out.tobytes() == ref.dequantized().tobytes()
            same_state(st.cache.state(), ref.state(), f"D={D} bits={bits} per_channel={per_channel}")


def test_nan_inf_and_constant_rows(rt):
    D = 32
    x = np.random.default_rng(0).standard_normal((1, 1, 4 + 64, D)).astype(np.float32)
    x[0, 0, 5, 3] = np.nan
    x[0, 0, 6, :] = np.nan
    x[0, 0, 7, 2] = np.inf
    x[0, 0, 8, 9] = -np.inf
    x[0, 0, 9, :] = 2.5
    x[0, 0, 40, 1] = np.nan
    x.view(np.uint32)[0, 0, 42, 2] = 0x7FA00000   # signalling NaNs: skipped like the quiet ones, in a token and in a channel
    x[0, 0, 42, 3], x[0, 0, 42, 1] = 50.0, -60.0
    x.view(np.uint32)[0, 0, 50, 7] = 0xFFA00001
    x[0, 0, 49, 7], x[0, 0, 51, 7] = 70.0, -80.0
    x[0, 0, 41, 2] = np.inf
    for per_channel in (False, True):
        for bits in (4, 8):
            st = tract_amd.QuantizedDynKeyValueCache("c", 2, bits, per_channel).state()
            ref = orc.KiviCache(per_channel, bits)
            out = st.eval(x).to_numpy()
            ref.ingest(x)
            assert out.tobytes() == ref.dequantized().tobytes(), (per_channel, bits)
            same_state(st.cache.state(), ref.state())


def test_load_from_save_to_freeze(rt):
    rng = np.random.default_rng(3)
    x = rng.standard_normal((1, 2, 50, 16)).astype(np.float32)
    st = tract_amd.QuantizedDynKeyValueCache("c", 2, 8, True).state()
    st.load_from([x])                                    # quant_dyn_kv_cache.rs:455-465
    assert st.resolve_symbols() == 50
    saved = []
    st.save_to(saved)                                    # :467-470: the dequantised cache
    ref = orc.KiviCache(True, 8)
    ref.ingest(x)
    assert saved[0].tobytes() == ref.dequantized().tobytes()
    frozen = st.freeze()                                 # :510-541
    y = rng.standard_normal((1, 2, 20, 16)).astype(np.float32)
    a = st.eval(y).to_numpy()
    assert frozen.resolve_symbols() == 50                # the copy did not move
    b = frozen.unfreeze().eval(y).to_numpy()
    ref.ingest(y)
    assert a.tobytes() == b.tobytes() == ref.dequantized().tobytes()
    with pytest.raises(tract_amd.TractRocmError, match="cache shape changed between steps"):
        st.eval(np.zeros((1, 3, 1, 16), np.float32))
    with pytest.raises(tract_amd.TractRocmError, match="rank-4"):
        tract_amd.QuantizedDynKeyValueCache("c", 2, 8, True).state().eval(np.zeros((2, 1, 16), np.float32))
    with pytest.raises(tract_amd.TractRocmError, match="bits must be 4 or 8"):
        tract_amd.QuantizedDynKeyValueCache("c", 2, 3, True)


# ---- the reference's unit tests on the device ops -----------------------------------------------------------------
def test_ref_quant_dequant_cases(rt):
    x = np.array([[0, 1, 2, 3], [-1, 0.5, 4, 9], [2, 2, 2, 2.1]], np.float32)       # kv_quant.rs:454-478
    for bits in (4, 8):
        for by_row in (False, True):
            assert kivi.quant_dequant(x, bits, by_row).tobytes() == orc.kivi_quant_dequant(x, bits, by_row).tobytes()
    e4 = np.abs(x - kivi.quant_dequant(x, 4, False)).max()
    e8 = np.abs(x - kivi.quant_dequant(x, 8, False)).max()
    assert e8 < e4
    x = np.array([[100, 0.10, -0.20, 0.05], [-90, 0.02, 0.30, -0.08], [120, -0.15, 0.10, 0.20],    # :483-505
                  [-110, 0.07, -0.05, 0.12]], np.float32)
    pc = np.abs(x - kivi.quant_dequant(x, 4, False))[:, 1:].max()
    pt = np.abs(x - kivi.quant_dequant(x, 4, True))[:, 1:].max()
    assert pc < pt * 0.2


def test_ref_quant_cache_accumulates_near_lossless_int8(rt):   # quant_dyn_kv_cache.rs:728-756
    for per_channel in (False, True):
        gen = lcg(3)
        st = tract_amd.QuantizedDynKeyValueCache("kv0", 2, 8, per_channel).state()
        acc = None
        for _ in range(40):
            step = take(gen, 1, 2, 1, 8)
            out = st.eval(step).to_numpy()
            acc = step if acc is None else np.concatenate([acc, step], axis=2)
            assert out.shape == acc.shape and close_enough_super(out, acc)


def test_ref_block_per_channel_key_consistent_over_growing_range(rt):   # quant_dyn_kv_cache.rs:758-778
    d = 16
    rows = np.array([[t * 2.0 if c == 0 else np.sin(np.float32((t * 7 + c) * 0.013)) * 0.1 for c in range(d)]
                     for t in range(80)], np.float32)
    st = tract_amd.QuantizedDynKeyValueCache("k", 2, 8, True).state()
    for r in rows:
        out = st.eval(r.reshape(1, 1, 1, d))
    assert st.resolve_symbols() == 80
    assert np.abs(out.to_numpy()[0, 0] - rows).max() < 1.0


def test_ref_quantized_kv_sdpa_runs_in_model(rt):              # kv_quant.rs:568-650
    b, h, d = 1, 2, 16
    st = tract_amd.QuantizedKvSdpa(axis=2, scale=None).state()
    kc, vc = orc.KiviCache(True, running=True), orc.KiviCache(False, running=True)
    kf = vf = None

    def mk(base):
        return (np.float32(base) + np.sin(np.arange(b * h * d, dtype=np.float32) * np.float32(0.013))).astype(np.float32).reshape(b, h, 1, d)

    for t in range(10):
        qi, ki, vi = mk(9.0 + t * 0.1), mk(1.0 + t * 0.07), mk(5.0 - t * 0.05)
        got = st.eval([qi, ki, vi]).to_numpy()
        kf = ki if kf is None else np.concatenate([kf, ki], axis=2)
        vf = vi if vf is None else np.concatenate([vf, vi], axis=2)
        want = orc.naive_sdpa_f64(qi, kf, vf, causal=False).astype(np.float32)
        assert close_enough_super(got, want), t
        kc.ingest(ki)
        vc.ingest(vi)
        assert max_abs(got, orc.flash_sdpa(qi, kc.dequantized(), vc.dequantized(), causal=False)) <= 1e-3
    same_state(st.k.state(), kc.state(), "K")
    same_state(st.v.state(), vc.state(), "V")
    assert st.k.memory_bytes() == b * h * (10 * d + d * 8) and st.v.memory_bytes() == b * h * (10 * d + 10 * 8)


@pytest.mark.parametrize("dt,tol", [(np.float32, 1e-3), (np.float16, 2e-2)])
def test_quantized_kv_sdpa_gqa_prefill_then_decode(rt, dt, tol):
    rng = np.random.default_rng(11)
    B, Hq, Hkv, D = 2, 8, 2, 128
    st = tract_amd.QuantizedKvSdpa(axis=2, scale=0.11).state()
    kc, vc = orc.KiviCache(True, running=True), orc.KiviCache(False, running=True)
    chan = rng.choice([1.0, 1.0, 1.0, 20.0], D)
    for n in (37, 1, 1, 8, 1, 200, 1):
        q = (rng.standard_normal((B, Hq, n, D)) / np.sqrt(D)).astype(dt)
        k = (rng.standard_normal((B, Hkv, n, D)) * chan).astype(dt)
        v = rng.standard_normal((B, Hkv, n, D)).astype(dt)
        got = st.eval([q, k, v]).to_numpy()
        kc.ingest(k)
        vc.ingest(v)
        want = orc.flash_sdpa(q.astype(np.float32), kc.dequantized(), vc.dequantized(), causal=False, scale=0.11)   # kv_quant.rs:326
        assert got.dtype == dt and max_abs(got, want) <= tol, n
    same_state(st.k.state(), kc.state(), "K")
    same_state(st.v.state(), vc.state(), "V")
    frozen = st.freeze()
    q = (rng.standard_normal((B, Hq, 1, D)) / np.sqrt(D)).astype(dt)
    k = rng.standard_normal((B, Hkv, 1, D)).astype(dt)
    assert st.eval([q, k, k]).to_numpy().tobytes() == frozen.eval([q, k, k]).to_numpy().tobytes()


@pytest.mark.parametrize("B,Hq,Hkv,T0", [(4, 32, 8, 4100), (1, 32, 8, 8192), (2, 32, 2, 1500), (3, 6, 2, 700)])
def test_quantized_kv_sdpa_decode_steps_over_the_codes(rt, B, Hq, Hkv, T0):
    """One f16 query token per step at head_dim 128: attention runs straight over the u8 codes (key features scaled
    once per launch, token scales folded into the probabilities), several key splits merged in the kernel.  Sampled kv
    heads against the oracle's attention over its dequantised stores; the stores stay bit-exact."""
    rng = np.random.default_rng(T0)
    D, g = 128, Hq // Hkv
    st = tract_amd.QuantizedKvSdpa(axis=2, scale=None).state()
    chan = rng.choice([1.0, 1.0, 1.0, 20.0], D)
    k0 = (rng.standard_normal((B, Hkv, T0, D)) * chan).astype(np.float16)
    v0 = rng.standard_normal((B, Hkv, T0, D)).astype(np.float16)
    v0[:, :, 5::97] += 40.0                      # tokens whose lo dominates
    v0[:, :, 11::131] = np.float16(-3.25)        # constant tokens: hi == lo, scale 1
    q0 = (rng.standard_normal((B, Hq, T0, D)) / np.sqrt(D)).astype(np.float16)
    st.eval([q0, k0, v0])
    sample = sorted({(0, 0), (B - 1, Hkv - 1), (B // 2, Hkv // 2)})
    refs = {}
    for (b, h) in sample:
        kc, vc = orc.KiviCache(True, running=True), orc.KiviCache(False, running=True)
        kc.ingest(k0[b:b + 1, h:h + 1])
        vc.ingest(v0[b:b + 1, h:h + 1])
        refs[(b, h)] = (kc, vc)
    worst = 0.0
    for step in range(4):
        q = (rng.standard_normal((B, Hq, 1, D)) * (3.0 if step == 2 else 1.0) / np.sqrt(D)).astype(np.float16)
        k = (rng.standard_normal((B, Hkv, 1, D)) * chan * (1.0 if step != 1 else 4.0)).astype(np.float16)   # step 1 widens the key ranges
        v = rng.standard_normal((B, Hkv, 1, D)).astype(np.float16)
        got = st.eval([q, k, v]).to_numpy()
        assert got.dtype == np.float16 and got.shape == (B, Hq, 1, D)
        for (b, h), (kc, vc) in refs.items():
            kc.ingest(k[b:b + 1, h:h + 1])
            vc.ingest(v[b:b + 1, h:h + 1])
            want = orc.flash_sdpa(q[b:b + 1, h * g:(h + 1) * g].astype(np.float32), kc.dequantized(), vc.dequantized(), causal=False)
            err = max_abs(got[b:b + 1, h * g:(h + 1) * g], want)
            worst = max(worst, err)
            assert err <= 2e-2, (step, b, h, err)
    state_k, state_v = st.k.state(), st.v.state()
    for (b, h), (kc, vc) in refs.items():
        i = b * Hkv + h
        same_state({n: a[i:i + 1] for n, a in state_k.items()}, kc.state(), f"K {b},{h}")
        same_state({n: a[i:i + 1] for n, a in state_v.items()}, vc.state(), f"V {b},{h}")
    assert worst <= 8e-3, worst   # what f16 outputs and f16 probabilities leave


def test_cache_of_the_decode_layer_shape(rt):
    """32q/8kv, d=128 at batch 8: a 2048-token prefill and decode steps; sampled heads against the oracle."""
    rng = np.random.default_rng(2)
    B, H, D, T = 8, 8, 128, 2048
    x = rng.standard_normal((B, H, T, D)).astype(np.float16)
    x[:, :, :, 5] *= 20
    for per_channel in (False, True):
        st = tract_amd.QuantizedDynKeyValueCache("kv", 2, 8, per_channel).state()
        out = st.eval(x).to_numpy()
        steps = [rng.standard_normal((B, H, 1, D)).astype(np.float16) for _ in range(3)]
        for s in steps:
            out = st.eval(s).to_numpy()
        assert out.shape == (B, H, T + 3, D)
        state = st.cache.state()
        for (b, h) in ((0, 0), (3, 5), (7, 7)):
            ref = orc.KiviCache(per_channel, 8)
            ref.ingest(x[b:b + 1, h:h + 1])
            for s in steps:
                ref.ingest(s[b:b + 1, h:h + 1])
            assert out[b, h].tobytes() == ref.dequantized()[0, 0].astype(np.float16).tobytes()
            same_state({k: v[b * H + h:b * H + h + 1] for k, v in state.items()}, ref.state(), f"head {b},{h}")


def test_running_key_store_prompt_push_equals_token_by_token(rt):
    """A long run of tokens takes the chunked scan (three passes over 64-token chunks); its codes and parameters are
    those of the token-by-token push, also on top of earlier state, with NaN, infinities and signed zeros in the data."""
    rng = np.random.default_rng(8)
    B, H, D = 1, 3, 40
    cache = kivi.KiviCache(kivi.KIVI_RUNNING_CHANNEL, 8, 0, B, H, D)
    ref = orc.KiviCache(True, running=True)
    for n, mag in ((5, 1.0), (300, 1.0), (1, 1.0), (1000, 3.0), (256, 0.1), (257, 30.0)):
        x = (rng.standard_normal((B, H, n, D)) * mag).astype(np.float32)
        x[0, 0, n // 2, 3] = np.nan
        x[0, 1, n // 3, 4] = 0.0
        x[0, 1, n // 3 + 1 if n > 1 else 0, 4] = -0.0
        if n > 600:
            x[0, 2, 600, 7] = np.inf
            x[0, 2, 100:200, 9] = np.linspace(5, -50, 100)     # the minimum keeps moving inside and across chunks
            x[0, 2, 200:, 9] = np.linspace(-50, 400, n - 200)  # then the range keeps growing
        cache.append(x)
        ref.ingest(x)
        got, want = cache.state(), ref.state()
        assert got["packed"].tobytes() == want["packed"].tobytes(), n
        assert got["lo"].tobytes() == want["lo"].tobytes() and got["scale"].tobytes() == want["scale"].tobytes(), n
    assert cache.dequantize(np.float32).to_numpy().tobytes() == ref.dequantized().tobytes()


@pytest.mark.parametrize("D,dt", [(128, np.float16), (128, np.float32), (64, np.float16), (256, np.float32)])
def test_running_key_store_prompt_push_with_128_bit_rows(rt, D, dt):
    """Head sizes 64 / 128 / 256 take the chunk passes in which a lane owns 8 channels and rows move as 128-bit words:
    the same codes and parameters as the token-by-token push, over several prompts, on top of earlier state, with a
    ragged last chunk, NaN, infinities, signed zeros and a minimum / range that keep moving."""
    rng = np.random.default_rng(D)
    B, H = 2, 3
    cache = kivi.KiviCache(kivi.KIVI_RUNNING_CHANNEL, 8, 0, B, H, D)
    refs = {(b, h): orc.KiviCache(True, running=True) for b in range(B) for h in (0, H - 1)}
    # (chunk counts 11, 5, 16, 35 and 49: the scan of the chunk results walks whole groups of 16 chunks, pairs of groups, and a tail)
    for n, mag in ((3, 1.0), (700, 1.0), (1, 1.0), (257, 4.0), (1024, 0.2), (2200, 1.0), (3100, 2.0)):
        x = (rng.standard_normal((B, H, n, D)) * mag).astype(dt)
        x[0, 0, n // 2, 3] = np.nan
        x[1, H - 1, n // 3, D - 1] = 0.0
        x[1, H - 1, n // 3 + 1 if n > 1 else 0, D - 1] = -0.0
        if n > 600:
            x[0, H - 1, 600, 7] = np.inf
            x[0, H - 1, 100:200, 9] = np.linspace(5, -50, 100).astype(dt)
            x[0, H - 1, 200:, 9] = np.linspace(-50, 400, n - 200).astype(dt)
        cache.append(x)
        got = cache.state()
        for (b, h), ref in refs.items():
            ref.ingest(x[b:b + 1, h:h + 1].astype(np.float32))
            want, i = ref.state(), b * H + h
            assert got["packed"][i:i + 1].tobytes() == want["packed"].tobytes(), (n, b, h)
            assert got["lo"][i:i + 1].tobytes() == want["lo"].tobytes() and got["scale"][i:i + 1].tobytes() == want["scale"].tobytes(), (n, b, h)


def test_growing_stores_then_attention_without_a_host_sync(rt):
    """A prompt into the running Key store and the per-token Value store, then decode steps that grow both stores,
    all queued behind other work on one stream: no call waits for the stream (growth and the prompt's scratch
    release their old memory behind events), and the state is what the synchronous order gives."""
    import time
    from tract_amd.runtime import Stream
    B, Hq, Hkv, D, T = 1, 8, 2, 128, 300
    rng = np.random.default_rng(12)
    k = rng.standard_normal((B, Hkv, T, D), dtype=np.float32).astype(np.float16)
    v = rng.standard_normal((B, Hkv, T, D), dtype=np.float32).astype(np.float16)
    steps = [(rng.standard_normal((B, Hq, 1, D), dtype=np.float32).astype(np.float16) * np.float16(0.1),
              rng.standard_normal((B, Hkv, 1, D), dtype=np.float32).astype(np.float16),
              rng.standard_normal((B, Hkv, 1, D), dtype=np.float32).astype(np.float16)) for _ in range(40)]
    stream = Stream()
    ref_state = kivi.QuantizedKvSdpa(axis=2).state()
    qp = rng.standard_normal((B, Hq, T, D), dtype=np.float32).astype(np.float16) * np.float16(0.1)
    want = [ref_state.eval([qp, k, v]).to_numpy()] + [ref_state.eval(list(s)).to_numpy() for s in steps]
    tract_amd.synchronize()
    st = kivi.QuantizedKvSdpa(axis=2).state()
    from tract_amd.runtime import Workspace
    st._ws = Workspace(B, Hq, T, D, stream)   # (the host mirror synchronises when it makes a workspace: made ahead of the queue)
    dev = [tract_amd.DeviceTensor.from_numpy(a, stream) for a in (qp, k, v)]
    dsteps = [[tract_amd.DeviceTensor.from_numpy(a, stream) for a in s] for s in steps]
    big = tract_amd.DeviceTensor((1 << 30,), np.uint8)   # 1 GiB, one half copied onto the other many times: ~60 ms of queued work
    half = 1 << 29
    shape, st1 = (C.c_int64 * 1)(half // 16), (C.c_int64 * 1)(1)
    stream.synchronize()
    from tract_amd._lib import call
    for _ in range(300):
        call("trocm_copy_nd", big.ptr, half, st1, big.ptr, 0, st1, shape, 1, 16, stream.handle)
    t0 = time.perf_counter()
    got = [st.eval(dev, stream=stream)] + [st.eval(s, stream=stream) for s in dsteps]   # 300 + 40 tokens: both stores double several times
    queued = time.perf_counter() - t0
    stream.synchronize()
    total = time.perf_counter() - t0
    assert queued < 0.5 * total, (queued, total)   # the calls returned while the stream was still busy
    for g, w in zip(got, want):
        assert g.to_numpy().tobytes() == w.tobytes()
    a, b = st.k.state(), ref_state.k.state()
    assert all(a[n].tobytes() == b[n].tobytes() for n in a)


def test_a_refused_append_changes_nothing_and_can_be_repeated(rt):
    """An append that cannot get its memory (more than the device has) fails before anything is counted: length, sink
    and row counts stay, and the next append works.  The same for a QuantizedKvSdpa step: K and V stay level."""
    import ctypes as C2
    from tract_amd._lib import load
    lib = load()
    B, H, D = 8, 512, 512                       # 4096 (batch, head) rows of 512 channels
    hbm = C2.c_size_t()
    assert lib.trocm_device_info(None, C2.byref(hbm), None, 0) == 0
    n_huge = (1 << 31) // D - 64                # the index range's limit: 4096 x 4 Mi x 512 bytes of codes = 8.8 TB
    assert B * H * n_huge * D > 4 * hbm.value
    for layout, bits, sink in ((kivi.KIVI_PER_TOKEN, 8, 4), (kivi.KIVI_BLOCK_CHANNEL, 4, 4), (kivi.KIVI_RUNNING_CHANNEL, 8, 0)):
        cache = kivi.KiviCache(layout, bits, sink, B, H, D)
        x = np.random.default_rng(1).standard_normal((B, H, 2, D)).astype(np.float32)
        cache.append(x)
        before = (cache.len(), cache.counts())
        small = tract_amd.DeviceTensor.from_numpy(x)   # never read: the call fails while it allocates
        assert lib.trocm_kivi_cache_append(cache.handle, small.ptr, 0, n_huge, None) == 1
        assert b"failed" in lib.trocm_last_error() or b"hipMalloc" in lib.trocm_last_error() or b"memory" in lib.trocm_last_error()
        assert (cache.len(), cache.counts()) == before
        cache.append(x)
        assert cache.len() == 4
    kc = kivi.KiviCache(kivi.KIVI_RUNNING_CHANNEL, 8, 0, B, H, D)
    vc = kivi.KiviCache(kivi.KIVI_PER_TOKEN, 8, 0, B, H, D)
    q = tract_amd.DeviceTensor.from_numpy(np.zeros((B, H, 1, D), np.float32))
    out = tract_amd.DeviceTensor((B, H, 1, D), np.float32)
    kn = tract_amd.DeviceTensor.from_numpy(np.ones((B, H, 1, D), np.float32))
    nan = C2.c_float(float("nan"))
    assert lib.trocm_quantized_kv_sdpa_eval(q.ptr, kn.ptr, kn.ptr, 0, H, 1, kc.handle, vc.handle, out.ptr, nan, None, 0, None) == 0
    assert lib.trocm_quantized_kv_sdpa_eval(q.ptr, kn.ptr, kn.ptr, 0, H, n_huge, kc.handle, vc.handle, out.ptr, nan, None, 0, None) == 1
    assert kc.len() == 1 and vc.len() == 1 and kc.counts() == {**kc.counts(), "n_rows": 1} and vc.counts()["n_rows"] == 1
    assert lib.trocm_quantized_kv_sdpa_eval(q.ptr, kn.ptr, kn.ptr, 0, H, 1, kc.handle, vc.handle, out.ptr, nan, None, 0, None) == 0
    assert kc.len() == 2 and vc.len() == 2


@pytest.mark.parametrize("k_mag,v_mag", [(1.0, 1e-3), (1.0, 1e-5), (1e-3, 1.0), (1e-3, 1e-4), (30.0, 200.0)])
def test_quantized_kv_sdpa_over_the_codes_with_small_and_large_magnitudes(rt, k_mag, v_mag):
    """Keys and Values far from unit magnitude: their scales (range / 255) fall below the smallest normal half, or grow
    large.  The products q * s_k and P * s_v that the matrix cores take as halves are first brought into range by a
    power of two, so the output keeps the accuracy it has at unit magnitude, relative to its own size.  Some tokens are
    20x larger than the rest, and come late, so that the running factor of the Values has to move."""
    rng = np.random.default_rng(5)
    B, Hq, Hkv, D, T0 = 2, 8, 2, 128, 1000
    g = Hq // Hkv
    st = tract_amd.QuantizedKvSdpa(axis=2, scale=None).state()
    k0 = (rng.standard_normal((B, Hkv, T0, D)) * k_mag).astype(np.float16)
    v0 = (rng.standard_normal((B, Hkv, T0, D)) * v_mag).astype(np.float32)
    v0[:, :, 700::50] *= 20.0
    v0 = v0.astype(np.float16)
    q_mag = 1.0 / (np.sqrt(D) * k_mag)    # logits of unit size whatever the keys' magnitude
    q0 = (rng.standard_normal((B, Hq, T0, D)) * q_mag).astype(np.float16)
    st.eval([q0, k0, v0])
    refs = {}
    for (b, h) in ((0, 0), (1, 1)):
        kc, vc = orc.KiviCache(True, running=True), orc.KiviCache(False, running=True)
        kc.ingest(k0[b:b + 1, h:h + 1])
        vc.ingest(v0[b:b + 1, h:h + 1])
        refs[(b, h)] = (kc, vc)
    for step in range(3):
        q = (rng.standard_normal((B, Hq, 1, D)) * q_mag).astype(np.float16)
        k = (rng.standard_normal((B, Hkv, 1, D)) * k_mag).astype(np.float16)
        v = (rng.standard_normal((B, Hkv, 1, D)) * v_mag).astype(np.float16)
        got = st.eval([q, k, v]).to_numpy().astype(np.float64)
        for (b, h), (kc, vc) in refs.items():
            kc.ingest(k[b:b + 1, h:h + 1])
            vc.ingest(v[b:b + 1, h:h + 1])
            want = orc.flash_sdpa(q[b:b + 1, h * g:(h + 1) * g].astype(np.float32), kc.dequantized(), vc.dequantized(), causal=False).astype(np.float64)
            size = float(np.abs(want).max())
            err = float(np.abs(got[b:b + 1, h * g:(h + 1) * g] - want).max())
            # 8e-3 is what f16 outputs and f16 probabilities leave at unit magnitude; outputs below the halves'
            # normal range (6e-5) are also limited by the output type's own subnormal step (6e-8)
            assert err <= 8e-3 * size + 6e-8, (step, b, h, err, size)
