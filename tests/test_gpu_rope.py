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


def _rope_step_inputs(rng, B, Hq, Hkv, n, D, dt, per_sequence):
    q = (rng.standard_normal((B, Hq, n, D)) / np.sqrt(D)).astype(dt)
    k = rng.standard_normal((B, Hkv, n, D)).astype(dt)
    v = rng.standard_normal((B, Hkv, n, D)).astype(dt)
    ang = rng.uniform(-7, 7, (B if per_sequence else 1, 1, n, D))
    return q, k, v, np.cos(ang).astype(dt), np.sin(ang).astype(dt)


@pytest.mark.parametrize("B,Hq,Hkv,D,T0,per_sequence", [(2, 32, 8, 128, 61, True), (1, 16, 2, 128, 2050, False), (3, 12, 2, 64, 30, True),
                                                        (8, 32, 8, 128, 2047, True), (1, 14, 2, 128, 95, False)])
def test_decode_steps_rotate_q_and_k_in_the_attention_launch(rt, B, Hq, Hkv, D, T0, per_sequence):
    """Single-token steps through the entry point that fuses ApplyRope on Q and K_new into the append + attention launch:
    after every step the cache's keys are the oracle's rope of the step's keys, bit for bit, and the output equals the
    unfused sequence (ApplyRope, ApplyRope, InPlaceKvSdpa) bit for bit and the oracle within the path's tolerance."""
    rng = np.random.default_rng(B * 1000 + Hq + T0)
    op = tract_amd.InPlaceKvSdpa(axis=2, causal=True)
    fused, plain = op.state(), op.state()
    k0, v0 = rng.standard_normal((B, Hkv, T0, D)).astype(np.float16), rng.standard_normal((B, Hkv, T0, D)).astype(np.float16)
    for st in (fused, plain):
        st.k.reserve(T0 + 3, like=(k0.shape, k0.dtype)), st.v.reserve(T0 + 3, like=(v0.shape, v0.dtype))   # two steps in place, then growth
        st.k.push(k0), st.v.push(v0)
    ks, vs = k0, v0
    for step in range(5):
        q, k, v, cos, sin = _rope_step_inputs(rng, B, Hq, Hkv, 1, D, np.float16, per_sequence)
        dq, dk, dv, dc, ds = (tract_amd.DeviceTensor.from_numpy(a) for a in (q, k, v, cos, sin))
        got = fused.eval_rope_into(dq, dk, dv, dc, ds).to_numpy()
        rq, rk = orc.apply_rope(q, cos, sin), orc.apply_rope(k, cos, sin)
        want_plain = plain.eval([tract_amd.ApplyRope().eval(q, cos, sin), tract_amd.ApplyRope().eval(k, cos, sin), v]).to_numpy()
        ks, vs = np.concatenate([ks, rk], axis=2), np.concatenate([vs, v], axis=2)
        assert fused.k.valid_contiguous().tobytes() == ks.tobytes(), step
        assert fused.v.valid_contiguous().tobytes() == vs.tobytes(), step
        assert got.tobytes() == want_plain.tobytes(), step
        want = orc.flash_sdpa(rq, ks, vs, causal=True)
        assert np.abs(got.astype(np.float32) - want.astype(np.float32)).max() <= 2e-2, step
    assert fused.k.len() == T0 + 5


@pytest.mark.parametrize("dt,B,Hq,Hkv,D,n", [(np.float16, 2, 32, 8, 128, 5), (np.float32, 2, 8, 2, 64, 1), (np.float16, 1, 8, 8, 128, 1),
                                             (np.float16, 1, 40, 2, 128, 1)])
def test_rope_steps_that_rotate_into_the_scratch(rt, dt, B, Hq, Hkv, D, n):
    """Chunks of several tokens, f32, one head per kv head and more than 16 heads per kv head have no fused kernel: the call
    rotates into its scratch and goes on as the plain step; same bits as the unfused sequence."""
    rng = np.random.default_rng(Hq * 7 + n)
    op = tract_amd.InPlaceKvSdpa(axis=2, causal=True)
    fused, plain = op.state(), op.state()
    k0, v0 = rng.standard_normal((B, Hkv, 40, D)).astype(dt), rng.standard_normal((B, Hkv, 40, D)).astype(dt)
    for st in (fused, plain):
        st.k.push(k0), st.v.push(v0)
    for step in range(3):
        q, k, v, cos, sin = _rope_step_inputs(rng, B, Hq, Hkv, n, D, dt, step % 2 == 0)
        got = fused.eval_rope_into(*(tract_amd.DeviceTensor.from_numpy(a) for a in (q, k, v, cos, sin))).to_numpy()
        want = plain.eval([tract_amd.ApplyRope().eval(q, cos, sin), tract_amd.ApplyRope().eval(k, cos, sin), v]).to_numpy()
        assert got.tobytes() == want.tobytes(), step
        assert fused.k.valid_contiguous().tobytes() == plain.k.valid_contiguous().tobytes()


def test_rope_step_refused_for_its_scratch_changes_nothing(rt):
    import ctypes as C
    from tract_amd._lib import call
    rng = np.random.default_rng(5)
    st = tract_amd.InPlaceKvSdpa(axis=2, causal=True).state()
    k0 = rng.standard_normal((1, 2, 33, 128)).astype(np.float16)
    st.k.push(k0), st.v.push(k0)
    q, k, v, cos, sin = _rope_step_inputs(rng, 1, 8, 2, 4, 128, np.float16, False)
    dq, dk, dv, dc, ds = (tract_amd.DeviceTensor.from_numpy(a) for a in (q, k, v, cos, sin))
    out = tract_amd.DeviceTensor(q.shape, q.dtype)
    ws = tract_amd.Workspace(1, 8, 4, 128)
    before = st.k.valid_contiguous().tobytes()
    with pytest.raises(tract_amd.TractRocmError, match="rot_scratch"):
        call("trocm_inplace_kv_sdpa_eval_rope", dq.ptr, dk.ptr, dv.ptr, dc.ptr, ds.ptr, 0, 1, 8, 4, st.k.handle, st.v.handle, out.ptr,
             C.c_float(float("nan")), 1, ws.ptr, ws.nbytes, None, 0, None)
    assert st.k.len() == 33 and st.k.valid_contiguous().tobytes() == before
    got = st.eval_rope_into(dq, dk, dv, dc, ds).to_numpy()   # the same call with its scratch goes through
    assert st.k.len() == 37 and not np.isnan(got).any()


@pytest.mark.parametrize("fmt_name", ["Q8_0", "Q4_0"])
@pytest.mark.parametrize("B,Hq,Hkv,T0,per_sequence", [(2, 32, 8, 61, True), (1, 16, 2, 2050, False), (3, 12, 2, 30, True), (1, 10, 2, 127, True),
                                                      (1, 32, 2, 40, False)])
def test_rope_steps_over_quantised_caches(rt, fmt_name, B, Hq, Hkv, T0, per_sequence):
    """The same over Q8_0 / Q4_0 caches: the key is rotated, then quantised, inside the attention launch (2..8 heads per kv
    head; 16 heads per kv head rotate into the scratch).  The cache's canonical blocks are the CPU quantiser's blocks of the
    oracle's rotated keys, the output equals the unfused sequence bit for bit."""
    fmt = {"Q8_0": tract_amd.Q8_0, "Q4_0": tract_amd.Q4_0}[fmt_name]
    orc_fmt = {"Q8_0": orc.FMT_Q8_0, "Q4_0": orc.FMT_Q4_0}[fmt_name]
    D = 128
    rng = np.random.default_rng(B * 100 + Hq + T0)
    op = tract_amd.InPlaceKvSdpa(axis=2, causal=True, storage_format=fmt)
    fused, plain = op.state(), op.state()
    k0, v0 = rng.standard_normal((B, Hkv, T0, D)).astype(np.float16), rng.standard_normal((B, Hkv, T0, D)).astype(np.float16)
    for st in (fused, plain):
        st.k.push(k0), st.v.push(v0)
    ks = k0
    for step in range(4):
        q, k, v, cos, sin = _rope_step_inputs(rng, B, Hq, Hkv, 1, D, np.float16, per_sequence)
        got = fused.eval_rope_into(*(tract_amd.DeviceTensor.from_numpy(a) for a in (q, k, v, cos, sin))).to_numpy()
        want = plain.eval([tract_amd.ApplyRope().eval(q, cos, sin), tract_amd.ApplyRope().eval(k, cos, sin), v]).to_numpy()
        ks = np.concatenate([ks, orc.apply_rope(k, cos, sin)], axis=2)
        assert fused.k.valid_contiguous().tobytes() == orc.quant(orc_fmt, ks).tobytes(), step
        assert fused.v.valid_contiguous().tobytes() == plain.v.valid_contiguous().tobytes(), step
        assert got.tobytes() == want.tobytes(), step
    assert fused.k.len() == T0 + 4


@pytest.mark.parametrize("fmt_name,Hq,Hkv,D", [("plain", 32, 8, 128), ("plain", 12, 2, 64), ("Q8_0", 32, 8, 128), ("Q4_0", 16, 2, 128),
                                              ("plain", 8, 8, 128), ("Q4_0", 32, 2, 128)])
def test_ragged_steps_with_rope(rt, fmt_name, Hq, Hkv, D):
    """Independent sequences of different lengths, every one rotated by its own position's cos / sin: the ragged step with its
    RoPE folded in (in the attention launch where a kernel rotates, through the scratch otherwise: one head per kv head, 16
    heads per kv head over a quantised cache) equals ApplyRope twice + the plain ragged step bit for bit, caches included."""
    fmt = {"plain": None, "Q8_0": tract_amd.Q8_0, "Q4_0": tract_amd.Q4_0}[fmt_name]
    rng = np.random.default_rng(Hq + D)
    lens = [1, 700, 33, 2049, 128, 5]
    n = len(lens)

    def caches():
        ks, vs = [], []
        for ln in lens:
            kc, vc = tract_amd.InPlaceKvCache(2, fmt), tract_amd.InPlaceKvCache(2, fmt)
            r = np.random.default_rng(ln)
            kc.push(r.standard_normal((1, Hkv, ln, D)).astype(np.float16)), vc.push(r.standard_normal((1, Hkv, ln, D)).astype(np.float16))
            ks.append(kc), vs.append(vc)
        return ks, vs

    (fk, fv), (pk, pv) = caches(), caches()
    for step in range(3):
        q = (rng.standard_normal((n, Hq, 1, D)) / np.sqrt(D)).astype(np.float16)
        k, v = rng.standard_normal((n, Hkv, 1, D)).astype(np.float16), rng.standard_normal((n, Hkv, 1, D)).astype(np.float16)
        ang = rng.uniform(-7, 7, (n, 1, 1, D))
        cos, sin = np.cos(ang).astype(np.float16), np.sin(ang).astype(np.float16)
        dq, dk, dv, dc, ds = (tract_amd.DeviceTensor.from_numpy(a) for a in (q, k, v, cos, sin))
        got = tract_amd.inplace_kv_sdpa_eval_ragged_rope(dq, dk, dv, dc, ds, fk, fv).to_numpy()
        want = tract_amd.inplace_kv_sdpa_eval_ragged(tract_amd.ApplyRope().eval(dq, dc, ds), tract_amd.ApplyRope().eval(dk, dc, ds), dv, pk, pv).to_numpy()
        assert got.tobytes() == want.tobytes(), step
        for a, b in zip(fk + fv, pk + pv):
            assert a.valid_contiguous().tobytes() == b.valid_contiguous().tobytes(), step
    assert fk[0].len() == 4
