"""Attention on the GPU vs the oracle (FlashSdpaOp restatement) and the f64 textbook
form.  Tolerances are the path's contract: max-abs 1e-3 for f32, 2e-2 for f16."""
import os

import numpy as np
import pytest

import tract_amd
from oracle import oracle as orc
from tests import cases
from tests.gpu_util import max_abs, rt  # noqa: F401

pytestmark = pytest.mark.gpu

TOL = {np.dtype(np.float32): 1e-3, np.dtype(np.float16): 2e-2}


@pytest.mark.parametrize("name", sorted(cases.sdpa_literal_cases()))
def test_literal_suite_cases(rt, name):
    q, k, v, mask, scale, causal = cases.sdpa_literal_cases()[name]
    got = tract_amd.Sdpa(scale=scale, datum_type=q.dtype, is_causal=causal).eval(q, k, v, mask).to_numpy()
    want = orc.flash_sdpa(q, k, v, mask=mask, causal=causal, scale=scale)
    assert got.dtype == q.dtype and got.shape == want.shape
    assert max_abs(got, want) <= TOL[q.dtype]
    assert max_abs(got, cases.textbook_sdpa(q, k, v, mask, scale, causal)) <= TOL[q.dtype]


@pytest.mark.parametrize("name,causal,scale", [("simple-causal-f32", True, None), ("simple-non-causal-f32", False, None),
                                               ("simple-scale-f32", False, 1.3)])
def test_reference_golden_f32(rt, golden_dir, name, causal, scale):
    z = np.load(os.path.join(golden_dir, "ref_sdpa", name, "io.npz"))
    x = z["input_0"]
    got = tract_amd.Sdpa(scale=scale, is_causal=causal).eval(x, x, x).to_numpy()
    assert max_abs(got, z["output_0"]) <= 1e-5


def test_reference_golden_mask_and_f16(rt, golden_dir):
    d = os.path.join(golden_dir, "ref_sdpa")
    z = np.load(os.path.join(d, "simple-mask-f32", "io.npz"))
    raw = np.fromfile(os.path.join(d, "simple-mask-f32", "v0.dat"), dtype=np.uint8)
    mask = np.ascontiguousarray(np.broadcast_to(raw[128:].view(np.float32).reshape(1, 2, 1), (1, 2, 2)))
    got = tract_amd.Sdpa().eval(z["input_0"], z["input_1"], z["input_2"], mask).to_numpy()
    assert max_abs(got, z["output_0"]) <= 1e-5
    z = np.load(os.path.join(d, "simple-f16", "io.npz"))
    x = z["input_0"].astype(np.float16)
    got = tract_amd.Sdpa(datum_type=np.float16).eval(x, x, x).to_numpy()
    assert max_abs(got, z["output_0"]) <= 2e-3


@pytest.mark.parametrize("dt", [np.float32, np.float16])
@pytest.mark.parametrize("B,Hq,Hkv,Sq,Sk,D,causal", [
    (1, 2, 2, 16, 24, 8, False), (1, 4, 2, 1, 33, 8, True), (2, 8, 2, 70, 70, 16, True),
    (1, 4, 1, 5, 133, 64, True), (2, 6, 3, 40, 97, 32, False), (1, 3, 1, 2, 300, 80, True),
])
def test_generic_shapes(rt, dt, B, Hq, Hkv, Sq, Sk, D, causal):
    rng = np.random.default_rng(7)
    q = rng.standard_normal((B, Hq, Sq, D), dtype=np.float32).astype(dt)
    k = rng.standard_normal((B, Hkv, Sk, D), dtype=np.float32).astype(dt)
    v = rng.standard_normal((B, Hkv, Sk, D), dtype=np.float32).astype(dt)
    got = tract_amd.Sdpa(datum_type=dt, is_causal=causal).eval(q, k, v).to_numpy()
    assert max_abs(got, orc.flash_sdpa(q, k, v, causal=causal)) <= TOL[np.dtype(dt)]
    assert max_abs(got, cases.textbook_sdpa(q, k, v, causal=causal)) <= TOL[np.dtype(dt)]


@pytest.mark.parametrize("dt", [np.float32, np.float16])
@pytest.mark.parametrize("shape_q,shape_kv,causal,with_mask,scale", [
    ((2, 4, 9, 16), (2, 2, 9, 16), True, False, None),           # generic kernel shapes
    ((1, 6, 5, 8), (1, 2, 23, 8), True, False, 0.7),             # kv_len > q_len: diagonal from the FIRST key
    ((1, 2, 17, 8), (1, 1, 6, 8), True, False, None),            # kv_len < q_len: the rule goes in as a mask
    ((1, 4, 6, 16), (1, 2, 11, 16), True, True, None),           # a mask overrides the causal flag
    ((1, 32, 256, 128), (1, 8, 256, 128), True, False, None),    # MFMA prefill, square causal
    ((1, 32, 128, 128), (1, 8, 640, 128), True, False, None),    # MFMA prefill over the first 128 of 640 keys
    ((2, 32, 1, 128), (2, 8, 1500, 128), False, True, None),     # split-K decode with a rank-2 mask row
    ((2, 40, 64), (2, 100, 64), False, False, None),             # rank 3
])
def test_streamed_sdpa_op(rt, dt, shape_q, shape_kv, causal, with_mask, scale):
    """StreamedSdpaOp (streamed_sdpa.rs:95-272) against the oracle's restatement of its row-streaming loop."""
    rng = np.random.default_rng(len(shape_q) * 100 + shape_q[-2] + shape_kv[-2])
    q = (rng.standard_normal(shape_q) / 3).astype(dt)
    k, v = (rng.standard_normal(shape_kv).astype(dt) for _ in range(2))
    Sq, Sk = shape_q[-2], shape_kv[-2]
    mask = None
    if with_mask:
        mask = rng.standard_normal((Sq, Sk)).astype(np.float32)   # any float type: the op casts it (:143-152)
        mask[rng.random((Sq, Sk)) < 0.3] = -np.inf
        mask[:, 0] = 0.0
        mask[Sq // 2, :] = -np.inf                                 # a row that sees nothing: zeros
        mask[0, 0] = 0.0 if Sq > 1 else -np.inf
    op = tract_amd.StreamedSdpaOp(causal=causal, block_k=32, scale=scale)
    assert op.output_facts(shape_q, shape_kv, shape_kv, None if mask is None else mask.shape) == tuple(shape_q)
    got = op.eval(q, k, v, mask).to_numpy()
    want = orc.streamed_sdpa(q, k, v, mask=mask, causal=causal, scale=scale, block_k=32)
    assert got.shape == want.shape and got.dtype == np.dtype(dt)
    assert max_abs(got, want) <= TOL[np.dtype(dt)]
    if with_mask:
        assert not got[..., Sq // 2, :].any()
    with pytest.raises(tract_amd.TractRocmError):
        op.output_facts(shape_q, shape_kv, shape_kv, (1, Sq, Sk))   # the mask is of rank 2 (:58-60)


def test_padding_mask_equals_shorter_sequence(rt):
    rng = np.random.default_rng(8)
    B, Hq, Hkv, Sq, Sk, D = 2, 4, 2, 3, 80, 16
    q = rng.standard_normal((B, Hq, Sq, D), dtype=np.float32)
    k = rng.standard_normal((B, Hkv, Sk, D), dtype=np.float32)
    v = rng.standard_normal((B, Hkv, Sk, D), dtype=np.float32)
    lens = [50, 80]
    mask = np.zeros((B, 1, Sq, Sk), dtype=np.float32)
    for b, n in enumerate(lens):
        mask[b, :, :, n:] = np.finfo(np.float32).min
    got = tract_amd.Sdpa().eval(q, k, v, mask).to_numpy()
    assert max_abs(got, orc.flash_sdpa(q, k, v, mask=mask)) <= 1e-3
    for b, n in enumerate(lens):
        assert max_abs(got[b:b + 1], cases.textbook_sdpa(q[b:b + 1], k[b:b + 1, :, :n], v[b:b + 1, :, :n])) <= 1e-5


@pytest.mark.parametrize("dt,B,Hq,Hkv,D,T", [
    (np.float16, 1, 32, 8, 128, 1), (np.float16, 1, 32, 8, 128, 31), (np.float16, 1, 32, 8, 128, 32),
    (np.float16, 2, 32, 8, 128, 33), (np.float16, 1, 32, 8, 128, 1000), (np.float16, 2, 32, 8, 128, 4097),
    (np.float32, 1, 32, 32, 64, 1), (np.float32, 1, 32, 32, 64, 255), (np.float32, 2, 8, 4, 64, 513),
    (np.float16, 1, 8, 8, 64, 300), (np.float16, 1, 16, 2, 64, 777), (np.float32, 1, 4, 2, 128, 200),
    (np.float16, 3, 8, 4, 128, 129), (np.float16, 1, 6, 2, 128, 100), (np.float16, 1, 8, 8, 96, 64),
])
def test_decode_split_k(rt, dt, B, Hq, Hkv, D, T):
    """Sq == 1 through the split-K kernel (and the generic one where no fast kernel fits),
    on caches with spare capacity (the tail holds NaN and must never be read)."""
    rng = np.random.default_rng(100 + T)
    q = (rng.standard_normal((B, Hq, 1, D), dtype=np.float32) / np.sqrt(D)).astype(dt)
    k = rng.standard_normal((B, Hkv, T, D), dtype=np.float32).astype(dt)
    v = rng.standard_normal((B, Hkv, T, D), dtype=np.float32).astype(dt)
    st = tract_amd.InPlaceKvSdpa(axis=2, causal=True).state()
    cap = T + 37
    for c in (st.k, st.v):
        c.reserve(cap, like=(k.shape, k.dtype))
        import ctypes as C
        from tract_amd._lib import call
        data = C.c_void_p()
        call("trocm_kv_cache_raw", c.handle, C.byref(data), None, None)
        call("trocm_memset", data, 0xFF, B * Hkv * cap * D * np.dtype(dt).itemsize, None)  # NaN fill
    out = st.eval([q, k, v]).to_numpy()
    want = orc.flash_sdpa(q, k, v, causal=True)
    assert not np.isnan(out).any()
    assert max_abs(out, want) <= TOL[np.dtype(dt)]
    assert max_abs(out, cases.textbook_sdpa(q, k, v, causal=True)) <= (2e-3 if dt == np.float16 else 2e-5)


@pytest.mark.parametrize("kind", ["random", "padding_min", "padding_inf", "leading_inf"])
@pytest.mark.parametrize("dt,B,Hq,Hkv,D,T,mb,mh", [
    (np.float16, 2, 32, 8, 128, 3000, 2, 1), (np.float16, 2, 32, 8, 128, 1025, 1, 32), (np.float16, 3, 8, 8, 64, 333, 3, 8),
    (np.float32, 2, 8, 4, 64, 513, 2, 1), (np.float32, 1, 4, 2, 128, 200, 1, 4), (np.float16, 1, 16, 2, 128, 97, 1, 1),
    # kv_len % 4 == 0 with grouped heads: the MFMA decode kernel (a partial last tile; 16 heads per kv head; group 3, d=64)
    (np.float16, 2, 32, 8, 128, 2052, 1, 32), (np.float16, 1, 32, 2, 128, 516, 1, 1), (np.float16, 2, 24, 8, 64, 1000, 2, 24),
    (np.float16, 8, 32, 8, 128, 8192, 8, 1),
])
def test_decode_with_additive_mask(rt, kind, dt, B, Hq, Hkv, D, T, mb, mh):
    """Sq == 1 with a mask input [mask_b, mask_h, 1, T] (broadcast over batch and/or heads), the form in
    which exported decoders state padding and windows (cuda/src/kernels/flash_attn.rs:138-143): served
    by the split-K kernel.  Padded columns at the reference's finite minimum, at -inf, and -inf over
    whole leading tiles (a tile, a wave or a split that sees nothing must contribute nothing)."""
    rng = np.random.default_rng(200 + T)
    q = (rng.standard_normal((B, Hq, 1, D), dtype=np.float32) / np.sqrt(D)).astype(dt)
    k = rng.standard_normal((B, Hkv, T, D), dtype=np.float32).astype(dt)
    v = rng.standard_normal((B, Hkv, T, D), dtype=np.float32).astype(dt)
    mask = np.zeros((mb, mh, 1, T), dtype=np.float32)
    if kind == "random":
        mask = rng.standard_normal((mb, mh, 1, T), dtype=np.float32) * 3
    else:
        lo = -np.inf if kind.endswith("inf") else float(np.finfo(dt).min)
        for b in range(mb):
            for h in range(mh):
                n = int(rng.integers(1, T))
                if kind == "leading_inf":
                    mask[b, h, 0, :T - n] = lo
                else:
                    mask[b, h, 0, n:] = lo
    mask = mask.astype(dt)
    got = tract_amd.Sdpa(datum_type=dt).eval(q, k, v, mask).to_numpy()
    assert not np.isnan(got).any()
    assert max_abs(got, orc.flash_sdpa(q, k, v, mask=mask)) <= TOL[np.dtype(dt)]
    assert max_abs(got, cases.textbook_sdpa(q, k, v, mask)) <= (2e-3 if dt == np.float16 else 2e-5)


def test_padded_batch_mask_skips_the_padding(rt):
    """A batch padded to its longest sequence with one mask row per sequence (finite minimum or -inf on the
    padded columns, flash_sdpa.rs:261-268): the decode kernel divides only the unpadded tokens among its
    workgroups; results as for any mask.  A row masked out entirely keeps all its tokens (uniform weights)."""
    rng = np.random.default_rng(515)
    B, Hq, Hkv, D, T = 6, 32, 8, 128, 4096
    lens = [4096, 1, 37, 2048, 4095, 0]     # 0: the whole row is masked
    q = (rng.standard_normal((B, Hq, 1, D), dtype=np.float32) / np.sqrt(D)).astype(np.float16)
    k = rng.standard_normal((B, Hkv, T, D), dtype=np.float32).astype(np.float16)
    v = rng.standard_normal((B, Hkv, T, D), dtype=np.float32).astype(np.float16)
    for lo in (float(np.finfo(np.float16).min), -np.inf):
        mask = np.zeros((B, 1, 1, T), dtype=np.float32)
        for b, n in enumerate(lens):
            mask[b, 0, 0, n:] = lo
        if lo == -np.inf:
            mask[5] = float(np.finfo(np.float16).min)   # (all -inf would be NaN in the reference too)
        mask = mask.astype(np.float16)
        got = tract_amd.Sdpa(datum_type=np.float16).eval(q, k, v, mask).to_numpy()
        assert not np.isnan(got).any()
        # (the reference's flash kernel skips key tiles masked below -65503 and returns zeros for the row that is
        # masked out entirely, flash_sdpa.rs:261-268, where its naive Sdpa and the textbook weigh that row's
        # tokens alike: the row is compared with the textbook only)
        assert max_abs(got[:5], orc.flash_sdpa(q, k, v, mask=mask)[:5]) <= 2e-2
        assert max_abs(got, cases.textbook_sdpa(q, k, v, mask)) <= 2e-3
        # a hole in the middle of the kept part stays a hole, and a token that counts after padding is kept
        mask2 = mask.copy()
        mask2[3, 0, 0, 100:1000] = lo
        mask2[2, 0, 0, 3000] = 0
        got = tract_amd.Sdpa(datum_type=np.float16).eval(q, k, v, mask2).to_numpy()
        assert max_abs(got, cases.textbook_sdpa(q, k, v, mask2)) <= 2e-3


_ODD_GROUPS = [(np.float16, 24, 8, 128, 1500), (np.float16, 14, 2, 128, 3000), (np.float16, 12, 2, 128, 700),
               (np.float16, 10, 2, 128, 333), (np.float32, 6, 2, 64, 513), (np.float16, 21, 3, 64, 200)]


@pytest.mark.parametrize("fmt_name,dt,Hq,Hkv,D,T", [("plain",) + c for c in _ODD_GROUPS] +
                         [(f,) + c for f in ("Q8_0", "Q4_0") for c in _ODD_GROUPS if c[0] == np.float16 and c[3] == 128])
def test_decode_group_sizes_that_are_not_powers_of_two(rt, fmt_name, dt, Hq, Hkv, D, T):
    """Group sizes 3, 5, 6, 7 (24q/8kv, 14q/2kv ... of current decoders) run on the split-K kernels of the
    next larger instantiated group size; prefill, fused decode steps, a masked step and the ragged
    form, each against the oracle."""
    fmt = {"plain": None, "Q8_0": tract_amd.Q8_0, "Q4_0": tract_amd.Q4_0}[fmt_name]
    tol = TOL[np.dtype(dt)] if fmt is None else 2e-2
    rng = np.random.default_rng(300 + Hq + T)
    B = 2
    k = rng.standard_normal((B, Hkv, T, D), dtype=np.float32).astype(dt)
    v = rng.standard_normal((B, Hkv, T, D), dtype=np.float32).astype(dt)
    st = tract_amd.InPlaceKvSdpa(axis=2, causal=True, storage_format=fmt).state()
    st.k.push(k), st.v.push(v)
    kd, vd = k, v
    if fmt is not None:   # the oracle attends over the dequantised blocks
        kd = orc.dequant(fmt, orc.quant(fmt, k), dt)
        vd = orc.dequant(fmt, orc.quant(fmt, v), dt)
    for _ in range(3):
        q = (rng.standard_normal((B, Hq, 1, D), dtype=np.float32) / np.sqrt(D)).astype(dt)
        kn = rng.standard_normal((B, Hkv, 1, D), dtype=np.float32).astype(dt)
        vn = rng.standard_normal((B, Hkv, 1, D), dtype=np.float32).astype(dt)
        got = st.eval([q, kn, vn]).to_numpy()
        kq, vq = (kn, vn) if fmt is None else (orc.dequant(fmt, orc.quant(fmt, kn), dt), orc.dequant(fmt, orc.quant(fmt, vn), dt))
        kd, vd = np.concatenate([kd, kq], axis=2), np.concatenate([vd, vq], axis=2)
        assert not np.isnan(got).any()
        assert max_abs(got, orc.flash_sdpa(q, kd, vd, causal=True, threads=4)) <= tol
    if fmt is None:
        assert st.k.valid_contiguous().tobytes() == kd.tobytes()
        # a per-head mask on the same shape
        mask = (rng.standard_normal((B, Hq, 1, kd.shape[2]), dtype=np.float32) * 2).astype(dt)
        got = tract_amd.Sdpa(datum_type=dt).eval(q, kd, vd, mask).to_numpy()
        assert max_abs(got, orc.flash_sdpa(q, kd, vd, mask=mask, threads=4)) <= tol
        # the ragged form: every batch entry as a sequence of its own
        caches = []
        for b in range(B):
            kc, vc = tract_amd.InPlaceKvCache(2), tract_amd.InPlaceKvCache(2)
            n = kd.shape[2] - 17 * b
            kc.push(kd[b:b + 1, :, :n]), vc.push(vd[b:b + 1, :, :n])
            caches.append((kc, vc, n))
        got = tract_amd.sdpa_decode_ragged(tract_amd.DeviceTensor.from_numpy(q), [c[0] for c in caches], [c[1] for c in caches]).to_numpy()
        for b, (_, _, n) in enumerate(caches):
            want = orc.flash_sdpa(q[b:b + 1], kd[b:b + 1, :, :n], vd[b:b + 1, :, :n], threads=4)
            assert max_abs(got[b:b + 1], want) <= tol


@pytest.mark.parametrize("B,Hq,Hkv,D,T", [
    (1, 64, 8, 128, 4097), (2, 64, 8, 128, 1000), (1, 128, 8, 128, 3000), (2, 16, 1, 128, 777), (1, 32, 1, 128, 2050),
    (3, 40, 8, 64, 513), (1, 96, 8, 64, 1500), (2, 24, 2, 128, 31), (1, 64, 8, 128, 1), (8, 64, 8, 128, 300),
    (1, 22, 2, 128, 640),
])
def test_decode_with_large_head_groups(rt, B, Hq, Hkv, D, T):
    """8, 16 or up to 32 query heads per kv head (the 70B / 405B class of decoders): the heads are the rows
    of MFMA tiles.  Over caches with spare capacity (NaN-filled tail), with and without key splits."""
    rng = np.random.default_rng(7000 + Hq + T)
    q = (rng.standard_normal((B, Hq, 1, D), dtype=np.float32) / np.sqrt(D)).astype(np.float16)
    k = rng.standard_normal((B, Hkv, T, D), dtype=np.float32).astype(np.float16)
    v = rng.standard_normal((B, Hkv, T, D), dtype=np.float32).astype(np.float16)
    k[:, :, T // 2] *= 5.0   # an outlier key: the running maxima of waves and splits differ
    st = tract_amd.InPlaceKvSdpa(axis=2, causal=True).state()
    import ctypes as C
    from tract_amd._lib import call
    cap = T + 45
    for c in (st.k, st.v):
        c.reserve(cap, like=(k.shape, k.dtype))
        data, pitch = C.c_void_p(), C.c_int64()
        call("trocm_kv_cache_raw", c.handle, C.byref(data), None, C.byref(pitch))
        call("trocm_memset", data, 0xFF, B * Hkv * pitch.value * D * 2, None)  # NaN fill
    out = st.eval([q, k, v]).to_numpy()
    assert not np.isnan(out).any()
    assert max_abs(out, orc.flash_sdpa(q, k, v, causal=True, threads=8)) <= 2e-2
    assert max_abs(out, cases.textbook_sdpa(q, k, v, causal=True)) <= 2e-3
    # a decode step on top (explicit append, then the same kernel)
    q1 = (rng.standard_normal((B, Hq, 1, D), dtype=np.float32) / np.sqrt(D)).astype(np.float16)
    k1 = rng.standard_normal((B, Hkv, 1, D), dtype=np.float32).astype(np.float16)
    v1 = rng.standard_normal((B, Hkv, 1, D), dtype=np.float32).astype(np.float16)
    out = st.eval([q1, k1, v1]).to_numpy()
    k2, v2 = np.concatenate([k, k1], axis=2), np.concatenate([v, v1], axis=2)
    assert max_abs(out, cases.textbook_sdpa(q1, k2, v2)) <= 2e-3
    assert st.k.valid_contiguous().tobytes() == k2.tobytes()


@pytest.mark.parametrize("splits", [1, 2, 3, 7, 64])
def test_decode_any_split_count_agrees(rt, splits, monkeypatch):
    # The split merge is exact in real arithmetic (log-sum-exp identity).
    import subprocess, sys, json
    code = f"""
import os, json, numpy as np
os.environ['TROCM_DECODE_SPLITS']='{splits}'
import tract_amd
tract_amd.runtime_for_name('rocm')
rng=np.random.default_rng(5)
q=(rng.standard_normal((2,32,1,128),dtype=np.float32)/11.3).astype(np.float16)
k=rng.standard_normal((2,8,3000,128),dtype=np.float32).astype(np.float16)
v=rng.standard_normal((2,8,3000,128),dtype=np.float32).astype(np.float16)
st=tract_amd.InPlaceKvSdpa(2,True).state()
o=st.eval([q,k,v]).to_numpy()
print(json.dumps(o.astype(np.float32).reshape(-1).tolist()))
"""
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, check=True,
                         cwd=os.path.dirname(os.path.dirname(os.path.abspath(__file__)))).stdout
    got = np.array(json.loads(out.strip().splitlines()[-1]), dtype=np.float32).reshape(2, 32, 1, 128)
    rng = np.random.default_rng(5)
    q = (rng.standard_normal((2, 32, 1, 128), dtype=np.float32) / 11.3).astype(np.float16)
    k = rng.standard_normal((2, 8, 3000, 128), dtype=np.float32).astype(np.float16)
    v = rng.standard_normal((2, 8, 3000, 128), dtype=np.float32).astype(np.float16)
    assert max_abs(got, cases.textbook_sdpa(q, k, v)) <= 2e-3


@pytest.mark.parametrize("period,splits", [(2, 4), (3, 2), (5, 8), (16, 4)])
def test_decode_with_unequal_shares_of_the_splits(rt, period, splits):
    """Odd splits (they run on the odd XCDs, which stream slower) leave every `period`-th round of tile groups to their
    even neighbours.  Small periods make many such rounds at a test's size; steps with the fused append and RoPE go
    through the same tile sequence.  Expected: the textbook result, and the same cache contents as without."""
    import subprocess, sys, json
    code = f"""
import os, json, numpy as np
os.environ['TROCM_DECODE_XCD_SKEW']='{period}'
os.environ['TROCM_DECODE_SPLITS']='{splits}'
import tract_amd
tract_amd.runtime_for_name('rocm')
rng=np.random.default_rng(17)
T=5000
q=(rng.standard_normal((3,2,32,1,128),dtype=np.float32)/11.3).astype(np.float16)
k=rng.standard_normal((2,8,T,128),dtype=np.float32).astype(np.float16)
v=rng.standard_normal((2,8,T,128),dtype=np.float32).astype(np.float16)
kn=rng.standard_normal((3,2,8,1,128),dtype=np.float32).astype(np.float16)
vn=rng.standard_normal((3,2,8,1,128),dtype=np.float32).astype(np.float16)
st=tract_amd.InPlaceKvSdpa(2,True).state()
st.eval([q[0][:, :, :1], k, v])
outs=[st.eval([q[i], kn[i], vn[i]]).to_numpy().astype(np.float32).reshape(-1).tolist() for i in range(3)]
tail=st.k.valid_contiguous()[:, :, -3:].astype(np.float32).reshape(-1).tolist()
print(json.dumps([outs, tail]))
"""
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, check=True,
                         cwd=os.path.dirname(os.path.dirname(os.path.abspath(__file__)))).stdout
    outs, tail = json.loads(out.strip().splitlines()[-1])
    rng = np.random.default_rng(17)
    T = 5000
    q = (rng.standard_normal((3, 2, 32, 1, 128), dtype=np.float32) / 11.3).astype(np.float16)
    k = rng.standard_normal((2, 8, T, 128), dtype=np.float32).astype(np.float16)
    v = rng.standard_normal((2, 8, T, 128), dtype=np.float32).astype(np.float16)
    kn = rng.standard_normal((3, 2, 8, 1, 128), dtype=np.float32).astype(np.float16)
    vn = rng.standard_normal((3, 2, 8, 1, 128), dtype=np.float32).astype(np.float16)
    for i in range(3):
        k, v = np.concatenate([k, kn[i]], axis=2), np.concatenate([v, vn[i]], axis=2)
        got = np.array(outs[i], dtype=np.float32).reshape(2, 32, 1, 128)
        assert max_abs(got, cases.textbook_sdpa(q[i], k, v)) <= 2e-3
    assert np.array_equal(np.array(tail, dtype=np.float32).reshape(2, 8, 3, 128), k[:, :, -3:].astype(np.float32))


def test_inplace_kv_sdpa_decode_loop_cfg1(rt):
    """cfg1: B=1, 32 q heads = 32 kv heads, D=64, f32, cache grows 0 -> 256 one token per
    step with causal attention at each step; fused op vs {concat cache, FlashSdpaOp}."""
    B, H, D, T = 1, 32, 64, 256
    q = cases.seeded_normal(cases.cfg_seed(1, "q"), (T, B, H, 1, D))
    k = cases.seeded_normal(cases.cfg_seed(1, "k"), (T, B, H, 1, D))
    v = cases.seeded_normal(cases.cfg_seed(1, "v"), (T, B, H, 1, D))
    st = tract_amd.InPlaceKvSdpa(axis=2, causal=True, scale=None).state()
    kc = vc = None
    worst = 0.0
    for t in range(T):
        out = st.eval([q[t], k[t], v[t]]).to_numpy()
        kc, vc = orc.concat_append(kc, k[t], 2), orc.concat_append(vc, v[t], 2)
        if t % 8 == 0 or t > 250:
            worst = max(worst, max_abs(out, orc.flash_sdpa(q[t], kc, vc, causal=True)))
    assert st.k.len() == T and st.k.capacity() == 256 and st.k.reallocs() == 8
    assert worst <= 1e-3
    saved = []
    st.save_to(saved)
    assert saved[0].tobytes() == kc.tobytes() and saved[1].tobytes() == vc.tobytes()


def test_ragged_decode_small(rt):
    rng = np.random.default_rng(21)
    Hq, Hkv, D = 32, 8, 128
    lens = [1, 31, 64, 200, 1025]
    ks, vs, qs = [], [], []
    kcs, vcs = [], []
    for n in lens:
        k = rng.standard_normal((1, Hkv, n, D), dtype=np.float32).astype(np.float16)
        v = rng.standard_normal((1, Hkv, n, D), dtype=np.float32).astype(np.float16)
        kc, vc = tract_amd.InPlaceKvCache(2), tract_amd.InPlaceKvCache(2)
        kc.push(k), vc.push(v)
        ks.append(k), vs.append(v), kcs.append(kc), vcs.append(vc)
    q = (rng.standard_normal((len(lens), Hq, 1, D), dtype=np.float32) / np.sqrt(D)).astype(np.float16)
    out = tract_amd.sdpa_decode_ragged(tract_amd.DeviceTensor.from_numpy(q), kcs, vcs).to_numpy()
    for i in range(len(lens)):
        want = orc.flash_sdpa(q[i:i + 1], ks[i], vs[i], causal=True)
        assert max_abs(out[i:i + 1], want) <= 2e-2


@pytest.mark.parametrize("fmt_name", ["Q8_0", "Q4_0"])
@pytest.mark.parametrize("B,Hq,Hkv,T", [(1, 32, 8, 1), (2, 32, 8, 100), (2, 32, 8, 1025), (1, 8, 8, 333), (1, 16, 2, 64),
                                         (1, 24, 8, 77), (2, 32, 2, 300), (1, 32, 1, 129), (1, 22, 2, 95),
                                         # 5..8 heads per kv head: two sets of four heads in the diagonal body
                                         (2, 64, 8, 1025), (1, 10, 2, 1), (3, 12, 2, 257), (1, 14, 2, 4100), (2, 16, 2, 33)])
def test_decode_quantised_cache(rt, fmt_name, B, Hq, Hkv, T):
    """cfg4 (reduced): K/V quantised on append, 1% outlier channels x20, decode with fused
    dequantisation.  Oracle: FlashSdpaOp over the dequantised blocks (f16 dequant like
    BlockQuant::dequant_f16, then the f16 eval path)."""
    D = 128
    dev_fmt = getattr(tract_amd, fmt_name)
    orc_fmt = getattr(orc, "FMT_" + fmt_name)
    rng = np.random.default_rng(cases.cfg_seed(4, "chan") + T)
    chan = rng.choice(Hkv * D, size=max(1, Hkv * D // 100), replace=False)

    def outliers(x):
        xf = x.transpose(0, 2, 1, 3).reshape(B, -1, Hkv * D).astype(np.float32)
        xf[:, :, chan] *= 20
        return xf.reshape(B, -1, Hkv, D).transpose(0, 2, 1, 3).astype(np.float16)

    k = outliers(cases.seeded_normal(cases.cfg_seed(4, "k") + T, (B, Hkv, T, D)))
    v = outliers(cases.seeded_normal(cases.cfg_seed(4, "v") + T, (B, Hkv, T, D)))
    q = (cases.seeded_normal(cases.cfg_seed(4, "q") + T, (B, Hq, 1, D)) / np.sqrt(D)).astype(np.float16)
    st = tract_amd.InPlaceKvSdpa(axis=2, causal=True, storage_format=dev_fmt).state()
    st.k.reserve(T + 19, like=(k.shape, k.dtype))
    st.v.reserve(T + 19, like=(v.shape, v.dtype))
    out = st.eval([q, k, v]).to_numpy()
    kq, vq = orc.quant(orc_fmt, k), orc.quant(orc_fmt, v)
    assert st.k.valid_contiguous().tobytes() == kq.tobytes() and st.v.valid_contiguous().tobytes() == vq.tobytes()
    kd, vd = orc.dequant(orc_fmt, kq, np.float16), orc.dequant(orc_fmt, vq, np.float16)
    want = orc.flash_sdpa(q, kd, vd, causal=True)
    assert not np.isnan(out).any()
    assert max_abs(out, want) <= 2e-2
    # attributable: against f32 dequantisation in f64 the fused kernel is much closer
    exact = cases.textbook_sdpa(q, orc.dequant(orc_fmt, kq, np.float32), orc.dequant(orc_fmt, vq, np.float32))
    # (the output is f16: allow its rounding, half an ulp relative, on the outlier-channel magnitudes)
    assert np.allclose(out.astype(np.float64), exact, rtol=1.5e-3, atol=2e-3)


@pytest.mark.parametrize("fmt_name", ["Q8_0", "Q4_0"])
@pytest.mark.parametrize("B,Hq,Hkv,T0", [(2, 32, 8, 61), (1, 16, 2, 30), (2, 32, 2, 95), (1, 6, 2, 0), (8, 32, 8, 2047), (1, 8, 8, 40),
                                          (2, 14, 2, 95), (1, 40, 8, 1021)])
def test_decode_steps_quantise_the_new_token_in_the_attention_launch(rt, fmt_name, B, Hq, Hkv, T0):
    """Single-token steps on a quantised cache (f16 inputs): the attention kernel quantises the step's K and V rows
    itself, stores them and attends over them.  After every step the cache's canonical blocks equal the CPU quantiser's
    on all tokens so far, and the output the oracle's attention over the dequantised blocks; the steps cross a tile
    boundary, and the new rows carry an outlier channel, a zero block and a block with +x and -x of equal magnitude.
    (One head per kv head takes the separate append launch: same checks.)"""
    D = 128
    dev_fmt, orc_fmt = getattr(tract_amd, fmt_name), getattr(orc, "FMT_" + fmt_name)
    rng = np.random.default_rng(T0 + Hq)
    st = tract_amd.InPlaceKvSdpa(axis=2, causal=True, storage_format=dev_fmt).state()
    ks = rng.standard_normal((B, Hkv, T0, D), dtype=np.float32).astype(np.float16)
    vs = rng.standard_normal((B, Hkv, T0, D), dtype=np.float32).astype(np.float16)
    if T0:
        st.k.push(ks), st.v.push(vs)
    for step in range(5):
        q = (rng.standard_normal((B, Hq, 1, D), dtype=np.float32) / np.sqrt(D)).astype(np.float16)
        kn = rng.standard_normal((B, Hkv, 1, D), dtype=np.float32).astype(np.float16)
        vn = rng.standard_normal((B, Hkv, 1, D), dtype=np.float32).astype(np.float16)
        kn[..., 7] *= 20
        vn[:, :, :, 32:64] = 0
        kn[:, :, :, 64], kn[:, :, :, 65] = np.float16(-30.0), np.float16(30.0)
        vn[:, :, :, 100], vn[:, :, :, 97] = np.float16(9.5), np.float16(-9.5)
        # products that round onto a rounding boundary (x = mx / 2: x * (1 / scale) is 63.49999.. before its rounding, 63.5
        # after): a multiply fused with the addition that follows it would code them differently
        kn[:, :, :, 96:128] *= np.float16(0.05)
        mx = np.float16(2.3476562 + 0.001 * step)
        kn[:, :, :, 96], kn[:, :, :, 97], kn[:, :, :, 98], kn[:, :, :, 99] = mx, mx / np.float16(2), mx / np.float16(16), np.float16(3) * mx / np.float16(16)
        vn[:, :, :, 0:32] *= np.float16(0.05)
        vn[:, :, :, 0], vn[:, :, :, 1], vn[:, :, :, 2] = -mx, -mx / np.float16(2), mx / np.float16(2)
        out = st.eval([q, kn, vn]).to_numpy()
        ks, vs = np.concatenate([ks, kn], axis=2), np.concatenate([vs, vn], axis=2)
        kq, vq = orc.quant(orc_fmt, ks), orc.quant(orc_fmt, vs)
        assert st.k.valid_contiguous().tobytes() == kq.tobytes(), step
        assert st.v.valid_contiguous().tobytes() == vq.tobytes(), step
        want = orc.flash_sdpa(q, orc.dequant(orc_fmt, kq, np.float16), orc.dequant(orc_fmt, vq, np.float16), causal=True)
        assert not np.isnan(out).any() and max_abs(out, want) <= 2e-2, step
    assert st.k.len() == T0 + 5


@pytest.mark.parametrize("fmt_name", ["Q8_0", "Q4_0"])
@pytest.mark.parametrize("Hq,Hkv,n_seq,lo,hi", [(32, 8, 12, 1, 2500), (16, 1, 5, 20, 700), (8, 8, 4, 10, 200), (16, 2, 9, 1, 3000),
                                                 (12, 2, 5, 30, 900)])
def test_ragged_decode_over_quantised_caches(rt, fmt_name, Hq, Hkv, n_seq, lo, hi):
    """Independent sequences with quantised caches of their own: every sequence equals the batch-1
    oracle over its dequantised blocks.  Two steps: attention only, then the append-and-attend step."""
    D = 128
    dev_fmt, orc_fmt = getattr(tract_amd, fmt_name), getattr(orc, "FMT_" + fmt_name)
    rng = np.random.default_rng(cases.cfg_seed(5, "len") + Hq)
    lens = rng.integers(lo, hi, size=n_seq, endpoint=True)
    kcs, vcs, ks, vs = [], [], [], []
    for n in lens:
        k = rng.standard_normal((1, Hkv, int(n), D), dtype=np.float32).astype(np.float16)
        v = rng.standard_normal((1, Hkv, int(n), D), dtype=np.float32).astype(np.float16)
        kc, vc = tract_amd.InPlaceKvCache(2, dev_fmt), tract_amd.InPlaceKvCache(2, dev_fmt)
        kc.push(k), vc.push(v)
        kcs.append(kc), vcs.append(vc), ks.append(k), vs.append(v)
    ws = tract_amd.Workspace(n_seq, Hq, 1, D)

    def check(out, q):
        assert not np.isnan(out).any()
        for i in range(n_seq):
            kd = orc.dequant(orc_fmt, orc.quant(orc_fmt, ks[i]), np.float16)
            vd = orc.dequant(orc_fmt, orc.quant(orc_fmt, vs[i]), np.float16)
            assert max_abs(out[i:i + 1], orc.flash_sdpa(q[i:i + 1], kd, vd, causal=True)) <= 2e-2, f"sequence {i} len {ks[i].shape[2]}"

    q = (rng.standard_normal((n_seq, Hq, 1, D), dtype=np.float32) / np.sqrt(D)).astype(np.float16)
    check(tract_amd.sdpa_decode_ragged(tract_amd.DeviceTensor.from_numpy(q), kcs, vcs, workspace=ws).to_numpy(), q)
    kn = rng.standard_normal((n_seq, Hkv, 1, D), dtype=np.float32).astype(np.float16)
    vn = rng.standard_normal((n_seq, Hkv, 1, D), dtype=np.float32).astype(np.float16)
    q = (rng.standard_normal((n_seq, Hq, 1, D), dtype=np.float32) / np.sqrt(D)).astype(np.float16)
    out = tract_amd.inplace_kv_sdpa_eval_ragged(tract_amd.DeviceTensor.from_numpy(q), tract_amd.DeviceTensor.from_numpy(kn),
                                                tract_amd.DeviceTensor.from_numpy(vn), kcs, vcs, workspace=ws).to_numpy()
    for i in range(n_seq):
        ks[i], vs[i] = np.concatenate([ks[i], kn[i:i + 1]], axis=2), np.concatenate([vs[i], vn[i:i + 1]], axis=2)
    check(out, q)
    for i in range(n_seq):   # the new tokens' blocks (quantised by the attention launch where it takes them) are the CPU quantiser's
        assert kcs[i].valid_contiguous().tobytes() == orc.quant(orc_fmt, ks[i]).tobytes(), i
        assert vcs[i].valid_contiguous().tobytes() == orc.quant(orc_fmt, vs[i]).tobytes(), i


def test_ragged_step_over_quantised_caches_with_f32_tokens(rt):
    """f32 queries and new tokens over Q8_0 caches: no fast attention kernel takes f32 queries (one generic call
    per sequence), but the step's tokens are still quantised by the one launch, from f32, to the oracle's blocks."""
    rng = np.random.default_rng(91)
    Hq, Hkv, D = 8, 2, 128
    lens = [40, 7, 130]
    kcs, vcs, ks, vs = [], [], [], []
    for n in lens:
        k = rng.standard_normal((1, Hkv, n, D), dtype=np.float32)
        v = rng.standard_normal((1, Hkv, n, D), dtype=np.float32)
        kc, vc = tract_amd.InPlaceKvCache(2, tract_amd.Q8_0), tract_amd.InPlaceKvCache(2, tract_amd.Q8_0)
        kc.push(k), vc.push(v)
        kcs.append(kc), vcs.append(vc), ks.append(k), vs.append(v)
    q = rng.standard_normal((len(lens), Hq, 1, D), dtype=np.float32) / np.sqrt(D).astype(np.float32)
    kn = rng.standard_normal((len(lens), Hkv, 1, D), dtype=np.float32)
    vn = rng.standard_normal((len(lens), Hkv, 1, D), dtype=np.float32)
    out = tract_amd.inplace_kv_sdpa_eval_ragged(tract_amd.DeviceTensor.from_numpy(q), tract_amd.DeviceTensor.from_numpy(kn),
                                                tract_amd.DeviceTensor.from_numpy(vn), kcs, vcs).to_numpy()
    for i, n in enumerate(lens):
        k = np.concatenate([ks[i], kn[i:i + 1]], axis=2)
        v = np.concatenate([vs[i], vn[i:i + 1]], axis=2)
        kq, vq = orc.quant(orc.FMT_Q8_0, k), orc.quant(orc.FMT_Q8_0, v)
        assert kcs[i].len() == n + 1
        assert kcs[i].valid_contiguous().tobytes() == kq.tobytes() and vcs[i].valid_contiguous().tobytes() == vq.tobytes()
        want = orc.flash_sdpa(q[i:i + 1], orc.dequant(orc.FMT_Q8_0, kq), orc.dequant(orc.FMT_Q8_0, vq), causal=True)
        assert max_abs(out[i:i + 1], want) <= 1e-3, f"sequence {i}"


def test_quantised_cache_with_f32_queries_uses_generic_kernel(rt):
    rng = np.random.default_rng(31)
    B, Hq, Hkv, T, D = 1, 4, 2, 50, 64
    k = rng.standard_normal((B, Hkv, T, D), dtype=np.float32)
    v = rng.standard_normal((B, Hkv, T, D), dtype=np.float32)
    q = rng.standard_normal((B, Hq, 3, D), dtype=np.float32) / 8
    for dev_fmt, orc_fmt in ((tract_amd.Q8_0, orc.FMT_Q8_0), (tract_amd.Q4_0, orc.FMT_Q4_0)):
        st = tract_amd.InPlaceKvSdpa(axis=2, causal=False, storage_format=dev_fmt).state()
        st.k.push(k), st.v.push(v)
        out = st.attend(tract_amd.DeviceTensor.from_numpy(q)).to_numpy()
        kd = orc.dequant(orc_fmt, orc.quant(orc_fmt, k))
        vd = orc.dequant(orc_fmt, orc.quant(orc_fmt, v))
        assert max_abs(out, orc.flash_sdpa(q, kd, vd)) <= 1e-3


@pytest.mark.parametrize("dt,Hq,Hkv,D,n_seq,lo,hi", [
    (np.float16, 32, 8, 128, 24, 1, 3000), (np.float32, 8, 8, 64, 7, 30, 900), (np.float16, 16, 2, 64, 40, 1, 400),
    (np.float16, 6, 2, 128, 5, 10, 300),   # group size 3: per-sequence fall-back
])
def test_ragged_decode_many_sequences(rt, dt, Hq, Hkv, D, n_seq, lo, hi):
    """cfg5 (reduced): independent sequences with their own capacity-doubling caches and
    lengths; every sequence must equal the batch-1 oracle.  Two decode steps with an append
    in between, so lengths (and the work plan) change from call to call."""
    rng = np.random.default_rng(cases.cfg_seed(5, "len"))
    lens = rng.integers(lo, hi, size=n_seq, endpoint=True)
    kcs, vcs, ks, vs = [], [], [], []
    for n in lens:
        k = rng.standard_normal((1, Hkv, int(n), D), dtype=np.float32).astype(dt)
        v = rng.standard_normal((1, Hkv, int(n), D), dtype=np.float32).astype(dt)
        kc, vc = tract_amd.InPlaceKvCache(2), tract_amd.InPlaceKvCache(2)
        kc.push(k), vc.push(v)
        kcs.append(kc), vcs.append(vc), ks.append(k), vs.append(v)
    ws = tract_amd.Workspace(n_seq, Hq, 1, D)
    for step in range(2):
        q = (rng.standard_normal((n_seq, Hq, 1, D), dtype=np.float32) / np.sqrt(D)).astype(dt)
        out = tract_amd.sdpa_decode_ragged(tract_amd.DeviceTensor.from_numpy(q), kcs, vcs, workspace=ws).to_numpy()
        assert not np.isnan(out).any()
        for i in range(n_seq):
            want = orc.flash_sdpa(q[i:i + 1], ks[i], vs[i], causal=True)
            assert max_abs(out[i:i + 1], want) <= TOL[np.dtype(dt)], f"sequence {i} len {ks[i].shape[2]}"
        for i in range(n_seq):  # append one token to every sequence
            kn = rng.standard_normal((1, Hkv, 1, D), dtype=np.float32).astype(dt)
            vn = rng.standard_normal((1, Hkv, 1, D), dtype=np.float32).astype(dt)
            kcs[i].push(kn), vcs[i].push(vn)
            ks[i], vs[i] = np.concatenate([ks[i], kn], axis=2), np.concatenate([vs[i], vn], axis=2)


@pytest.mark.parametrize("fmt_name", ["plain", "Q8_0"])
@pytest.mark.parametrize("ws_bytes", [0, 70_000, 400_000])
def test_decode_with_a_small_or_no_workspace(rt, fmt_name, ws_bytes):
    """A decode call whose workspace has no room for the splits it would like runs with fewer, down to one
    (no workspace at all): the result does not change."""
    from tract_amd._lib import call
    from tract_amd.runtime import dtype_code
    rng = np.random.default_rng(88)
    B, Hq, Hkv, D, T = 1, 32, 8, 128, 3000
    fmt = None if fmt_name == "plain" else tract_amd.Q8_0
    k = rng.standard_normal((B, Hkv, T, D), dtype=np.float32).astype(np.float16)
    v = rng.standard_normal((B, Hkv, T, D), dtype=np.float32).astype(np.float16)
    q = (rng.standard_normal((B, Hq, 1, D), dtype=np.float32) / np.sqrt(D)).astype(np.float16)
    st = tract_amd.InPlaceKvSdpa(axis=2, causal=True, storage_format=fmt).state()
    st.k.push(k), st.v.push(v)
    qd, out = tract_amd.DeviceTensor.from_numpy(q), tract_amd.DeviceTensor(q.shape, np.float16)
    want = st.attend(qd).to_numpy()
    ws = tract_amd.DeviceTensor((max(ws_bytes, 16),), np.uint8)
    if ws_bytes:
        call("trocm_sdpa_workspace_init", ws.ptr, ws_bytes, None)
    call("trocm_sdpa_cached", qd.ptr, dtype_code(np.float16), Hq, 1, st.k.handle, st.v.handle, out.ptr,
         float("nan"), 1, ws.ptr if ws_bytes else None, ws_bytes, None)
    assert max_abs(out.to_numpy(), want) <= 2e-3


def test_one_workspace_shared_by_ragged_and_dense_calls(rt):
    """A ragged call keeps its launch plan in the workspace; a dense decode that follows on the same
    workspace counts workgroup arrivals there.  Neither may disturb the other, in either order."""
    rng = np.random.default_rng(404)
    Hq, Hkv, D, B, T = 32, 8, 128, 4, 2100
    lens = [700, 2100, 1300, 4000, 64, 900]
    kcs, vcs, ks = [], [], []
    for n in lens:
        k = rng.standard_normal((1, Hkv, n, D), dtype=np.float32).astype(np.float16)
        kc, vc = tract_amd.InPlaceKvCache(2), tract_amd.InPlaceKvCache(2)
        kc.push(k), vc.push(k)
        kcs.append(kc), vcs.append(vc), ks.append(k)
    kd = rng.standard_normal((B, Hkv, T, D), dtype=np.float32).astype(np.float16)
    st = tract_amd.InPlaceKvSdpa(axis=2, causal=True).state()
    st.k.push(kd), st.v.push(kd)
    ws = tract_amd.Workspace(max(B, len(lens)), Hq, 1, D)
    qr = (rng.standard_normal((len(lens), Hq, 1, D), dtype=np.float32) / np.sqrt(D)).astype(np.float16)
    qd = (rng.standard_normal((B, Hq, 1, D), dtype=np.float32) / np.sqrt(D)).astype(np.float16)
    want_d = orc.flash_sdpa(qd, kd, kd, causal=True)
    from tract_amd._lib import call
    from tract_amd.runtime import dtype_code
    qd_dev, out_d = tract_amd.DeviceTensor.from_numpy(qd), tract_amd.DeviceTensor(qd.shape, np.float16)
    for turn in range(3):
        got_r = tract_amd.sdpa_decode_ragged(tract_amd.DeviceTensor.from_numpy(qr), kcs, vcs, workspace=ws).to_numpy()
        call("trocm_sdpa_cached", qd_dev.ptr, dtype_code(np.float16), Hq, 1, st.k.handle, st.v.handle, out_d.ptr,
             float("nan"), 1, ws.ptr, ws.nbytes, None)
        got_d = out_d.to_numpy()
        assert max_abs(got_d, want_d) <= 2e-2, f"dense after ragged, turn {turn}"
        for i in range(len(lens)):
            assert max_abs(got_r[i:i + 1], orc.flash_sdpa(qr[i:i + 1], ks[i], ks[i], causal=True)) <= 2e-2, f"ragged, turn {turn}, sequence {i}"


def test_ragged_decode_with_a_thousand_short_sequences(rt):
    """More sequences than compute units: every sequence is one work item, the plan holds a thousand of them."""
    rng = np.random.default_rng(1000)
    Hq, Hkv, D, n_seq = 8, 2, 64, 1000
    lens = rng.integers(1, 40, size=n_seq, endpoint=True)
    pool = tract_amd.KvPool(64 << 20)
    kcs, vcs, ks, vs = [], [], [], []
    for n in lens:
        k = rng.standard_normal((1, Hkv, int(n), D), dtype=np.float32).astype(np.float16)
        v = rng.standard_normal((1, Hkv, int(n), D), dtype=np.float32).astype(np.float16)
        kc, vc = tract_amd.InPlaceKvCache(2, pool=pool), tract_amd.InPlaceKvCache(2, pool=pool)
        kc.push(k), vc.push(v)
        kcs.append(kc), vcs.append(vc), ks.append(k), vs.append(v)
    q = (rng.standard_normal((n_seq, Hq, 1, D), dtype=np.float32) / np.sqrt(D)).astype(np.float16)
    out = tract_amd.sdpa_decode_ragged(tract_amd.DeviceTensor.from_numpy(q), kcs, vcs).to_numpy()
    assert not np.isnan(out).any()
    for i in range(0, n_seq, 7):
        assert max_abs(out[i:i + 1], orc.flash_sdpa(q[i:i + 1], ks[i], vs[i], causal=True)) <= 2e-2, f"sequence {i}"


@pytest.mark.parametrize("n_seq", [600, 2048])
def test_ragged_decode_with_many_sequences_of_a_grouped_head_model(rt, n_seq):
    """32 query heads on 8 kv heads at head_dim 128 (padded groups of 8 rows per record) with a workspace of exactly
    the size the library asks for: many short sequences that are one work item each (they need no partial record)
    next to a few long ones that are cut."""
    rng = np.random.default_rng(n_seq)
    Hq, Hkv, D = 32, 8, 128
    lens = rng.integers(1, 48, size=n_seq, endpoint=True)
    lens[[3, n_seq // 2, n_seq - 1]] = [9000, 5000, 2500]
    pool = tract_amd.KvPool(int(lens.sum()) * Hkv * D * 2 * 2 * 2 + (128 << 20))
    kcs, vcs, ks, vs = [], [], [], []
    for n in lens:
        k = rng.standard_normal((1, Hkv, int(n), D), dtype=np.float32).astype(np.float16)
        v = rng.standard_normal((1, Hkv, int(n), D), dtype=np.float32).astype(np.float16)
        kc, vc = tract_amd.InPlaceKvCache(2, pool=pool), tract_amd.InPlaceKvCache(2, pool=pool)
        kc.push(k), vc.push(v)
        kcs.append(kc), vcs.append(vc), ks.append(k), vs.append(v)
    q = (rng.standard_normal((n_seq, Hq, 1, D), dtype=np.float32) / np.sqrt(D)).astype(np.float16)
    ws = tract_amd.Workspace(n_seq, Hq, 1, D)
    assert ws.nbytes == tract_amd.Workspace.bytes_for(n_seq, Hq, 1, D)
    qd = tract_amd.DeviceTensor.from_numpy(q)
    out = tract_amd.sdpa_decode_ragged(qd, kcs, vcs, workspace=ws).to_numpy()
    assert not np.isnan(out).any()
    for i in sorted(set(range(0, n_seq, 41)) | {3, n_seq // 2, n_seq - 1}):
        assert max_abs(out[i:i + 1], orc.flash_sdpa(q[i:i + 1], ks[i], vs[i], causal=True)) <= 2e-2, f"sequence {i}"
    # a fused step on the same workspace
    kn = rng.standard_normal((n_seq, Hkv, 1, D), dtype=np.float32).astype(np.float16)
    vn = rng.standard_normal((n_seq, Hkv, 1, D), dtype=np.float32).astype(np.float16)
    out = tract_amd.inplace_kv_sdpa_eval_ragged(qd, tract_amd.DeviceTensor.from_numpy(kn), tract_amd.DeviceTensor.from_numpy(vn),
                                                kcs, vcs, workspace=ws).to_numpy()
    for i in sorted(set(range(0, n_seq, 97)) | {3, n_seq - 1}):
        kk, vv = np.concatenate([ks[i], kn[i:i + 1]], 2), np.concatenate([vs[i], vn[i:i + 1]], 2)
        assert max_abs(out[i:i + 1], orc.flash_sdpa(q[i:i + 1], kk, vv, causal=True)) <= 2e-2, f"fused step, sequence {i}"
        assert kcs[i].valid_contiguous().tobytes() == kk.tobytes()


def test_ragged_equals_padded_batch_with_mask(rt):
    """The reference's statement of a ragged batch: a dense batch padded to the longest
    sequence with an additive mask whose padded columns are <= -65504 (flash_sdpa.rs:261-268)."""
    rng = np.random.default_rng(77)
    Hq, Hkv, D = 8, 2, 64
    lens = [5, 64, 33, 100]
    Tmax = max(lens)
    kp = np.zeros((len(lens), Hkv, Tmax, D), np.float32)
    vp = np.zeros((len(lens), Hkv, Tmax, D), np.float32)
    mask = np.zeros((len(lens), 1, 1, Tmax), np.float32)
    kcs, vcs = [], []
    for i, n in enumerate(lens):
        k = rng.standard_normal((1, Hkv, n, D), dtype=np.float32)
        v = rng.standard_normal((1, Hkv, n, D), dtype=np.float32)
        kp[i, :, :n], vp[i, :, :n] = k[0], v[0]
        mask[i, :, :, n:] = -65504.0
        kc, vc = tract_amd.InPlaceKvCache(2), tract_amd.InPlaceKvCache(2)
        kc.push(k), vc.push(v)
        kcs.append(kc), vcs.append(vc)
    q = rng.standard_normal((len(lens), Hq, 1, D), dtype=np.float32) / 8
    got = tract_amd.sdpa_decode_ragged(tract_amd.DeviceTensor.from_numpy(q), kcs, vcs).to_numpy()
    want = orc.flash_sdpa(q, kp, vp, mask=mask)
    assert max_abs(got, want) <= 1e-3
    dense = tract_amd.Sdpa().eval(q, kp, vp, mask).to_numpy()
    assert max_abs(got, dense) <= 1e-5


@pytest.mark.parametrize("B,Hq,Hkv,Sq,Sk,D,causal", [
    (1, 4, 1, 32, 32, 128, True), (1, 4, 2, 64, 64, 128, True), (1, 8, 2, 100, 100, 128, True),
    (1, 4, 4, 33, 200, 128, True), (2, 8, 2, 77, 301, 128, False), (1, 32, 8, 128, 384, 128, True),
    (2, 32, 8, 512, 512, 128, True),      # >= 256 workgroups: 128-query tiles (4x1 waves)
    (1, 32, 8, 200, 712, 128, True),      # 64-query tiles (2x2 waves), ragged edges
    (1, 8, 8, 90, 90, 64, True), (2, 64, 8, 256, 300, 64, False), (1, 4, 2, 2, 9, 128, True),
])
def test_prefill_mfma(rt, B, Hq, Hkv, Sq, Sk, D, causal):
    rng = np.random.default_rng(1000 + Sq + Sk)
    q = (rng.standard_normal((B, Hq, Sq, D), dtype=np.float32) / np.sqrt(D)).astype(np.float16)
    k = rng.standard_normal((B, Hkv, Sk, D), dtype=np.float32).astype(np.float16)
    v = rng.standard_normal((B, Hkv, Sk, D), dtype=np.float32).astype(np.float16)
    got = tract_amd.Sdpa(datum_type=np.float16, is_causal=causal).eval(q, k, v).to_numpy()
    want = orc.flash_sdpa(q, k, v, causal=causal, threads=8)
    assert not np.isnan(got).any()
    assert max_abs(got, want) <= 2e-2
    assert max_abs(got, cases.textbook_sdpa(q, k, v, causal=causal)) <= 4e-3


@pytest.mark.parametrize("B,Hq,Hkv,Sq,Sk,D,causal", [
    (1, 2, 2, 256, 256, 128, True),       # one head per workgroup (8 query blocks), key splits
    (1, 3, 3, 300, 1000, 128, True),      # ... ragged, last query tile mostly empty
    (1, 4, 2, 128, 640, 128, True),       # two heads per workgroup
    (2, 12, 2, 130, 515, 128, False),     # group of 6: two heads per workgroup, three workgroups per kv head
    (1, 32, 8, 512, 2048, 128, True),     # four heads per workgroup, four key splits (the chunked-prefill shape)
    (1, 8, 2, 64, 4096, 128, True),       # few queries, long cache: 16 key splits
    (1, 8, 2, 33, 65, 128, True),         # second tile of 1 key
    (3, 8, 8, 256, 256, 64, True), (1, 16, 4, 96, 1500, 64, False),
    (16, 32, 8, 64, 64, 128, True),       # enough workgroups without splitting
])
def test_prefill_grouped_heads_and_key_splits(rt, B, Hq, Hkv, Sq, Sk, D, causal):
    rng = np.random.default_rng(2000 + Sq + Sk + Hq)
    q = (rng.standard_normal((B, Hq, Sq, D), dtype=np.float32) / np.sqrt(D)).astype(np.float16)
    k = rng.standard_normal((B, Hkv, Sk, D), dtype=np.float32).astype(np.float16)
    v = rng.standard_normal((B, Hkv, Sk, D), dtype=np.float32).astype(np.float16)
    k[:, :, Sk // 3] *= 6.0   # an outlier key: the running maximum moves late and the splits' maxima differ
    got = tract_amd.Sdpa(datum_type=np.float16, is_causal=causal).eval(q, k, v).to_numpy()
    want = orc.flash_sdpa(q, k, v, causal=causal, threads=8)
    assert not np.isnan(got).any()
    assert max_abs(got, want) <= 2e-2
    assert max_abs(got, cases.textbook_sdpa(q, k, v, causal=causal)) <= 4e-3


@pytest.mark.parametrize("B,Hq,Hkv,Sq,Sk,D,masked", [
    (1, 32, 8, 512, 2048, 128, False),    # four key splits merged by whichever workgroup arrives last
    (2, 32, 8, 848, 848, 128, False),     # two splits
    (2, 32, 8, 848, 848, 128, True),      # the mask-input instantiation
    (1, 8, 2, 64, 4096, 128, False),      # 16 splits: merged two at a time
    (1, 16, 4, 96, 1500, 64, False),
])
def test_prefill_key_splits_give_the_same_bits_every_time(rt, B, Hq, Hkv, Sq, Sk, D, masked):
    """The split that arrives last merges the others and takes its own partial from registers; which one that is
    changes from launch to launch, the output bits must not."""
    rng = np.random.default_rng(2100 + Sq + Sk + Hq)
    q = (rng.standard_normal((B, Hq, Sq, D), dtype=np.float32) / np.sqrt(D)).astype(np.float16)
    k = rng.standard_normal((B, Hkv, Sk, D), dtype=np.float32).astype(np.float16)
    v = rng.standard_normal((B, Hkv, Sk, D), dtype=np.float32).astype(np.float16)
    if masked:
        mask = np.where(np.arange(Sk)[None, :] <= np.arange(Sq)[:, None] + (Sk - Sq), 0.0, -np.inf).astype(np.float16)[None, None]
        op, inputs = tract_amd.Sdpa(datum_type=np.float16), (q, k, v, mask)
    else:
        op, inputs = tract_amd.Sdpa(datum_type=np.float16, is_causal=True), (q, k, v)
    first = op.eval(*inputs).to_numpy()
    assert max_abs(first, cases.textbook_sdpa(q, k, v, causal=True)) <= 4e-3
    for _ in range(12):
        assert op.eval(*inputs).to_numpy().tobytes() == first.tobytes()


@pytest.mark.parametrize("Sq", [2, 3, 5, 8, 17, 31])
@pytest.mark.parametrize("Hq,Hkv,D,T", [(32, 8, 128, 3000), (16, 2, 128, 1100), (8, 4, 64, 777)])
def test_few_queries_over_a_long_cache(rt, Sq, Hq, Hkv, D, T):
    """q_len of a few tokens (speculative decoding, tiny chunks) with grouped heads: served by the MFMA
    kernel that reads K/V once per kv head.  Causal row r must also equal the decode step that sees the
    first T - Sq + r + 1 keys."""
    rng = np.random.default_rng(4000 + Sq + T)
    B = 2
    q = (rng.standard_normal((B, Hq, Sq, D), dtype=np.float32) / np.sqrt(D)).astype(np.float16)
    k = rng.standard_normal((B, Hkv, T, D), dtype=np.float32).astype(np.float16)
    v = rng.standard_normal((B, Hkv, T, D), dtype=np.float32).astype(np.float16)
    got = tract_amd.Sdpa(datum_type=np.float16, is_causal=True).eval(q, k, v).to_numpy()
    assert not np.isnan(got).any()
    assert max_abs(got, orc.flash_sdpa(q, k, v, causal=True, threads=8)) <= 2e-2
    assert max_abs(got, cases.textbook_sdpa(q, k, v, causal=True)) <= 4e-3
    r = Sq // 2
    n = T - Sq + r + 1
    step = tract_amd.Sdpa(datum_type=np.float16).eval(q[:, :, r:r + 1], k[:, :, :n].copy(), v[:, :, :n].copy()).to_numpy()
    assert max_abs(got[:, :, r:r + 1], step) <= 2e-3


@pytest.mark.parametrize("kind", ["random", "causal_min", "causal_inf", "window_inf"])
@pytest.mark.parametrize("B,Hq,Hkv,Sq,Sk,D,mb,mh", [
    (1, 32, 8, 512, 2048, 128, 1, 1),     # the chunked-prefill shape, one mask for all heads, key splits
    (2, 8, 2, 130, 516, 128, 2, 8),       # a mask per batch and head
    (1, 4, 2, 128, 641, 128, 1, 4),       # odd row length: element-wise mask loads
    (2, 12, 2, 77, 302, 128, 2, 1), (3, 8, 8, 256, 256, 64, 1, 1), (1, 16, 4, 96, 1500, 64, 1, 16),
    (1, 2, 2, 256, 256, 128, 1, 2),
])
def test_prefill_with_additive_mask(rt, kind, B, Hq, Hkv, Sq, Sk, D, mb, mh):
    """q_len > 1 with a mask input [mask_b, mask_h, q_len, kv_len] (cuda/src/kernels/flash_attn.rs:138-143),
    served by the MFMA kernel.  A causal mask stated as an input, with the reference's finite minimum
    (sdpa.rs:550-553) or -inf above the diagonal, must reproduce is_causal; a banded (sliding-window)
    mask leaves whole tiles and whole key splits with nothing visible."""
    rng = np.random.default_rng(3000 + Sq + Sk + Hq)
    q = (rng.standard_normal((B, Hq, Sq, D), dtype=np.float32) / np.sqrt(D)).astype(np.float16)
    k = rng.standard_normal((B, Hkv, Sk, D), dtype=np.float32).astype(np.float16)
    v = rng.standard_normal((B, Hkv, Sk, D), dtype=np.float32).astype(np.float16)
    i = np.arange(Sq)[:, None] + (Sk - Sq)
    j = np.arange(Sk)[None, :]
    if kind == "random":
        mask = rng.standard_normal((mb, mh, Sq, Sk), dtype=np.float32) * 3
    else:
        lo = -np.inf if kind.endswith("inf") else float(np.finfo(np.float16).min)
        hidden = j > i
        if kind == "window_inf":
            hidden = hidden | (j < i - 100)
        mask = np.broadcast_to(np.where(hidden, lo, 0.0).astype(np.float32), (mb, mh, Sq, Sk)).copy()
    mask = mask.astype(np.float16)
    got = tract_amd.Sdpa(datum_type=np.float16).eval(q, k, v, mask).to_numpy()
    assert not np.isnan(got).any()
    if kind != "window_inf":
        # (the CPU kernel starts from m = -inf and yields NaN for a row whose first key tile is all -inf
        # while other rows of the tile are not, flash_sdpa.rs:309-316; the band is held to the f64 form)
        assert max_abs(got, orc.flash_sdpa(q, k, v, mask=mask, threads=8)) <= 2e-2
    assert max_abs(got, cases.textbook_sdpa(q, k, v, mask)) <= 4e-3
    if kind.startswith("causal"):
        same = tract_amd.Sdpa(datum_type=np.float16, is_causal=True).eval(q, k, v).to_numpy()
        assert max_abs(got, same) <= 2e-3


@pytest.mark.parametrize("fmt_name", ["Q8_0", "Q4_0"])
@pytest.mark.parametrize("B,Hq,Hkv,D,chunks", [
    (1, 32, 8, 128, (512, 512, 300)),     # chunked prefill into a quantised cache, key splits
    (2, 8, 2, 128, (100, 77, 33)), (1, 4, 4, 128, (64, 200)), (2, 6, 2, 128, (40, 130)),
    (1, 8, 2, 64, (96, 160)), (3, 16, 16, 64, (70,)),
    (1, 8, 8, 128, (300, 5, 2)), (1, 6, 2, 128, (200, 9)),   # a few queries, one head per workgroup
])
def test_prefill_over_a_quantised_cache(rt, fmt_name, B, Hq, Hkv, D, chunks):
    """Chunks of a prompt appended to a Q8_0 / Q4_0 cache (quantised on append), each attending causally
    over the cache so far: the MFMA kernel dequantises the blocks while staging its K/V tiles.  The
    oracle attends over the dequantised blocks (the reference states attention over a block-quantised
    tensor through simulate_precision_loss, block_quant/mod.rs:110-155)."""
    fmt = {"Q8_0": tract_amd.Q8_0, "Q4_0": tract_amd.Q4_0}[fmt_name]
    rng = np.random.default_rng(5000 + Hq + sum(chunks))
    st = tract_amd.InPlaceKvSdpa(axis=2, causal=True, storage_format=fmt).state()
    kd = vd = None
    for S in chunks:
        q = (rng.standard_normal((B, Hq, S, D), dtype=np.float32) / np.sqrt(D)).astype(np.float16)
        k = rng.standard_normal((B, Hkv, S, D), dtype=np.float32).astype(np.float16)
        v = rng.standard_normal((B, Hkv, S, D), dtype=np.float32).astype(np.float16)
        k[:, :, :, 5] *= 12.0   # an outlier channel: blocks with very different scales
        got = st.eval([q, k, v]).to_numpy()
        kq = orc.dequant(fmt, orc.quant(fmt, k), np.float16)
        vq = orc.dequant(fmt, orc.quant(fmt, v), np.float16)
        kd = kq if kd is None else np.concatenate([kd, kq], axis=2)
        vd = vq if vd is None else np.concatenate([vd, vq], axis=2)
        assert not np.isnan(got).any()
        assert max_abs(got, orc.flash_sdpa(q, kd, vd, causal=True, threads=8)) <= 2e-2
        assert max_abs(got, cases.textbook_sdpa(q, kd, vd, causal=True)) <= 4e-3
    # the stored blocks are the oracle's, bit for bit
    want_blocks = orc.quant(fmt, k)   # last chunk
    got_blocks = st.k.valid_contiguous()[:, :, -chunks[-1]:]
    assert got_blocks.tobytes() == want_blocks.tobytes()


def test_f32_prompt_through_the_f16_kernels_like_the_cuda_translator(rt):
    """convert_sdpa_to_cuda_flash_attn (cuda/src/transform.rs:358-406) casts Q, K, V and the mask to f16
    around its kernel and casts the result back: the same option on the Sdpa mirror, held to the f16
    tolerance; without it an f32 prompt keeps f32 arithmetic (generic kernel) and the f32 tolerance."""
    rng = np.random.default_rng(6000)
    B, Hq, Hkv, Sq, Sk, D = 1, 8, 2, 96, 300, 128
    q = (rng.standard_normal((B, Hq, Sq, D), dtype=np.float32) / np.sqrt(D)).astype(np.float32)
    k = rng.standard_normal((B, Hkv, Sk, D), dtype=np.float32)
    v = rng.standard_normal((B, Hkv, Sk, D), dtype=np.float32)
    want = cases.textbook_sdpa(q, k, v, causal=True)
    exact = tract_amd.Sdpa(is_causal=True).eval(q, k, v).to_numpy()
    fast = tract_amd.Sdpa(is_causal=True, f16_flash_attention=True).eval(q, k, v).to_numpy()
    assert exact.dtype == fast.dtype == np.float32
    assert max_abs(exact, want) <= 2e-5
    assert 2e-5 < max_abs(fast, want) <= 2e-2     # f16 arithmetic, as on the reference's GPU path
    mask = (rng.standard_normal((1, 1, Sq, Sk), dtype=np.float32))
    fast = tract_amd.Sdpa(f16_flash_attention=True).eval(q, k, v, mask).to_numpy()
    assert max_abs(fast, cases.textbook_sdpa(q, k, v, mask)) <= 2e-2


_PREFILL_ENV_CODE = """
import os, sys, numpy as np
import tract_amd
tract_amd.runtime_for_name('rocm')
rng=np.random.default_rng(77)
q=(rng.standard_normal((1,32,192,128),dtype=np.float32)/11.3).astype(np.float16)
k=rng.standard_normal((1,8,1100,128),dtype=np.float32).astype(np.float16)
v=rng.standard_normal((1,8,1100,128),dtype=np.float32).astype(np.float16)
o=tract_amd.Sdpa(datum_type=np.float16,is_causal=True).eval(q,k,v).to_numpy()
sys.stdout.buffer.write(o.tobytes())
"""


@pytest.mark.parametrize("env", [{"TROCM_PREFILL_SPLITS": "1"}, {"TROCM_PREFILL_SPLITS": "2"},
                                 {"TROCM_PREFILL_SPLITS": "5"}, {"TROCM_PREFILL_SPLITS": "16"},
                                 {"TROCM_PREFILL_HG": "1"}, {"TROCM_PREFILL_HG": "2"}, {"TROCM_PREFILL_PP": "0"},
                                 {"TROCM_PREFILL_TAIL_MERGE": "0"}, {"TROCM_PREFILL_TAIL_MERGE": "0", "TROCM_PREFILL_SPLITS": "7"},
                                 {"TROCM_PREFILL_PING": "1"}, {"TROCM_PREFILL_PING": "1", "TROCM_PREFILL_SPLITS": "1"},
                                 {"TROCM_PREFILL_PING": "1", "TROCM_PREFILL_HG": "1"}, {"TROCM_PREFILL_PING": "1", "TROCM_PREFILL_HG": "2", "TROCM_PREFILL_SPLITS": "3"}])
def test_prefill_any_split_count_and_head_grouping_agree(rt, env):
    """The key-split merge is exact in real arithmetic and the head grouping only changes which
    workgroup computes a head: every setting must agree with the textbook form.  TROCM_PREFILL_PING=1
    selects the tile loop that loads K/V straight into LDS and alternates two groups of waves between the
    matrix and the vector half of a tile."""
    import subprocess, sys
    e = dict(os.environ)
    e.update(env)
    out = subprocess.run([sys.executable, "-c", _PREFILL_ENV_CODE], capture_output=True, check=True, env=e,
                         cwd=os.path.dirname(os.path.dirname(os.path.abspath(__file__)))).stdout
    got = np.frombuffer(out[-1 * 32 * 192 * 128 * 2:], dtype=np.float16).reshape(1, 32, 192, 128)
    rng = np.random.default_rng(77)
    q = (rng.standard_normal((1, 32, 192, 128), dtype=np.float32) / 11.3).astype(np.float16)
    k = rng.standard_normal((1, 8, 1100, 128), dtype=np.float32).astype(np.float16)
    v = rng.standard_normal((1, 8, 1100, 128), dtype=np.float32).astype(np.float16)
    assert max_abs(got, cases.textbook_sdpa(q, k, v, causal=True)) <= 4e-3


def test_prefill_with_a_workspace_too_small_for_key_splits(rt):
    """A caller may hand over a workspace with room for fewer key splits than the prefill would like, for none
    at all, or no workspace: prefill then runs with fewer splits or unsplit."""
    from tract_amd._lib import call
    from tract_amd.runtime import DeviceTensor, Workspace
    B, Hq, Hkv, Sq, Sk, D = 1, 32, 8, 512, 1024, 128
    rng = np.random.default_rng(4)
    q = (rng.standard_normal((B, Hq, Sq, D), dtype=np.float32) / np.sqrt(D)).astype(np.float16)
    k = rng.standard_normal((B, Hkv, Sk, D), dtype=np.float32).astype(np.float16)
    v = rng.standard_normal((B, Hkv, Sk, D), dtype=np.float32).astype(np.float16)
    full = Workspace.bytes_for(B, Hq, Sq, D)
    small = [DeviceTensor((n,), np.uint8) for n in (full // 2, 80_000)]
    for t in small:
        call("trocm_sdpa_workspace_init", t.ptr, t.shape[0], None)
    dq, dk, dv = (DeviceTensor.from_numpy(t) for t in (q, k, v))
    out = DeviceTensor(q.shape, q.dtype)
    for wsp, wsn in ((small[0].ptr, small[0].shape[0]), (small[1].ptr, small[1].shape[0]), (None, 0)):
        call("trocm_sdpa", dq.ptr, dk.ptr, dv.ptr, None, out.ptr, 1, B, Hq, Hkv, Sq, Sk, D, None, 1, 1,
             float("nan"), 1, wsp, wsn, None)
        assert max_abs(out.to_numpy(), cases.textbook_sdpa(q, k, v, causal=True)) <= 4e-3


def test_chunked_prefill_into_cache_cfg3_reduced(rt):
    """cfg3 (reduced to 8 chunks of 96 tokens): each chunk is appended to the in-place cache,
    then attends causally to the whole cache so far (q_len 96, kv_len 96*c), reading K/V from
    the capacity buffer.  The concatenated outputs equal one causal pass over all tokens."""
    rng = np.random.default_rng(cases.cfg_seed(3, "q"))
    B, Hq, Hkv, D, S, C = 1, 32, 8, 128, 96, 8
    q = (cases.seeded_normal(cases.cfg_seed(3, "q"), (B, Hq, S * C, D)) / np.sqrt(D)).astype(np.float16)
    k = cases.seeded_normal(cases.cfg_seed(3, "k"), (B, Hkv, S * C, D), np.float16)
    v = cases.seeded_normal(cases.cfg_seed(3, "v"), (B, Hkv, S * C, D), np.float16)
    st = tract_amd.InPlaceKvSdpa(axis=2, causal=True).state()
    outs = []
    for c in range(C):
        sl = slice(c * S, (c + 1) * S)
        outs.append(st.eval([q[:, :, sl], k[:, :, sl], v[:, :, sl]]).to_numpy())
        assert st.k.len() == (c + 1) * S
    got = np.concatenate(outs, axis=2)
    assert st.k.capacity() == 768 and st.k.reallocs() == 3
    assert st.k.valid_contiguous().tobytes() == k.tobytes()
    want = orc.flash_sdpa(q, k, v, causal=True, threads=8)
    assert max_abs(got, want) <= 2e-2
    # chunk c on its own against the oracle with the bottom-right aligned causal rule
    c = 5
    one = orc.flash_sdpa(q[:, :, c * S:(c + 1) * S], k[:, :, :(c + 1) * S], v[:, :, :(c + 1) * S], causal=True, threads=8)
    assert max_abs(outs[c], one) <= 2e-2


@pytest.mark.parametrize("dt,Hq,Hkv,D", [(np.float16, 32, 8, 128), (np.float32, 8, 8, 64), (np.float16, 6, 2, 128)])
def test_fused_step_appends_in_the_attention_launch(rt, dt, Hq, Hkv, D):
    """InPlaceKvSdpaState::eval as ONE call per step: the new token is read from the inputs and
    stored into the cache by the decode kernel.  Cache bytes must stay identical to concat and
    the output must match the oracle, across tile boundaries and across a capacity doubling."""
    rng = np.random.default_rng(2024)
    B, T0 = 2, 29
    k = rng.standard_normal((B, Hkv, T0, D), dtype=np.float32).astype(dt)
    v = rng.standard_normal((B, Hkv, T0, D), dtype=np.float32).astype(dt)
    st = tract_amd.InPlaceKvSdpa(axis=2, causal=True).state()
    st.k.push(k), st.v.push(v)
    kc, vc = k, v
    for step in range(40):  # 29 -> 69 tokens: crosses tiles of 32 and the 29 -> 58 -> 116 doublings
        q = (rng.standard_normal((B, Hq, 1, D), dtype=np.float32) / np.sqrt(D)).astype(dt)
        kn = rng.standard_normal((B, Hkv, 1, D), dtype=np.float32).astype(dt)
        vn = rng.standard_normal((B, Hkv, 1, D), dtype=np.float32).astype(dt)
        out = st.eval([q, kn, vn]).to_numpy()
        kc, vc = orc.concat_append(kc, kn, 2), orc.concat_append(vc, vn, 2)
        assert st.k.len() == kc.shape[2] == st.v.len()
        assert max_abs(out, orc.flash_sdpa(q, kc, vc, causal=True)) <= TOL[np.dtype(dt)], f"step {step}"
        if step % 7 == 0 or step == 39:
            assert st.k.valid_contiguous().tobytes() == kc.tobytes()
            assert st.v.valid_contiguous().tobytes() == vc.tobytes()
    assert st.k.capacity() == 116 and st.k.reallocs() == 2


def test_fused_ragged_step(rt):
    rng = np.random.default_rng(4242)
    Hq, Hkv, D, n_seq = 32, 8, 128, 9
    lens = [1, 31, 32, 33, 63, 64, 500, 1000, 2047]
    pool = tract_amd.KvPool(64 << 20)
    kcs, vcs, ks, vs = [], [], [], []
    for n in lens:
        k = rng.standard_normal((1, Hkv, n, D), dtype=np.float32).astype(np.float16)
        v = rng.standard_normal((1, Hkv, n, D), dtype=np.float32).astype(np.float16)
        kc, vc = tract_amd.InPlaceKvCache(2, pool=pool), tract_amd.InPlaceKvCache(2, pool=pool)
        kc.push(k), vc.push(v)
        kcs.append(kc), vcs.append(vc), ks.append(k), vs.append(v)
    ws = tract_amd.Workspace(n_seq, Hq, 1, D)
    for step in range(3):
        q = (rng.standard_normal((n_seq, Hq, 1, D), dtype=np.float32) / np.sqrt(D)).astype(np.float16)
        kn = rng.standard_normal((n_seq, Hkv, 1, D), dtype=np.float32).astype(np.float16)
        vn = rng.standard_normal((n_seq, Hkv, 1, D), dtype=np.float32).astype(np.float16)
        out = tract_amd.inplace_kv_sdpa_eval_ragged(
            tract_amd.DeviceTensor.from_numpy(q), tract_amd.DeviceTensor.from_numpy(kn),
            tract_amd.DeviceTensor.from_numpy(vn), kcs, vcs, workspace=ws).to_numpy()
        for i in range(n_seq):
            ks[i] = np.concatenate([ks[i], kn[i:i + 1]], axis=2)
            vs[i] = np.concatenate([vs[i], vn[i:i + 1]], axis=2)
            assert kcs[i].len() == ks[i].shape[2]
            assert max_abs(out[i:i + 1], orc.flash_sdpa(q[i:i + 1], ks[i], vs[i], causal=True)) <= 2e-2
    for i in range(n_seq):
        assert kcs[i].valid_contiguous().tobytes() == ks[i].tobytes()
        assert vcs[i].valid_contiguous().tobytes() == vs[i].tobytes()
    # quantised caches take the explicit-append route behind the same call
    qk, qv = tract_amd.InPlaceKvCache(2, storage_format=tract_amd.Q8_0), tract_amd.InPlaceKvCache(2, storage_format=tract_amd.Q8_0)
    qk.push(ks[6]), qv.push(vs[6])
    q1 = (rng.standard_normal((1, Hq, 1, D), dtype=np.float32) / np.sqrt(D)).astype(np.float16)
    kn = rng.standard_normal((1, Hkv, 1, D), dtype=np.float32).astype(np.float16)
    out = tract_amd.inplace_kv_sdpa_eval_ragged(tract_amd.DeviceTensor.from_numpy(q1), tract_amd.DeviceTensor.from_numpy(kn),
                                                tract_amd.DeviceTensor.from_numpy(kn), [qk], [qv]).to_numpy()
    kd = orc.dequant(orc.FMT_Q8_0, orc.quant(orc.FMT_Q8_0, np.concatenate([ks[6], kn], axis=2)), np.float16)
    vd = orc.dequant(orc.FMT_Q8_0, orc.quant(orc.FMT_Q8_0, np.concatenate([vs[6], kn], axis=2)), np.float16)
    assert qk.len() == ks[6].shape[2] + 1 and max_abs(out, orc.flash_sdpa(q1, kd, vd, causal=True)) <= 2e-2
