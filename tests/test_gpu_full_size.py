"""Parity at the full sizes of the benchmark configurations: the oracle where it finishes in
seconds (decode is one query row per head), size-independent properties elsewhere."""
import hashlib

import numpy as np
import pytest

import tract_amd
from oracle import oracle as orc
from tests import cases
from tests.gpu_util import max_abs, rt  # noqa: F401

pytestmark = pytest.mark.gpu

HQ, HKV, D = 32, 8, 128


def _prefill(B, T, fmt=None, seed=0):
    k = np.empty((B, HKV, T, D), np.float16)
    v = np.empty((B, HKV, T, D), np.float16)
    for b in range(B):
        k[b] = cases.seeded_normal(cases.cfg_seed(2, "k") + seed + 1000 * b, (HKV, T, D), np.float16)
        v[b] = cases.seeded_normal(cases.cfg_seed(2, "v") + seed + 1000 * b, (HKV, T, D), np.float16)
    st = tract_amd.InPlaceKvSdpa(axis=2, causal=True, storage_format=fmt).state()
    st.k.push(k), st.v.push(v)
    return st, k, v


def test_cfg2_full_size_decode_b8_ctx8192(rt):
    """cfg2 at full size: cache prefilled to 8192 tokens, single-token steps; every step's output
    against the oracle on the concatenated cache, the final cache bytes against concat."""
    B, T = 8, 8192
    st, k, v = _prefill(B, T)
    kc, vc = k, v
    for step in range(5):
        q = (cases.seeded_normal(cases.cfg_seed(2, "q") + step, (B, HQ, 1, D)) / np.sqrt(D)).astype(np.float16)
        kn = cases.seeded_normal(cases.cfg_seed(2, "k") + 7 + step, (B, HKV, 1, D), np.float16)
        vn = cases.seeded_normal(cases.cfg_seed(2, "v") + 7 + step, (B, HKV, 1, D), np.float16)
        out = st.eval([q, kn, vn]).to_numpy()
        kc, vc = np.concatenate([kc, kn], axis=2), np.concatenate([vc, vn], axis=2)
        want = orc.flash_sdpa(q, kc, vc, causal=True, threads=8)
        assert max_abs(out, want) <= 2e-2
        assert max_abs(out, cases.textbook_sdpa(q, kc, vc)) <= 2e-3
    assert (st.k.len(), st.k.capacity(), st.k.reallocs()) == (T + 5, 2 * T, 1)
    assert hashlib.sha256(st.k.valid_contiguous().tobytes()).digest() == hashlib.sha256(kc.tobytes()).digest()
    assert hashlib.sha256(st.v.valid_contiguous().tobytes()).digest() == hashlib.sha256(vc.tobytes()).digest()


def test_cfg2_full_size_properties_b32(rt):
    """Batch 32 at 8192 tokens (1 GiB of K and V): properties that need no oracle at this size —
    identical sequences give identical rows; q heads of a group with equal queries agree; a
    zero query averages V; batch entries are independent of their neighbours."""
    B, T = 32, 8192
    k1 = cases.seeded_normal(11, (1, HKV, T, D), np.float16)
    v1 = cases.seeded_normal(12, (1, HKV, T, D), np.float16)
    st = tract_amd.InPlaceKvSdpa(axis=2, causal=True).state()
    st.k.push(np.ascontiguousarray(np.broadcast_to(k1, (B, HKV, T, D))))
    st.v.push(np.ascontiguousarray(np.broadcast_to(v1, (B, HKV, T, D))))
    q1 = (cases.seeded_normal(13, (1, HKV, 1, D)) / np.sqrt(D)).astype(np.float16)
    q = np.ascontiguousarray(np.broadcast_to(np.repeat(q1, HQ // HKV, axis=1), (B, HQ, 1, D))).copy()
    q[5] = 0  # zero query: uniform weights
    out = st.attend(tract_amd.DeviceTensor.from_numpy(q)).to_numpy()
    ref = orc.flash_sdpa(q[:1], k1, v1, causal=True, threads=8)
    assert max_abs(out[0:1], ref) <= 2e-2
    for b in range(B):
        if b != 5:
            assert np.array_equal(out[b], out[0]), f"batch {b} differs from batch 0 on identical inputs"
    g = HQ // HKV
    for h in range(HKV):
        for j in range(1, g):
            assert np.array_equal(out[0, h * g + j], out[0, h * g])
    mean_v = np.repeat(v1[0].astype(np.float32).mean(axis=1), g, axis=0)
    assert max_abs(out[5, :, 0], mean_v) <= 2e-3


def test_cfg3_full_size_chunked_prefill(rt):
    """cfg3 at full size: 8 chunks of 512 tokens; each chunk's output against the oracle
    (causal, bottom-right aligned) on a sample of heads, and chunk 8 == rows of a one-shot
    causal pass (decode/prefill consistency)."""
    S, C = 512, 8
    q = (cases.seeded_normal(cases.cfg_seed(3, "q"), (1, HQ, S * C, D)) / np.sqrt(D)).astype(np.float16)
    k = cases.seeded_normal(cases.cfg_seed(3, "k"), (1, HKV, S * C, D), np.float16)
    v = cases.seeded_normal(cases.cfg_seed(3, "v"), (1, HKV, S * C, D), np.float16)
    st = tract_amd.InPlaceKvSdpa(axis=2, causal=True).state()
    heads = [0, 5, 31]  # q heads 0, 5, 31 -> kv heads 0, 1, 7
    for c in range(C):
        sl = slice(c * S, (c + 1) * S)
        out = st.eval([q[:, :, sl], k[:, :, sl], v[:, :, sl]]).to_numpy()
        if c in (0, 3, 7):
            for h in heads:
                kh = h // 4
                want = orc.flash_sdpa(q[:, h:h + 1, sl], k[:, kh:kh + 1, :(c + 1) * S], v[:, kh:kh + 1, :(c + 1) * S],
                                      causal=True, threads=8)
                assert max_abs(out[:, h:h + 1], want) <= 2e-2, f"chunk {c} head {h}"
    assert (st.k.len(), st.k.capacity(), st.k.reallocs()) == (4096, 4096, 3)
    assert st.k.valid_contiguous().tobytes() == k.tobytes()
    # a decode step on top of the prefilled cache equals the matching row of a longer causal pass
    qd = (cases.seeded_normal(5, (1, HQ, 1, D)) / np.sqrt(D)).astype(np.float16)
    kn, vn = cases.seeded_normal(6, (1, HKV, 1, D), np.float16), cases.seeded_normal(7, (1, HKV, 1, D), np.float16)
    got = st.eval([qd, kn, vn]).to_numpy()
    want = orc.flash_sdpa(qd, np.concatenate([k, kn], 2), np.concatenate([v, vn], 2), causal=True, threads=8)
    assert max_abs(got, want) <= 2e-2


def _with_outlier_channels(x, chan):
    """1 % of the kv_heads * head_dim channels scaled by 20, the same channels for every token."""
    B, H, T, Dh = x.shape
    f = x.transpose(0, 2, 1, 3).reshape(B, T, H * Dh).copy()
    f[:, :, chan] *= 20
    return np.ascontiguousarray(f.reshape(B, T, H, Dh).transpose(0, 2, 1, 3)).astype(np.float16)


@pytest.mark.parametrize("fmt_name,T", [("Q8_0", 16384), ("Q4_0", 16384), ("Q8_0", 4096), ("Q4_0", 4096)])
def test_cfg4_full_size_quantised(rt, fmt_name, T):
    """cfg4 at full size (batch 8), K and V different tensors: blocks bit-exact via a checksum of
    checksums per sequence and tensor, decode vs the oracle over the dequantised blocks (a swap of the
    K and V planes or of their scales would fail either)."""
    B = 8
    dev_fmt, orc_fmt = getattr(tract_amd, fmt_name), getattr(orc, "FMT_" + fmt_name)
    rng = np.random.default_rng(cases.cfg_seed(4, "chan"))
    chan = rng.choice(HKV * D, size=10, replace=False)
    k = _with_outlier_channels(cases.seeded_normal(cases.cfg_seed(4, "k"), (B, HKV, T, D)), chan)
    v = _with_outlier_channels(cases.seeded_normal(cases.cfg_seed(4, "v"), (B, HKV, T, D)), chan)
    st = tract_amd.InPlaceKvSdpa(axis=2, causal=True, storage_format=dev_fmt).state()
    st.k.push(k), st.v.push(v)
    kq, vq = orc.quant(orc_fmt, k), orc.quant(orc_fmt, v)
    for name, got, want in (("K", st.k.valid_contiguous(), kq), ("V", st.v.valid_contiguous(), vq)):
        for b in range(B):
            assert hashlib.sha256(got[b].tobytes()).digest() == hashlib.sha256(want[b].tobytes()).digest(), f"{name}, sequence {b}"
    q = (cases.seeded_normal(cases.cfg_seed(4, "q"), (B, HQ, 1, D)) / np.sqrt(D)).astype(np.float16)
    out = st.attend(tract_amd.DeviceTensor.from_numpy(q)).to_numpy()
    kd, vd = orc.dequant(orc_fmt, kq, np.float16), orc.dequant(orc_fmt, vq, np.float16)
    assert max_abs(out, orc.flash_sdpa(q, kd, vd, causal=True, threads=8)) <= 2e-2
    # and a fused step on top: the new token quantised on append, then attended to
    kn = _with_outlier_channels(cases.seeded_normal(31, (B, HKV, 1, D)), chan)
    vn = _with_outlier_channels(cases.seeded_normal(32, (B, HKV, 1, D)), chan)
    out = st.eval([q, kn, vn]).to_numpy()
    kd = np.concatenate([kd, orc.dequant(orc_fmt, orc.quant(orc_fmt, kn), np.float16)], axis=2)
    vd = np.concatenate([vd, orc.dequant(orc_fmt, orc.quant(orc_fmt, vn), np.float16)], axis=2)
    assert max_abs(out, orc.flash_sdpa(q, kd, vd, causal=True, threads=8)) <= 2e-2
    assert st.k.valid_contiguous()[:, :, T:].tobytes() == orc.quant(orc_fmt, kn).tobytes()
    assert st.v.valid_contiguous()[:, :, T:].tobytes() == orc.quant(orc_fmt, vn).tobytes()


def test_cfg5_ragged_long_sequences(rt):
    """cfg5's length range (512..32768) on 12 sequences in one pool: fused append + decode steps,
    each sequence against the batch-1 oracle; lengths straddle capacity doublings."""
    rng = np.random.default_rng(cases.cfg_seed(5, "len"))
    lens = [512, 32768, 4096, 4095, 4097] + [int(x) for x in rng.integers(512, 32768, size=7, endpoint=True)]
    n = len(lens)
    pool = tract_amd.KvPool(sum(lens) * HKV * D * 2 * 2 * 3 + (32 << 20))
    kcs, vcs, ks, vs = [], [], [], []
    for i, t in enumerate(lens):
        k = cases.seeded_normal(cases.cfg_seed(5, "k") + i, (1, HKV, t, D), np.float16)
        v = cases.seeded_normal(cases.cfg_seed(5, "v") + i, (1, HKV, t, D), np.float16)
        kc, vc = tract_amd.InPlaceKvCache(2, pool=pool), tract_amd.InPlaceKvCache(2, pool=pool)
        kc.push(k), vc.push(v)
        kcs.append(kc), vcs.append(vc), ks.append(k), vs.append(v)
    ws = tract_amd.Workspace(n, HQ, 1, D)
    for step in range(2):
        q = (cases.seeded_normal(cases.cfg_seed(5, "q") + step, (n, HQ, 1, D)) / np.sqrt(D)).astype(np.float16)
        kn = cases.seeded_normal(900 + step, (n, HKV, 1, D), np.float16)
        vn = cases.seeded_normal(950 + step, (n, HKV, 1, D), np.float16)
        out = tract_amd.inplace_kv_sdpa_eval_ragged(tract_amd.DeviceTensor.from_numpy(q), tract_amd.DeviceTensor.from_numpy(kn),
                                                    tract_amd.DeviceTensor.from_numpy(vn), kcs, vcs, workspace=ws).to_numpy()
        for i in range(n):
            ks[i], vs[i] = np.concatenate([ks[i], kn[i:i + 1]], 2), np.concatenate([vs[i], vn[i:i + 1]], 2)
            assert max_abs(out[i:i + 1], orc.flash_sdpa(q[i:i + 1], ks[i], vs[i], causal=True, threads=8)) <= 2e-2, f"seq {i}"
    for i in range(n):
        assert kcs[i].len() == lens[i] + 2 and kcs[i].capacity() == 2 * lens[i] and kcs[i].reallocs() == 1
        assert hashlib.sha256(kcs[i].valid_contiguous().tobytes()).digest() == hashlib.sha256(ks[i].tobytes()).digest()
