"""The configurations at their full step counts, and the split merge under many back-to-back launches.

cfg2: caches prefilled to 8192 tokens, then 128 single-token steps (append + decode attention) at batch 1
(every step against the oracle) and batch 8 (every 16th step), final cache bytes against concatenation.
cfg5: 64 ragged sequences in one pool, 64 fused steps; a rotating sample of sequences against the batch-1
oracle at every step, every cache's bytes at the end.
Merge ordering: thousands of consecutive launches on ONE workspace, a different query each launch, at the
split counts the benchmark runs (4 at batch 8, 32 at batch 1; 16 key splits for prefill), each output against
the same launch without a workspace (one split: nothing to merge), within a few f16 units of outputs of order 1."""
import ctypes as C
import hashlib

import numpy as np
import pytest

import tract_amd as ta
from oracle import oracle as orc
from tests import cases
from tests.gpu_util import max_abs, rt  # noqa: F401
from tract_amd._lib import call
from tract_amd.runtime import DeviceTensor, Workspace

pytestmark = pytest.mark.gpu

HQ, HKV, D = 32, 8, 128
NAN = C.c_float(float("nan"))
ONE = C.c_float(1.0)   # softmax scale of the merge tests: their queries carry the sharpness themselves


def _sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).digest()


@pytest.mark.parametrize("B,check_every", [(1, 1), (8, 16)])
def test_cfg2_128_steps_at_8192(rt, B, check_every):
    T, steps = 8192, 128
    kh = np.empty((B, HKV, T + steps, D), np.float16)   # the host's copy of the caches, grown in place
    vh = np.empty((B, HKV, T + steps, D), np.float16)
    for b in range(B):
        kh[b, :, :T] = cases.seeded_normal(cases.cfg_seed(2, "k") + 1000 * b, (HKV, T, D), np.float16)
        vh[b, :, :T] = cases.seeded_normal(cases.cfg_seed(2, "v") + 1000 * b, (HKV, T, D), np.float16)
    st = ta.InPlaceKvSdpa(axis=2, causal=True).state()
    st.k.push(np.ascontiguousarray(kh[:, :, :T])), st.v.push(np.ascontiguousarray(vh[:, :, :T]))
    q_all = (cases.seeded_normal(cases.cfg_seed(2, "q"), (steps, B, HQ, 1, D)) / np.sqrt(D)).astype(np.float16)
    k_all = cases.seeded_normal(cases.cfg_seed(2, "k") + 7, (steps, B, HKV, 1, D), np.float16)
    v_all = cases.seeded_normal(cases.cfg_seed(2, "v") + 7, (steps, B, HKV, 1, D), np.float16)
    worst = 0.0
    for s in range(steps):
        out = st.eval([q_all[s], k_all[s], v_all[s]]).to_numpy()
        kh[:, :, T + s], vh[:, :, T + s] = k_all[s][:, :, 0], v_all[s][:, :, 0]
        if s % check_every == 0 or s == steps - 1:
            n = T + s + 1
            want = orc.flash_sdpa(q_all[s], np.ascontiguousarray(kh[:, :, :n]), np.ascontiguousarray(vh[:, :, :n]), causal=True, threads=8)
            err = max_abs(out, want)
            worst = max(worst, err)
            assert err <= 2e-2, f"step {s}: {err}"
    assert (st.k.len(), st.k.capacity(), st.k.reallocs()) == (T + steps, 2 * T, 1)
    assert (st.v.len(), st.v.capacity(), st.v.reallocs()) == (T + steps, 2 * T, 1)
    assert _sha(st.k.valid_contiguous()) == _sha(kh)
    assert _sha(st.v.valid_contiguous()) == _sha(vh)
    assert worst <= 2e-3   # in practice an order of magnitude inside the bar


def test_cfg2_batch_32_fused_steps_at_8192(rt):
    """cfg2's largest batch: 32 sequences prefilled to 8192 tokens (1 GiB of K and V), 32 fused steps (the first one
    doubles both capacities).  Sequences 3 and 29 against the oracle on their own caches every 16 steps and at the
    end, the final caches of all 32 sequences against the concatenation by hash."""
    B, T, steps, watch = 32, 8192, 32, (3, 29)
    kh = np.empty((B, HKV, T + steps, D), np.float16)
    vh = np.empty((B, HKV, T + steps, D), np.float16)
    for b in range(B):
        kh[b, :, :T] = cases.seeded_normal(cases.cfg_seed(2, "k") + 1000 * b, (HKV, T, D), np.float16)
        vh[b, :, :T] = cases.seeded_normal(cases.cfg_seed(2, "v") + 1000 * b, (HKV, T, D), np.float16)
    st = ta.InPlaceKvSdpa(axis=2, causal=True).state()
    st.k.push(np.ascontiguousarray(kh[:, :, :T])), st.v.push(np.ascontiguousarray(vh[:, :, :T]))
    q_all = (cases.seeded_normal(cases.cfg_seed(2, "q") + 32, (steps, B, HQ, 1, D)) / np.sqrt(D)).astype(np.float16)
    k_all = cases.seeded_normal(cases.cfg_seed(2, "k") + 39, (steps, B, HKV, 1, D), np.float16)
    v_all = cases.seeded_normal(cases.cfg_seed(2, "v") + 39, (steps, B, HKV, 1, D), np.float16)
    worst = 0.0
    for s in range(steps):
        out = st.eval([q_all[s], k_all[s], v_all[s]]).to_numpy()
        kh[:, :, T + s], vh[:, :, T + s] = k_all[s][:, :, 0], v_all[s][:, :, 0]
        if s % 16 == 0 or s == steps - 1:
            n = T + s + 1
            for b in watch:
                want = orc.flash_sdpa(q_all[s][b:b + 1], np.ascontiguousarray(kh[b:b + 1, :, :n]), np.ascontiguousarray(vh[b:b + 1, :, :n]),
                                      causal=True, threads=8)
                err = max_abs(out[b:b + 1], want)
                worst = max(worst, err)
                assert err <= 2e-2, f"step {s}, sequence {b}: {err}"
    assert (st.k.len(), st.k.capacity(), st.k.reallocs()) == (T + steps, 2 * T, 1)
    assert (st.v.len(), st.v.capacity(), st.v.reallocs()) == (T + steps, 2 * T, 1)
    assert _sha(st.k.valid_contiguous()) == _sha(kh)
    assert _sha(st.v.valid_contiguous()) == _sha(vh)
    assert worst <= 2e-3


def test_cfg5_64_sequences_64_fused_steps(rt):
    n_seq, steps, per_step = 64, 64, 3
    rng = np.random.default_rng(cases.cfg_seed(5, "len"))
    lens = [int(x) for x in rng.integers(512, 32768, size=n_seq, endpoint=True)]
    pool = ta.KvPool(sum(lens) * HKV * D * 2 * 2 * 3 + (64 << 20))
    kcs, vcs, ks, vs = [], [], [], []
    for i, t in enumerate(lens):
        k = np.empty((1, HKV, t + steps, D), np.float16)
        v = np.empty((1, HKV, t + steps, D), np.float16)
        k[:, :, :t] = cases.seeded_normal(cases.cfg_seed(5, "k") + i, (1, HKV, t, D), np.float16)
        v[:, :, :t] = cases.seeded_normal(cases.cfg_seed(5, "v") + i, (1, HKV, t, D), np.float16)
        kc, vc = ta.InPlaceKvCache(2, pool=pool), ta.InPlaceKvCache(2, pool=pool)
        kc.push(np.ascontiguousarray(k[:, :, :t])), vc.push(np.ascontiguousarray(v[:, :, :t]))
        kcs.append(kc), vcs.append(vc), ks.append(k), vs.append(v)
    ws = Workspace(n_seq, HQ, 1, D)
    order = np.random.default_rng(1).permutation(n_seq * per_step) % n_seq   # every sequence is checked about 3 times
    for s in range(steps):
        q = (cases.seeded_normal(cases.cfg_seed(5, "q") + s, (n_seq, HQ, 1, D)) / np.sqrt(D)).astype(np.float16)
        kn = cases.seeded_normal(900 + s, (n_seq, HKV, 1, D), np.float16)
        vn = cases.seeded_normal(1900 + s, (n_seq, HKV, 1, D), np.float16)
        out = ta.inplace_kv_sdpa_eval_ragged(DeviceTensor.from_numpy(q), DeviceTensor.from_numpy(kn), DeviceTensor.from_numpy(vn),
                                             kcs, vcs, workspace=ws).to_numpy()
        for i in range(n_seq):
            ks[i][0, :, lens[i] + s], vs[i][0, :, lens[i] + s] = kn[i, :, 0], vn[i, :, 0]
        assert np.isfinite(out.astype(np.float32)).all(), f"step {s}"
        for i in order[s * per_step:(s + 1) * per_step]:
            n = lens[i] + s + 1
            want = orc.flash_sdpa(q[i:i + 1], np.ascontiguousarray(ks[i][:, :, :n]), np.ascontiguousarray(vs[i][:, :, :n]),
                                  causal=True, threads=8)
            assert max_abs(out[i:i + 1], want) <= 2e-2, f"step {s}, sequence {i} of {n} tokens"
    for i in range(n_seq):
        cap = lens[i] * 2 if steps <= lens[i] else None
        assert kcs[i].len() == lens[i] + steps and vcs[i].len() == lens[i] + steps
        assert cap is None or (kcs[i].capacity() == cap and kcs[i].reallocs() == 1)
        assert _sha(kcs[i].valid_contiguous()) == _sha(ks[i]), f"K cache of sequence {i}"
        assert _sha(vcs[i].valid_contiguous()) == _sha(vs[i]), f"V cache of sequence {i}"


def _decode_many(B, T, launches, n_queries=64):
    """`launches` decode launches back to back on one workspace, launch j with query j % n_queries into its own
    output row; then the same queries without a workspace (a single split per sequence-head)."""
    rng = np.random.default_rng(B * 1000 + T)
    k = rng.standard_normal((B, HKV, T, D), dtype=np.float32).astype(np.float16)
    v = rng.standard_normal((B, HKV, T, D), dtype=np.float32).astype(np.float16)
    st = ta.InPlaceKvSdpa(axis=2, causal=True).state()
    st.k.push(k), st.v.push(v)
    q = (rng.standard_normal((n_queries, B, HQ, 1, D), dtype=np.float32) * (8.0 / np.sqrt(D))).astype(np.float16)
    qd = DeviceTensor.from_numpy(q)
    row = B * HQ * D * 2
    got = DeviceTensor((launches, B, HQ, 1, D), np.float16)
    call("trocm_memset", got.ptr, 0xFF, got.nbytes, None)
    ws = Workspace(B, HQ, 1, D)
    for j in range(launches):
        call("trocm_sdpa_cached", C.c_void_p(qd.ptr.value + (j % n_queries) * row), ta.F16, HQ, 1, st.k.handle, st.v.handle,
             C.c_void_p(got.ptr.value + j * row), ONE, 1, ws.ptr, ws.nbytes, None)
    ref = DeviceTensor((n_queries, B, HQ, 1, D), np.float16)
    for j in range(n_queries):
        call("trocm_sdpa_cached", C.c_void_p(qd.ptr.value + j * row), ta.F16, HQ, 1, st.k.handle, st.v.handle,
             C.c_void_p(ref.ptr.value + j * row), ONE, 1, None, 0, None)
    return got.to_numpy(), ref.to_numpy(), (q, k, v)


@pytest.mark.parametrize("B,T,launches", [(8, 8200, 2400), (1, 8200, 2400), (2, 4100, 1200)])
def test_split_merge_over_many_launches_on_one_workspace(rt, B, T, launches):
    """A partial record read before its store had landed would be the previous launch's, i.e. another
    query's: every launch's output must be its own query's result."""
    got, ref, (q, k, v) = _decode_many(B, T, launches)
    n_queries = ref.shape[0]
    # the single-split reference itself, on a few queries, against the oracle
    for j in (0, n_queries - 1):
        assert max_abs(ref[j], orc.flash_sdpa(q[j], k, v, causal=True, scale=1.0, threads=8)) <= 2e-2
    # sharp softmaxes (logits of standard deviation 8): distinct queries give outputs of order 1 that differ by
    # order 1, so one stale record among the splits would be off by a hundred times the tolerance
    assert max_abs(ref[0], ref[1]) > 0.5
    for j in range(launches):
        err = max_abs(got[j], ref[j % n_queries])
        assert err <= 4e-3, f"launch {j} (query {j % n_queries}): max-abs {err} against the single-split result"


def test_prefill_split_merge_over_many_launches_on_one_workspace(rt):
    """The same for the prefill kernel's key splits (16 workgroups per query tile here) and its last-arriver merge."""
    B, Hq, Hkv, Sq, Sk, launches, n_queries = 1, 32, 8, 128, 4096, 400, 8
    rng = np.random.default_rng(99)
    k = rng.standard_normal((B, Hkv, Sk, D), dtype=np.float32).astype(np.float16)
    v = rng.standard_normal((B, Hkv, Sk, D), dtype=np.float32).astype(np.float16)
    st = ta.InPlaceKvSdpa(axis=2, causal=True).state()
    st.k.push(k), st.v.push(v)
    q = (rng.standard_normal((n_queries, B, Hq, Sq, D), dtype=np.float32) * (8.0 / np.sqrt(D))).astype(np.float16)
    qd = DeviceTensor.from_numpy(q)
    row = B * Hq * Sq * D * 2
    got = DeviceTensor((launches, B, Hq, Sq, D), np.float16)
    call("trocm_memset", got.ptr, 0xFF, got.nbytes, None)
    ws = Workspace(B, Hq, Sq, D)
    for j in range(launches):
        call("trocm_sdpa_cached", C.c_void_p(qd.ptr.value + (j % n_queries) * row), ta.F16, Hq, Sq, st.k.handle, st.v.handle,
             C.c_void_p(got.ptr.value + j * row), ONE, 1, ws.ptr, ws.nbytes, None)
    ref = DeviceTensor((n_queries, B, Hq, Sq, D), np.float16)
    for j in range(n_queries):
        call("trocm_sdpa_cached", C.c_void_p(qd.ptr.value + j * row), ta.F16, Hq, Sq, st.k.handle, st.v.handle,
             C.c_void_p(ref.ptr.value + j * row), ONE, 1, None, 0, None)
    got, ref = got.to_numpy(), ref.to_numpy()
    want = orc.flash_sdpa(q[0][:, :4], k[:, :1], v[:, :1], causal=True, scale=1.0, threads=8)
    assert max_abs(ref[0][:, :4], want) <= 2e-2
    assert max_abs(ref[0], ref[1]) > 0.5
    for j in range(launches):
        err = max_abs(got[j], ref[j % n_queries])
        assert err <= 8e-3, f"launch {j}: max-abs {err} against the unsplit result"   # partial outputs travel as f16
