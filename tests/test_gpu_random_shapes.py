"""Seeded random shapes through the decode-step entry points: batch, heads per kv head, head size, storage format,
prefill length (around the 32-token tile boundaries) and step count are drawn per case; after every step the cache
bytes equal the CPU restatement's and the output its attention over them."""
import numpy as np
import pytest

import tract_amd
from oracle import oracle as orc
from tests.gpu_util import rt  # noqa: F401

pytestmark = pytest.mark.gpu


def _blocks(fmtn, x):
    if fmtn == "f16":
        return x.tobytes(), x
    of = getattr(orc, "FMT_" + fmtn)
    q = orc.quant(of, x)
    return q.tobytes(), orc.dequant(of, q, np.float16)


@pytest.mark.parametrize("seed", range(6))
def test_dense_steps_on_random_shapes(rt, seed):
    for it in range(8):
        rng = np.random.default_rng(1000 * seed + it)
        D = int(rng.choice([128, 128, 128, 64]))
        fmtn = str(rng.choice(["f16", "Q8_0", "Q4_0"])) if D == 128 else "f16"
        Hkv, g, B = int(rng.choice([1, 2, 3, 8])), int(rng.choice([1, 2, 3, 4, 5, 8, 12, 16])), int(rng.choice([1, 2, 3, 8]))
        T0 = int(rng.choice([0, 1, 5, 31, 32, 33, 63, 64, 65, 200, 511, 1000, 2049]))
        n0 = int(rng.choice([1, 1, 2, 7]))   # tokens of the first call after the prefill (1: a decode step)
        where = f"seed {seed} case {it}: B={B} Hq={Hkv * g} Hkv={Hkv} D={D} T0={T0} {fmtn} n0={n0}"
        st = tract_amd.InPlaceKvSdpa(axis=2, causal=True, storage_format=None if fmtn == "f16" else getattr(tract_amd, fmtn)).state()
        ks = rng.standard_normal((B, Hkv, T0, D), dtype=np.float32).astype(np.float16)
        vs = rng.standard_normal((B, Hkv, T0, D), dtype=np.float32).astype(np.float16)
        if T0:
            st.k.push(ks), st.v.push(vs)
        for s in range(int(rng.integers(1, 4))):
            n = n0 if s == 0 else 1
            q = (rng.standard_normal((B, Hkv * g, n, D), dtype=np.float32) / np.sqrt(D)).astype(np.float16)
            kn = (rng.standard_normal((B, Hkv, n, D), dtype=np.float32) * rng.choice([1.0, 1.0, 8.0])).astype(np.float16)
            vn = rng.standard_normal((B, Hkv, n, D), dtype=np.float32).astype(np.float16)
            out = st.eval([q, kn, vn]).to_numpy()
            ks, vs = np.concatenate([ks, kn], axis=2), np.concatenate([vs, vn], axis=2)
            (kb, kd), (vb, vd) = _blocks(fmtn, ks), _blocks(fmtn, vs)
            assert st.k.valid_contiguous().tobytes() == kb and st.v.valid_contiguous().tobytes() == vb, (where, s)
            want = orc.flash_sdpa(q, kd, vd, causal=True, threads=8)
            assert not np.isnan(out).any() and np.abs(out.astype(np.float32) - want.astype(np.float32)).max() <= 2e-2, (where, s)


@pytest.mark.parametrize("seed", range(4))
def test_ragged_steps_on_random_shapes(rt, seed):
    for it in range(5):
        rng = np.random.default_rng(7000 * seed + it)
        D = 128 if rng.random() < 0.8 else 64
        fmtn = str(rng.choice(["f16", "Q8_0", "Q4_0"])) if D == 128 else "f16"
        Hkv, g = int(rng.choice([1, 2, 8])), int(rng.choice([1, 2, 4, 5, 8, 16]))
        n_seq = int(rng.choice([1, 2, 5, 17]))
        lens = rng.integers(1, int(rng.choice([40, 300, 3000])), size=n_seq, endpoint=True)
        where = f"seed {seed} case {it}: {fmtn} D={D} Hq={Hkv * g} Hkv={Hkv} lens={lens.tolist()}"
        dev_fmt = None if fmtn == "f16" else getattr(tract_amd, fmtn)
        kcs, vcs, ks, vs = [], [], [], []
        for n in lens:
            k = rng.standard_normal((1, Hkv, int(n), D), dtype=np.float32).astype(np.float16)
            v = rng.standard_normal((1, Hkv, int(n), D), dtype=np.float32).astype(np.float16)
            kc, vc = tract_amd.InPlaceKvCache(2, dev_fmt), tract_amd.InPlaceKvCache(2, dev_fmt)
            kc.push(k), vc.push(v)
            kcs.append(kc), vcs.append(vc), ks.append(k), vs.append(v)
        ws = tract_amd.Workspace(n_seq, Hkv * g, 1, D)
        for s in range(int(rng.integers(1, 3))):
            q = (rng.standard_normal((n_seq, Hkv * g, 1, D), dtype=np.float32) / np.sqrt(D)).astype(np.float16)
            kn = rng.standard_normal((n_seq, Hkv, 1, D), dtype=np.float32).astype(np.float16)
            vn = rng.standard_normal((n_seq, Hkv, 1, D), dtype=np.float32).astype(np.float16)
            out = tract_amd.inplace_kv_sdpa_eval_ragged(tract_amd.DeviceTensor.from_numpy(q), tract_amd.DeviceTensor.from_numpy(kn),
                                                        tract_amd.DeviceTensor.from_numpy(vn), kcs, vcs, workspace=ws).to_numpy()
            for i in range(n_seq):
                ks[i], vs[i] = np.concatenate([ks[i], kn[i:i + 1]], axis=2), np.concatenate([vs[i], vn[i:i + 1]], axis=2)
                (kb, kd), (vb, vd) = _blocks(fmtn, ks[i]), _blocks(fmtn, vs[i])
                assert kcs[i].valid_contiguous().tobytes() == kb and vcs[i].valid_contiguous().tobytes() == vb, (where, s, i)
                want = orc.flash_sdpa(q[i:i + 1], kd, vd, causal=True, threads=8)
                assert np.abs(out[i:i + 1].astype(np.float32) - want.astype(np.float32)).max() <= 2e-2, (where, s, i)
