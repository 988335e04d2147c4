"""Shared inputs for the parity tests.

`SDPA_LITERAL_CASES` restates, as data, the hand-written problems of the reference's
cross-backend suite (test-rt/suite-unit/src/sdpa.rs:346-548): name -> (q, k, v, mask,
scale, is_causal).  Rank-3 tensors are single-head `[B,S,D]`.
"""
import numpy as np


def _z(*shape, dt=np.float32):
    return np.zeros(shape, dtype=dt)


def _a(x, dt=np.float32):
    return np.array(x, dtype=dt)


def sdpa_literal_cases():
    c = {}
    c["trivial_f32_0"] = (_a([[[0]]]), _a([[[0]]]), _a([[[0]]]), None, None, True)
    c["causal_f32_0"] = (_a([[[0]]]), _a([[[0]]]), _a([[[0]]]), None, None, True)
    c["causal_f32_1"] = (_a([[[0], [0]]]), _a([[[0], [0]]]), _a([[[0], [0]]]), None, None, True)
    c["causal_f32_2"] = c["causal_f32_1"]
    c["causal_with_s_and_p_0"] = (_a([[[0], [0]]]), _a([[[0], [0], [0]]]), _a([[[0], [0], [1]]]), None, None, True)
    c["gqa_f32_0"] = (_z(1, 2, 1, 1), _z(1, 2, 1, 1), _a([[[[0]], [[1]]]]), None, None, False)
    c["gqa_f32_1"] = (_z(1, 2, 1, 1), _z(1, 1, 1, 1), _z(1, 1, 1, 1), None, None, False)
    c["gqa_f32_big_0"] = (_z(2, 8, 5, 64), _z(2, 4, 5, 64), _z(2, 4, 5, 64), None, None, True)
    c["gqa_f32_big_1"] = (_z(2, 8, 5, 64), _z(2, 1, 5, 64), _z(2, 1, 5, 64), None, None, True)
    c["gqa_f32_big_2"] = (_z(2, 2, 3, 64), _z(2, 1, 3, 64), _z(2, 1, 3, 64), None, None, True)
    c["mask_0"] = (_z(1, 2, 1), _z(1, 2, 1), _a([[[2], [0]]]), _a([[[0, 0], [0, -1]]]), None, False)
    c["gqa_f32_mask_simple"] = (_z(1, 1, 1), _z(1, 1, 1), _z(1, 1, 1), _a([[[0]]]), None, False)
    c["gqa_f32_mask_0"] = (_z(2, 2, 3, 64), _z(2, 1, 3, 64), _z(2, 1, 3, 64), _z(1, 1, 3, 3), None, False)
    c["gqa_f16_0"] = (_z(1, 2, 64, dt=np.float16), _z(1, 3, 64, dt=np.float16), _z(1, 3, 64, dt=np.float16), None, None, True)
    c["gqa_f32_nocausal_nomask"] = (_z(1, 1, 2, 1), _z(1, 1, 2, 1), _a([[[[0], [1]]]]), None, None, False)
    c["f32_nocausal_nomask"] = (_a([[[0], [1]]]), _a([[[0], [1]]]), _a([[[1], [0]]]), None, None, False)
    c["gqa_mh_mask"] = (_z(1, 2, 2, 1), _z(1, 1, 2, 1), _a([[[[0], [0.01]]]]),
                        _a([[[[0, 0], [0, 0]], [[0, 0], [-2, 0]]]]), None, False)
    v = _z(2, 2, 64)
    v[1, 1, 63] = -0.25
    m = _a([[[0.0, 0.25], [0.0, 0.0]], [[0.375, -0.25], [0.0, 0.0]]])
    c["f32_mask_with_batch_cuda"] = (_z(2, 2, 64), _z(2, 2, 64), v, m, None, False)
    c["f16_mask_with_batch_cuda"] = (_z(2, 2, 64, dt=np.float16), _z(2, 2, 64, dt=np.float16),
                                     v.astype(np.float16), m.astype(np.float16), None, False)
    return c


def textbook_sdpa(q, k, v, mask=None, scale=None, causal=False):
    """numpy float64 softmax(QK^T*scale + mask)V, written independently of the C
    oracle (vectorised, not a transcription of it): used to pin the oracle."""
    r3 = q.ndim == 3
    if r3:
        q, k, v = q[:, None], k[:, None], v[:, None]
        mask = None if mask is None else mask[:, None]
    q, k, v = (a.astype(np.float64) for a in (q, k, v))
    B, Hq, Sq, D = q.shape
    Hkv, Sk = k.shape[1], k.shape[2]
    g = Hq // Hkv
    k = np.repeat(k, g, axis=1)
    v = np.repeat(v, g, axis=1)
    s = np.einsum("bhqd,bhkd->bhqk", q, k) * (scale if scale is not None else 1.0 / np.sqrt(D))
    if causal:
        i = np.arange(Sq)[:, None]
        j = np.arange(Sk)[None, :]
        s = np.where(j > i + max(Sk - Sq, 0), -np.inf, s)
    if mask is not None:
        s = s + mask.astype(np.float64)
    s = s - s.max(axis=-1, keepdims=True)
    p = np.exp(s)
    p /= p.sum(axis=-1, keepdims=True)
    o = np.einsum("bhqk,bhkd->bhqd", p, v)
    return o[:, 0] if r3 else o


def seeded_normal(seed, shape, dtype=np.float32):
    """The synthetic-input generator of every config: PCG64(seed) standard normal
    f32, cast (RNE) to the config's dtype."""
    g = np.random.Generator(np.random.PCG64(seed))
    return g.standard_normal(shape, dtype=np.float32).astype(dtype)


def cfg_seed(cfg, what):
    return 20260000 + 100 * cfg + {"q": 0, "k": 1, "v": 2, "len": 3, "chan": 4}[what]
