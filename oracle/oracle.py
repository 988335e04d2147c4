"""ctypes front end of the CPU oracle (``oracle/tract_oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` as the checker; never by the product package.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libtract_oracle.so")

FMT_Q8_0, FMT_Q4_0, FMT_Q8_1 = 2, 3, 4
BLOCK_BYTES = {FMT_Q8_0: 34, FMT_Q4_0: 18, FMT_Q8_1: 36}


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (a few hundred ms)."""
    srcs = [os.path.join(_HERE, f) for f in ("tract_oracle.c", "kivi_oracle.c")]
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < max(os.path.getmtime(s) for s in srcs):
        subprocess.check_call(["make", "-s", "-C", _HERE, "-B" if force else "-s"])
    return _SO


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = C.CDLL(_SO)
        sz, vp, i, f = C.c_size_t, C.c_void_p, C.c_int, C.c_float
        L.orc_f32_to_f16.restype = C.c_uint16
        L.orc_f32_to_f16.argtypes = [f]
        L.orc_f16_to_f32.restype = f
        L.orc_f16_to_f32.argtypes = [C.c_uint16]
        L.orc_f32_to_f16_n.argtypes = [vp, vp, sz]
        L.orc_f16_to_f32_n.argtypes = [vp, vp, sz]
        L.orc_win_new.restype = vp
        L.orc_win_new.argtypes = [sz, sz, sz]
        L.orc_win_free.argtypes = [vp]
        for n in ("len", "cursor", "capacity"):
            fn = getattr(L, "orc_win_" + n)
            fn.restype = sz
            fn.argtypes = [vp]
        L.orc_win_push.argtypes = [vp, vp, sz]
        L.orc_win_valid.argtypes = [vp, vp]
        L.orc_rotate_half.argtypes = [i, vp, vp, sz, sz]
        L.orc_apply_rope.argtypes = [i, vp, vp, vp, vp, i, vp, vp]
        L.orc_block_bytes.restype = sz
        L.orc_block_bytes.argtypes = [i]
        L.orc_quant.argtypes = [i, i, vp, sz, vp]
        L.orc_dequant.argtypes = [i, i, vp, sz, vp]
        L.orc_q4_0_matvec.argtypes = [vp, sz, sz, sz, vp, i, sz, sz, vp]
        L.orc_streamed_sdpa_f32.argtypes = [vp, vp, vp, vp, sz, sz, sz, sz, sz, sz, i, i, f, sz, vp]
        L.orc_kv_new.restype = vp
        L.orc_kv_new.argtypes = [sz, sz]
        L.orc_kv_free.argtypes = [vp]
        for n in ("len", "capacity", "reallocs"):
            fn = getattr(L, "orc_kv_" + n)
            fn.restype = sz
            fn.argtypes = [vp]
        L.orc_kv_buffer.restype = vp
        L.orc_kv_buffer.argtypes = [vp]
        L.orc_kv_push.argtypes = [vp, vp, sz]
        L.orc_kv_valid_contiguous.argtypes = [vp, vp]
        L.orc_concat_append.restype = vp
        L.orc_concat_append.argtypes = [vp, sz, vp, sz, sz, sz]
        L.orc_free.argtypes = [vp]
        L.orc_flash_sdpa_f32.argtypes = [vp, vp, vp, vp] + [sz] * 6 + [sz] * 3 + [sz, sz, i, i, f, vp, i]
        L.orc_flash_sdpa_eval_f16.argtypes = [vp, vp, vp, vp] + [sz] * 6 + [sz, sz, i, i, f, vp, i]
        L.orc_naive_sdpa_f64.argtypes = [vp, vp, vp, vp] + [sz] * 6 + [sz, sz, i, i, f, vp]
        L.orc_max_threads.restype = i
        L.orc_decode_step_f16.argtypes = [vp] * 5 + [sz] * 5 + [i, vp, C.POINTER(vp), C.POINTER(vp)]
        L.orc_kivi_quant_dequant.argtypes = [vp, sz, sz, C.c_uint, i, vp]
        L.orc_kivi_new.restype = vp
        L.orc_kivi_new.argtypes = [i, sz, C.c_uint, sz]
        L.orc_kivi_clone.restype = vp
        L.orc_kivi_clone.argtypes = [vp]
        L.orc_kivi_free.argtypes = [vp]
        L.orc_kivi_push.argtypes = [vp, vp]
        for n in ("len", "n_sink", "n_rows", "n_res", "n_params", "row_bytes", "memory_bytes"):
            fn = getattr(L, "orc_kivi_" + n)
            fn.restype = sz
            fn.argtypes = [vp]
        L.orc_kivi_state.argtypes = [vp] * 6
        L.orc_kivi_dequant_all.argtypes = [vp, vp]
        _lib = L
    return _lib


def _p(a: np.ndarray | None):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


# ----------------------------------------------------------------------------- f16
def f32_to_f16_bits(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().orc_f32_to_f16_n(_p(x), _p(out), x.size)
    return out


def f16_bits_to_f32(h: np.ndarray) -> np.ndarray:
    h = np.ascontiguousarray(h, dtype=np.uint16)
    out = np.empty(h.shape, dtype=np.float32)
    lib().orc_f16_to_f32_n(_p(h), _p(out), h.size)
    return out


# ----------------------------------------------------------------------------- block quant
def quant(fmt: int, x: np.ndarray) -> np.ndarray:
    """BlockQuant::quant_f32 / quant_f16: blocks of 32 along the last axis.

    Returns uint8 array of shape x.shape[:-1] + (D/32 * block_bytes,)."""
    assert x.dtype in (np.float32, np.float16) and x.shape[-1] % 32 == 0
    x = np.ascontiguousarray(x)
    bb = BLOCK_BYTES[fmt]
    out = np.empty(x.shape[:-1] + (x.shape[-1] // 32 * bb,), dtype=np.uint8)
    rc = lib().orc_quant(fmt, int(x.dtype == np.float16), _p(x), x.size, _p(out))
    assert rc == 0
    return out


def dequant(fmt: int, q: np.ndarray, dtype=np.float32) -> np.ndarray:
    """BlockQuant::dequant_f32 / dequant_f16 of a canonical block byte array."""
    q = np.ascontiguousarray(q, dtype=np.uint8)
    bb = BLOCK_BYTES[fmt]
    assert q.shape[-1] % bb == 0
    d = q.shape[-1] // bb * 32
    out = np.empty(q.shape[:-1] + (d,), dtype=dtype)
    rc = lib().orc_dequant(fmt, int(dtype == np.float16), _p(q), out.size, _p(out))
    assert rc == 0
    return out


def simulate_precision_loss(fmt: int, x: np.ndarray) -> np.ndarray:
    """BlockQuant::simulate_precision_loss (block_quant/mod.rs:130-154): every block of 32 along the last axis is
    quantised and dequantised in the tensor's own type."""
    return dequant(fmt, quant(fmt, x), dtype=x.dtype).reshape(x.shape)


def q4_0_matvec(blocks: np.ndarray, act: np.ndarray) -> np.ndarray:
    """GgmlGemm's Q4_0 matrix-vector arm as its test defines it (cuda/src/kernels/matmul/mod.rs:864-890):
    blocks uint8 [w_batch, n, k/32*18], act [act_batch, m, k] f32 or f16 -> [act_batch, m, n]."""
    blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
    act = np.ascontiguousarray(act)
    wb, n, rb = blocks.shape
    ab, m, k = act.shape
    assert rb == k // 32 * 18 and act.dtype in (np.float32, np.float16)
    out = np.empty((ab, m, n), dtype=act.dtype)
    rc = lib().orc_q4_0_matvec(_p(blocks), wb, n, k, _p(act), int(act.dtype == np.float16), ab, m, _p(out))
    assert rc == 0
    return out


# ----------------------------------------------------------------------------- kv cache
class InPlaceKvCache:
    """InPlaceKvCache (inplace_kv_cache.rs:28-114) over numpy arrays; `axis` is the
    sequence axis of the pushed tensors."""

    def __init__(self, axis: int):
        self.axis = axis
        self._h = None
        self._shape = None
        self._dtype = None

    def push(self, x: np.ndarray) -> None:
        x = np.ascontiguousarray(x)
        if self._h is None:
            outer = int(np.prod(x.shape[: self.axis], dtype=np.int64))
            inner = int(np.prod(x.shape[self.axis + 1:], dtype=np.int64)) * x.dtype.itemsize
            self._h = lib().orc_kv_new(outer, inner)
            self._shape, self._dtype = list(x.shape), x.dtype
        assert x.dtype == self._dtype
        assert lib().orc_kv_push(self._h, _p(x), x.shape[self.axis]) == 0

    def len(self) -> int:
        return 0 if self._h is None else lib().orc_kv_len(self._h)

    def capacity(self) -> int:
        return 0 if self._h is None else lib().orc_kv_capacity(self._h)

    def reallocs(self) -> int:
        return 0 if self._h is None else lib().orc_kv_reallocs(self._h)

    def valid_contiguous(self) -> np.ndarray:
        shape = list(self._shape)
        shape[self.axis] = self.len()
        out = np.empty(shape, dtype=self._dtype)
        lib().orc_kv_valid_contiguous(self._h, _p(out))
        return out

    def __del__(self):
        if self._h is not None and _lib is not None:
            _lib.orc_kv_free(self._h)
            self._h = None


def concat_append(past: np.ndarray | None, new: np.ndarray, axis: int) -> np.ndarray:
    """DynKeyValueCacheState::eval (dyn_kv_cache.rs:158-174): fresh concat."""
    new = np.ascontiguousarray(new)
    if past is None:
        return new.copy()
    past = np.ascontiguousarray(past)
    outer = int(np.prod(new.shape[:axis], dtype=np.int64))
    inner = int(np.prod(new.shape[axis + 1:], dtype=np.int64)) * new.dtype.itemsize
    ptr = lib().orc_concat_append(_p(past), past.shape[axis], _p(new), new.shape[axis], outer, inner)
    shape = list(new.shape)
    shape[axis] = past.shape[axis] + new.shape[axis]
    n = int(np.prod(shape, dtype=np.int64)) * new.dtype.itemsize
    out = np.frombuffer(C.string_at(ptr, n), dtype=new.dtype).reshape(shape).copy()
    lib().orc_free(ptr)
    return out


# ----------------------------------------------------------------------------- attention
def _as4(q, k, v, mask):
    r3 = q.ndim == 3
    if r3:
        q, k, v = q[:, None], k[:, None], v[:, None]
        if mask is not None:
            mask = mask[:, None]
    return q, k, v, mask, r3


def flash_sdpa(q, k, v, mask=None, causal=False, scale=None, threads=1):
    """FlashSdpaOp::eval (flash_sdpa.rs:103-163).  f32 or f16 inputs (rank 3 or 4);
    output has Q's shape and dtype."""
    q, k, v, mask, r3 = _as4(q, k, v, mask)
    B, Hq, Sq, D = q.shape
    _, Hkv, Sk, _ = k.shape
    mb, mh = (mask.shape[0], mask.shape[1]) if mask is not None else (1, 1)
    if mask is not None:
        mask = np.ascontiguousarray(np.broadcast_to(mask, (mb, mh, Sq, Sk)))
    hs, sc = (0, 0.0) if scale is None else (1, float(scale))
    if q.dtype == np.float16:
        qq, kk, vv = (np.ascontiguousarray(a, dtype=np.float16) for a in (q, k, v))
        mm = None if mask is None else np.ascontiguousarray(mask, dtype=np.float16)
        out = np.empty(q.shape, dtype=np.float16)
        lib().orc_flash_sdpa_eval_f16(_p(qq), _p(kk), _p(vv), _p(mm), B, Hq, Hkv, Sq, Sk, D, mb, mh,
                                      int(causal), hs, sc, _p(out), threads)
    else:
        qq, kk, vv = (np.ascontiguousarray(a, dtype=np.float32) for a in (q, k, v))
        mm = None if mask is None else np.ascontiguousarray(mask, dtype=np.float32)
        out = np.empty(q.shape, dtype=np.float32)
        lib().orc_flash_sdpa_f32(_p(qq), _p(kk), _p(vv), _p(mm), B, Hq, Hkv, Sq, Sk, D,
                                 Hkv * Sk * D, Sk * D, D, mb, mh, int(causal), hs, sc, _p(out), threads)
    return out[:, 0] if r3 else out


def streamed_sdpa(q, k, v, mask=None, causal=False, scale=None, block_k=64):
    """StreamedSdpaOp::eval (streamed_sdpa.rs:95-160): f32 or f16 inputs of rank 3 or 4, optional rank-2 mask
    [q_len, kv_len]; computed in f32, returned in Q's type and shape."""
    dt = q.dtype
    r3 = q.ndim == 3
    q4, k4, v4 = ((a[:, None] if r3 else a) for a in (q, k, v))
    qq, kk, vv = (np.ascontiguousarray(a, dtype=np.float32) for a in (q4, k4, v4))
    B, Hq, Sq, D = qq.shape
    _, Hkv, Sk, _ = kk.shape
    mm = None
    if mask is not None:
        assert mask.shape == (Sq, Sk)
        mm = np.ascontiguousarray(mask, dtype=np.float32)
    out = np.empty(qq.shape, dtype=np.float32)
    hs, sc = (0, 0.0) if scale is None else (1, float(scale))
    rc = lib().orc_streamed_sdpa_f32(_p(qq), _p(kk), _p(vv), _p(mm), B, Hq, Hkv, Sq, Sk, D, int(causal), hs, sc,
                                     int(block_k), _p(out))
    assert rc == 0
    out = out.astype(dt)
    return out[:, 0] if r3 else out


def flash_sdpa_view(q, kbuf, vbuf, length, causal=False, scale=None, threads=1):
    """flash_attention_gqa over zero-copy [0..length] views of capacity buffers
    [B,Hkv,cap,D] f32 — what InPlaceKvSdpaState::eval does (inplace_kv_cache.rs:191-216)."""
    B, Hq, Sq, D = q.shape
    _, Hkv, cap, _ = kbuf.shape
    assert kbuf.dtype == np.float32 and kbuf.flags.c_contiguous and vbuf.flags.c_contiguous
    qq = np.ascontiguousarray(q, dtype=np.float32)
    out = np.empty(q.shape, dtype=np.float32)
    hs, sc = (0, 0.0) if scale is None else (1, float(scale))
    lib().orc_flash_sdpa_f32(_p(qq), _p(kbuf), _p(vbuf), None, B, Hq, Hkv, Sq, length, D,
                             Hkv * cap * D, cap * D, D, 1, 1, int(causal), hs, sc, _p(out), threads)
    return out


def naive_sdpa_f64(q, k, v, mask=None, causal=False, scale=None):
    """Textbook softmax(QK^T*scale+mask)V in f64 over the f32 images of the inputs."""
    q, k, v, mask, r3 = _as4(q, k, v, mask)
    B, Hq, Sq, D = q.shape
    _, Hkv, Sk, _ = k.shape
    mb, mh = (mask.shape[0], mask.shape[1]) if mask is not None else (1, 1)
    qq, kk, vv = (np.ascontiguousarray(a, dtype=np.float32) for a in (q, k, v))
    mm = None
    if mask is not None:
        mm = np.ascontiguousarray(np.broadcast_to(mask, (mb, mh, Sq, Sk)), dtype=np.float32)
    out = np.empty(q.shape, dtype=np.float64)
    hs, sc = (0, 0.0) if scale is None else (1, float(scale))
    lib().orc_naive_sdpa_f64(_p(qq), _p(kk), _p(vv), _p(mm), B, Hq, Hkv, Sq, Sk, D, mb, mh,
                             int(causal), hs, sc, _p(out))
    return out[:, 0] if r3 else out


def decode_step_f16(q, k_past, v_past, k_new, v_new, threads=1):
    """One decode step of the reference's default CPU path with its costs (concat
    reallocation of K and V, whole-tensor f32 casts).  Returns (out, K, V)."""
    B, Hq, _, D = q.shape
    _, Hkv, T, _ = k_past.shape
    out = np.empty(q.shape, dtype=np.float16)
    kp, vp = C.c_void_p(), C.c_void_p()
    lib().orc_decode_step_f16(_p(q), _p(k_past), _p(v_past), _p(k_new), _p(v_new), B, Hq, Hkv, T, D,
                              threads, _p(out), C.byref(kp), C.byref(vp))
    n = B * Hkv * (T + 1) * D
    k = np.ctypeslib.as_array(C.cast(kp, C.POINTER(C.c_uint16)), shape=(n,)).view(np.float16).reshape(B, Hkv, T + 1, D).copy()
    v = np.ctypeslib.as_array(C.cast(vp, C.POINTER(C.c_uint16)), shape=(n,)).view(np.float16).reshape(B, Hkv, T + 1, D).copy()
    lib().orc_free(kp)
    lib().orc_free(vp)
    return out, k, v


def max_threads() -> int:
    return lib().orc_max_threads()


def rotate_half(x: np.ndarray) -> np.ndarray:
    """RotateHalf (apply_rope.rs:58-76) on a dense f32/f16 array."""
    x = np.ascontiguousarray(x)
    out = np.empty_like(x)
    inner = x.shape[-1]
    lib().orc_rotate_half(int(x.dtype == np.float16), _p(x), _p(out), x.size // max(inner, 1), inner)
    return out


def apply_rope(x: np.ndarray, cos: np.ndarray, sin: np.ndarray) -> np.ndarray:
    """ApplyRope (apply_rope.rs:169-176): x*cos + rotate_half(x)*sin in x's datum type; cos and
    sin (same shape) broadcast against x numpy-style."""
    x = np.ascontiguousarray(x)
    assert cos.shape == sin.shape and cos.dtype == sin.dtype == x.dtype and 2 <= x.ndim <= 4
    cos, sin = np.ascontiguousarray(cos), np.ascontiguousarray(sin)
    pad = (1,) * (x.ndim - cos.ndim) + cos.shape
    strides, acc = [], 1
    for d in range(x.ndim - 1, -1, -1):
        assert pad[d] in (1, x.shape[d])
        strides.append(0 if pad[d] == 1 and x.shape[d] != 1 else acc)
        acc *= pad[d]
    strides = strides[::-1]
    out = np.empty_like(x)
    shp = (C.c_size_t * x.ndim)(*x.shape)
    cs = (C.c_size_t * x.ndim)(*strides)
    lib().orc_apply_rope(int(x.dtype == np.float16), _p(x), _p(cos), _p(sin), _p(out), x.ndim, shp, cs)
    return out


class WindowKvCache:
    """WindowKvCache (window_kv_cache.rs:80-154) over [B, H, S, D] arrays, token axis 2."""

    def __init__(self, window: int):
        assert window > 0
        self.window, self._h, self._like = window, None, None

    def push(self, x: np.ndarray) -> None:
        x = np.ascontiguousarray(x)
        if x.shape[2] == 0:
            return
        if self._h is None:
            self._like = (x.shape, x.dtype)
            self._h = lib().orc_win_new(x.shape[0] * x.shape[1], self.window, x.shape[3] * x.dtype.itemsize)
        lib().orc_win_push(self._h, _p(x), x.shape[2])

    def len(self) -> int:
        return 0 if self._h is None else lib().orc_win_len(self._h)

    def cursor(self) -> int:
        return 0 if self._h is None else lib().orc_win_cursor(self._h)

    def capacity(self) -> int:
        return 0 if self._h is None else lib().orc_win_capacity(self._h)

    def valid_view(self) -> np.ndarray:
        shape, dt = self._like
        out = np.empty((shape[0], shape[1], self.len(), shape[3]), dt)
        lib().orc_win_valid(self._h, _p(out))
        return out

    def __del__(self):
        if self._h is not None and _lib is not None:
            _lib.orc_win_free(self._h)
            self._h = None


# ---- NNEF tensor files (nnef/src/tensors.rs), restated with `struct` -------------------------------
_DAT_VENDOR_TRACT = (ord("T") << 8) | ord("R")   # tensors.rs:8


def dat_header_fields(data: bytes) -> dict:
    """The 128-byte header (tensors.rs:10-25), little endian, field by field."""
    import struct
    magic0, magic1, vmaj, vmin, size, rank = struct.unpack_from("<BBBBII", data, 0)
    dims = struct.unpack_from("<8I", data, 12)
    bits, item, vendor = struct.unpack_from("<IHH", data, 44)
    return {"magic": (magic0, magic1), "version": (vmaj, vmin), "data_size_bytes": size, "rank": rank,
            "dims": dims[:rank], "bits_per_item": bits, "item_type": item, "item_type_vendor": vendor,
            "rest_is_zero": not any(data[52:128])}


def dat_write_plain(a: np.ndarray) -> bytes:
    """write_tensor for f32 / f16 (tensors.rs:186-248): vendor 0, item type 0."""
    import struct
    a = np.require(a, requirements="C")
    dims = list(a.shape) + [0] * (8 - a.ndim)
    head = struct.pack("<BBBBII8IIHH", 0x4E, 0xEF, 1, 0, a.nbytes, a.ndim, *dims, a.dtype.itemsize * 8, 0, 0)
    return head + b"\0" * (128 - len(head)) + a.tobytes()


def dat_write_block_quant(item_type: int, blocks: bytes, shape) -> bytes:
    """write_block_quant_value (tensors.rs:300-322): shape flattened to [prod(leading), last]."""
    import struct
    m = int(np.prod(shape[:-1], dtype=np.int64))
    dims = [m, shape[-1]] + [0] * 6
    head = struct.pack("<BBBBII8IIHH", 0x4E, 0xEF, 1, 0, len(blocks), 2, *dims, 0xFFFFFFFF, item_type, _DAT_VENDOR_TRACT)
    return head + b"\0" * (128 - len(head)) + bytes(blocks)


def q4_0_legacy_to_gguf(blocks: np.ndarray) -> np.ndarray:
    """tract_to_gguf_q4_0_packing (tensors.rs:250-273), statement by statement."""
    out = np.array(blocks, dtype=np.uint8).reshape(-1, 18).copy()
    for b in range(out.shape[0]):
        nibbles = out[b, 2:18]            # a view: written in place, from the top down, like the reference
        second = nibbles[8:].copy()
        for i in range(15, -1, -1):
            lsb = (nibbles[i // 2] & 0x0F) if i % 2 == 0 else ((nibbles[i // 2] & 0xF0) >> 4)
            msb = ((second[i // 2] & 0x0F) << 4) if i % 2 == 0 else (second[i // 2] & 0xF0)
            nibbles[i] = msb | lsb
    return out.reshape(blocks.shape)


# ---- KIVI-style affine KV quantisation (kv_quant.rs, quant_dyn_kv_cache.rs) --------------------------
KIVI_PER_TOKEN, KIVI_BLOCK_CHANNEL, KIVI_RUNNING_CHANNEL = 0, 1, 2
KIVI_SINK_TOKENS, KIVI_KEY_BLOCK = 4, 32   # quant_dyn_kv_cache.rs:92, :153


def kivi_quant_dequant(x: np.ndarray, bits: int, by_row: bool) -> np.ndarray:
    """quant_dequant (kv_quant.rs:73-98) of a [rows, cols] f32 matrix."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty_like(x)
    lib().orc_kivi_quant_dequant(_p(x), x.shape[0], x.shape[1], bits, int(by_row), _p(out))
    return out


class KiviStore:
    """One head's store: PerTokenStore / BlockChannelStore (quant_dyn_kv_cache.rs:97-250, sink_tokens=4) or
    QuantValueCache / QuantKeyCache (kv_quant.rs:121-236: KIVI_PER_TOKEN / KIVI_RUNNING_CHANNEL, 8 bits, no sinks)."""

    def __init__(self, layout: int, d: int, bits: int = 8, sink_tokens: int = KIVI_SINK_TOKENS, _h=None):
        self.layout, self.d, self.bits, self.sink_tokens = layout, d, bits, sink_tokens
        self._h = _h if _h is not None else lib().orc_kivi_new(layout, d, bits, sink_tokens)

    def push_token(self, row: np.ndarray) -> None:
        row = np.ascontiguousarray(row, dtype=np.float32)
        assert row.shape == (self.d,)
        lib().orc_kivi_push(self._h, _p(row))

    def clone(self) -> "KiviStore":
        return KiviStore(self.layout, self.d, self.bits, self.sink_tokens, _h=lib().orc_kivi_clone(self._h))

    def len(self) -> int:
        return lib().orc_kivi_len(self._h)

    def memory_bytes(self) -> int:
        return lib().orc_kivi_memory_bytes(self._h)

    def dequant_all(self) -> np.ndarray:
        out = np.empty((self.len(), self.d), np.float32)
        lib().orc_kivi_dequant_all(self._h, _p(out))
        return out

    def state(self) -> dict:
        """Raw state: sink [n_sink, d] f32, packed [n_rows, row_bytes] u8, lo / scale f32, residual [n_res, d] f32."""
        L = lib()
        ns, nr, nres, npar, rb = (getattr(L, "orc_kivi_" + n)(self._h) for n in ("n_sink", "n_rows", "n_res", "n_params", "row_bytes"))
        st = {"sink": np.empty((ns, self.d), np.float32), "packed": np.empty((nr, rb), np.uint8),
              "lo": np.empty(npar, np.float32), "scale": np.empty(npar, np.float32),
              "residual": np.empty((nres, self.d), np.float32)}
        L.orc_kivi_state(self._h, _p(st["sink"]), _p(st["packed"]), _p(st["lo"]), _p(st["scale"]), _p(st["residual"]))
        return st

    def __del__(self):
        if self._h is not None and _lib is not None:
            _lib.orc_kivi_free(self._h)
            self._h = None


class KiviCache:
    """QuantizedDynKvCacheState (quant_dyn_kv_cache.rs:334-449): one store per (batch, head) of a
    [B, H, S, D] tensor, Keys block x channel (per_channel) or Values per token; `running` selects the
    stores of QuantizedKvSdpaState (kv_quant.rs:270-330: no sink tokens, 8 bits, Keys with running scales)."""

    def __init__(self, per_channel: bool, bits: int = 8, running: bool = False):
        self.per_channel, self.bits, self.running = per_channel, bits, running
        self.stores: list[KiviStore] = []
        self.lead = None
        self.length = 0

    def ingest(self, x: np.ndarray) -> None:
        x = np.ascontiguousarray(x).astype(np.float32)
        b, h, s, d = x.shape
        if not self.stores:
            self.lead = (b, h)
            layout = (KIVI_RUNNING_CHANNEL if self.running else KIVI_BLOCK_CHANNEL) if self.per_channel else KIVI_PER_TOKEN
            self.stores = [KiviStore(layout, d, 8 if self.running else self.bits, 0 if self.running else KIVI_SINK_TOKENS)
                           for _ in range(b * h)]
        assert self.lead == (b, h), "cache shape changed between steps"
        for bi in range(b):
            for hi in range(h):
                for t in range(s):
                    self.stores[bi * h + hi].push_token(x[bi, hi, t])
        self.length += s

    def dequantized(self) -> np.ndarray:
        b, h = self.lead
        return np.stack([st.dequant_all() for st in self.stores]).reshape(b, h, self.length, -1)

    def state(self) -> dict:
        sts = [st.state() for st in self.stores]
        return {k: np.stack([s[k] for s in sts]) for k in sts[0]}
