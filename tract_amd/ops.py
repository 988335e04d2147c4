"""Host-side mirror of tract's KV-cache operators over the rocm C ABI.

Names, arguments and error behaviour follow the reference operators so that the
parity tests read like tract's own unit tests:

* ``InPlaceKvCache``      transformers/src/ops/inplace_kv_cache.rs:28-114
* ``InPlaceKvSdpa``/State transformers/src/ops/inplace_kv_cache.rs:131-290
* ``DynKeyValueCache``/State transformers/src/ops/dyn_kv_cache.rs:90-183 (device twin:
  gpu/src/ops/dyn_kv_cache.rs:8-125), here backed by the in-place cache
* ``Sdpa``                transformers/src/ops/sdpa.rs:83-89, 296-356
* ``BlockQuant``          linalg/src/frame/block_quant/mod.rs:36-108 (Q4_0; Q8_0 = Q8_1 without sum)
* ``WindowKvCache``, ``WindowKvSdpa``/State transformers/src/ops/window_kv_cache.rs:80-154, 156-239
* ``ApplyRope``/``RotateHalf`` transformers/src/ops/apply_rope.rs:44-86, 150-188 (device twin:
  cuda/src/kernels/nn/apply_rope.rs:41-129)
* ``Cast``                cuda/src/kernels/array/cast.rs:17-90 (f32 <-> f16 only)
"""
from __future__ import annotations

import ctypes as C
import math

import numpy as np

from . import _lib
from ._lib import F16, F32, Q4_0, Q8_0, TractRocmError, call
from .runtime import DeviceTensor, Workspace, _sh, dtype_code, synchronize

_I64x4 = C.c_int64 * 4
_I64x3 = C.c_int64 * 3


def _as_device(x, stream=None) -> DeviceTensor:
    return x if isinstance(x, DeviceTensor) else DeviceTensor.from_numpy(np.asarray(x), stream)


def _canon4(shape):
    """[B,H,S,D] view of a rank-3 ([B,S,D]) or rank-4 shape."""
    if len(shape) == 4:
        return tuple(shape)
    if len(shape) == 3:
        return (shape[0], 1, shape[1], shape[2])
    raise TractRocmError(f"Inputs must be of rank 3 or 4, found {len(shape)}")


class KvPool:
    """One device allocation shared by many caches (per-sequence capacity-doubling caches of a
    ragged batch)."""

    def __init__(self, nbytes: int):
        h = C.c_void_p()
        call("trocm_kv_pool_create", C.byref(h), nbytes)
        self.handle = h

    def stats(self) -> dict:
        total, used, largest, base = C.c_size_t(), C.c_size_t(), C.c_size_t(), C.c_void_p()
        call("trocm_kv_pool_stats", self.handle, C.byref(total), C.byref(used), C.byref(largest), C.byref(base))
        return {"bytes_total": total.value, "bytes_in_use": used.value, "largest_free": largest.value,
                "base": base.value}

    def close(self) -> None:
        if self.handle:
            call("trocm_kv_pool_destroy", self.handle)
            self.handle = None


class InPlaceKvCache:
    """Geometric-growth in-place cache along `axis` (the token axis, rank-2)."""

    def __init__(self, axis: int, storage_format: int | None = None, pool: KvPool | None = None):
        self.axis = axis
        self.pool = pool
        self.storage_format = storage_format  # None: same as the first pushed tensor
        self._h = None
        self._shape = None
        self._dtype = None

    # -- lifetime
    def _create(self, shape, dtype):
        if self.axis != len(shape) - 2:
            raise TractRocmError(f"kv-cache axis {self.axis} unsupported: the token axis must be rank-2")
        B, H, _, D = _canon4(shape)
        fmt = dtype_code(dtype) if self.storage_format is None else self.storage_format
        h = C.c_void_p()
        if self.pool is not None:
            call("trocm_kv_cache_create_in_pool", C.byref(h), self.pool.handle, fmt, B, H, D)
        else:
            call("trocm_kv_cache_create", C.byref(h), fmt, B, H, D)
        self._h, self._shape, self._dtype, self.storage_format = h, tuple(shape), np.dtype(dtype), fmt

    def __del__(self):
        try:
            if self._h:
                _lib.load().trocm_kv_cache_destroy(self._h)
                self._h = None
        except Exception:
            pass

    # -- InPlaceKvCache API
    def _get(self, what) -> int:
        if self._h is None:
            return 0
        v = C.c_int64()
        call("trocm_kv_cache_" + what, self._h, C.byref(v))
        return v.value

    def len(self) -> int:
        return self._get("len")

    def is_empty(self) -> bool:
        return self.len() == 0

    def capacity(self) -> int:
        return self._get("capacity")

    def reallocs(self) -> int:
        return self._get("reallocs")

    def reserve(self, capacity: int, like=None, stream=None) -> None:
        if self._h is None:
            if like is None:
                raise TractRocmError("reserve on a cache that has seen no tensor needs `like=(shape, dtype)`")
            self._create(*like)
        call("trocm_kv_cache_reserve", self._h, capacity, _sh(stream))

    def push(self, x, strides=None, stream=None) -> None:
        """Append `x` ([.., S, D] device tensor or numpy array) along the token axis.
        `strides`: element strides of a non-dense source view (shape stays x.shape)."""
        t = _as_device(x, stream)
        if self._h is None:
            if t.shape[self.axis if self.axis >= 0 else 0] == 0:
                return
            self._create(t.shape, t.dtype)
        self._check_push_shape(t.shape)
        B, H, S, D = _canon4(t.shape)
        st = strides if strides is not None else t.strides()
        if len(st) == 3:
            st = (st[0], 0, st[1], st[2])
        call("trocm_kv_append", self._h, t.ptr, dtype_code(t.dtype), _I64x4(*st), S, _sh(stream))

    def _check_push_shape(self, shape) -> None:
        if len(shape) != len(self._shape):
            raise TractRocmError("rank mismatch in kv-cache push")
        want, got = list(self._shape), list(shape)
        want[self.axis] = got[self.axis] = 0
        if want != got:
            raise TractRocmError(f"kv-cache push: shape {tuple(shape)} does not match the cache's {self._shape} off-axis")

    def truncate(self, length: int) -> None:
        if self._h is None:
            raise TractRocmError("Can not truncate a zero-len kv-cache value")
        call("trocm_kv_cache_truncate", self._h, length)

    def row_bytes(self) -> int:
        n = C.c_size_t()
        call("trocm_kv_row_bytes", self._h, C.byref(n))
        return n.value

    def valid_contiguous(self, stream=None) -> np.ndarray:
        """Dense host copy of the valid [0..len] region: the tensor for F32/F16 storage, the
        canonical block bytes `[.., len, D/32*block_bytes]` (uint8) for Q8_0/Q4_0."""
        if self._h is None:
            raise TractRocmError("empty kv-cache")
        n = self.len()
        shape = list(self._shape)
        shape[self.axis] = n
        if self.storage_format in (F32, F16):
            out = DeviceTensor(shape, np.float32 if self.storage_format == F32 else np.float16)
        else:
            shape[-1] = self.row_bytes()
            out = DeviceTensor(shape, np.uint8)
        call("trocm_kv_export", self._h, out.ptr, _sh(stream))
        return out.to_numpy(stream)

    def save_dat(self, stream=None) -> bytes:
        """The valid region as an NNEF tensor file: a rank-4 f32/f16 tensor, or the canonical blocks
        of a quantised cache (no dequantisation) under the flattened shape [B*H*len, D]."""
        from . import dat
        v = self.valid_contiguous(stream)
        if self.storage_format in (F32, F16):
            return dat.write_tensor(v)
        B, H, _, D = _canon4(self._shape)
        return dat.write_block_quant(self.storage_format, v, (B * H * self.len(), D))

    def load_dat(self, data: bytes, like=None, stream=None) -> None:
        """Append the tokens of an NNEF tensor file written by `save_dat`.  A quantised file records
        only [rows, D]: `like=(shape, dtype)` gives batch and heads when the cache is still empty."""
        from . import dat
        item, shape, payload = dat.read_tensor(data)
        if item in (F32, F16):
            self.push(payload, stream=stream)
            return
        if self._h is None:
            if like is None:
                raise TractRocmError("load_dat of block-quantised data into an empty cache needs `like=(shape, dtype)`")
            if self.storage_format is None:
                self.storage_format = item
            self._create(*like)
        if self.storage_format != item:
            raise TractRocmError("the file's block format differs from the cache's storage format")
        B, H, _, D = _canon4(self._shape)
        if shape[-1] != D or shape[0] % (B * H):
            raise TractRocmError(f"file shape {shape} does not match a cache of {B} x {H} heads of {D}")
        n = shape[0] // (B * H)
        dev = DeviceTensor.from_numpy(payload, stream)
        call("trocm_kv_import_blocks", self._h, dev.ptr, n, _sh(stream))
        call("trocm_stream_sync", _sh(stream))

    def clone(self, stream=None) -> "InPlaceKvCache":
        c = InPlaceKvCache(self.axis, self.storage_format, self.pool)
        if self._h is not None:
            h = C.c_void_p()
            call("trocm_kv_cache_clone", self._h, C.byref(h), _sh(stream))
            c._h, c._shape, c._dtype = h, self._shape, self._dtype
        return c

    def close(self) -> None:
        """Release the device planes now (otherwise at garbage collection)."""
        if self._h:
            call("trocm_kv_cache_destroy", self._h)
            self._h = None

    def raw(self):
        """(data pointer, scales pointer or None, capacity) of the device planes."""
        d, sc, cap = C.c_void_p(), C.c_void_p(), C.c_int64()
        call("trocm_kv_cache_raw", self._h, C.byref(d), C.byref(sc), C.byref(cap))
        return d.value, sc.value, cap.value

    @property
    def handle(self):
        return self._h


class WindowKvCache(InPlaceKvCache):
    """Fixed-capacity sliding-window KV cache (ring buffer) along `axis`: once `window` slots are
    full an append overwrites the oldest; the valid slots are [0, len) in physical order."""

    def __init__(self, axis: int, window: int, storage_format: int | None = None):
        if window <= 0:
            raise TractRocmError("window must be > 0")
        super().__init__(axis, storage_format)
        self.window = window

    def _create(self, shape, dtype):
        if self.axis != len(shape) - 2:
            raise TractRocmError(f"kv-cache axis {self.axis} unsupported: the token axis must be rank-2")
        B, H, _, D = _canon4(shape)
        fmt = dtype_code(dtype) if self.storage_format is None else self.storage_format
        h = C.c_void_p()
        call("trocm_kv_cache_create_window", C.byref(h), fmt, B, H, D, self.window)
        self._h, self._shape, self._dtype, self.storage_format = h, tuple(shape), np.dtype(dtype), fmt

    def cursor(self) -> int:
        if self._h is None:
            return 0
        w, c = C.c_int64(), C.c_int64()
        call("trocm_kv_cache_window", self._h, C.byref(w), C.byref(c))
        return c.value

    def valid_view(self, stream=None) -> np.ndarray:
        return self.valid_contiguous(stream)

    def clone(self, stream=None) -> "WindowKvCache":
        c = WindowKvCache(self.axis, self.window, self.storage_format)
        if self._h is not None:
            h = C.c_void_p()
            call("trocm_kv_cache_clone", self._h, C.byref(h), _sh(stream))
            c._h, c._shape, c._dtype = h, self._shape, self._dtype
        return c


def _scale_arg(scale) -> float:
    return float("nan") if scale is None else float(scale)


class Sdpa:
    """Scaled dot-product attention on plain device tensors (sdpa.rs:83-89)."""

    def __init__(self, scale=None, datum_type=np.float32, acc_datum_type=np.float32, is_causal=False,
                 f16_flash_attention=False):
        """`f16_flash_attention=True` is what the reference's CUDA translator does to every Sdpa
        (convert_sdpa_to_cuda_flash_attn, cuda/src/transform.rs:358-406): Q, K, V and the mask are cast
        to f16, the f16 kernel runs, the output is cast back.  f32 inputs then take the MFMA kernels
        (and the f16 tolerance) instead of the generic f32 kernel; off by default (CPU parity)."""
        self.scale, self.datum_type, self.acc_datum_type, self.is_causal = scale, datum_type, acc_datum_type, is_causal
        self.f16_flash_attention = f16_flash_attention
        self._ws = None

    def output_facts(self, q_shape, k_shape, v_shape, mask_shape=None):
        """sdpa.rs:296-356."""
        if self.is_causal and mask_shape is not None:
            raise TractRocmError("Mask cannot be provided if is_causal=true")
        rank = len(q_shape)
        if rank not in (3, 4):
            raise TractRocmError("Input tensors must be 3D or 4D")
        if len(k_shape) != rank or len(v_shape) != rank:
            raise TractRocmError(f"Q, K and V should have the same rank {rank}")
        if rank == 4 and q_shape[1] % k_shape[1] != 0:
            raise TractRocmError(f"Q heads ({q_shape[1]}) must be a multiple of K/V heads ({k_shape[1]})")
        return tuple(q_shape[:-1]) + (v_shape[-1],)

    def eval(self, q, k, v, mask=None, stream=None, out=None) -> DeviceTensor:
        q, k, v = (_as_device(t, stream) for t in (q, k, v))
        m = None if mask is None else _as_device(mask, stream)
        self.output_facts(q.shape, k.shape, v.shape, None if m is None else m.shape)
        if not (q.dtype == k.dtype == v.dtype) or (m is not None and m.dtype != q.dtype):
            raise TractRocmError("Q, K, V and mask must share a datum type")
        B, Hq, Sq, D = _canon4(q.shape)
        _, Hkv, Sk, Dk = _canon4(k.shape)
        if _canon4(v.shape) != (B, Hkv, Sk, D) or Dk != D:
            raise TractRocmError("K/V shape mismatch")
        if self.f16_flash_attention and q.dtype == np.float32:
            half = Cast(np.float16)
            inner = Sdpa(self.scale, np.float16, self.acc_datum_type, self.is_causal)
            o16 = inner.eval(half.eval(q, stream), half.eval(k, stream), half.eval(v, stream),
                             None if m is None else half.eval(m, stream), stream)
            if out is None:
                out = DeviceTensor(q.shape, np.float32)
            elif tuple(out.shape) != tuple(q.shape) or out.dtype != np.float32:
                raise TractRocmError("out must have Q's shape and datum type")
            call("trocm_cast", o16.ptr, dtype_code(np.float16), out.ptr, dtype_code(np.float32),
                 int(np.prod(q.shape, dtype=np.int64)), _sh(stream))
            return out   # (the f16 temporaries are released by hipFree, which waits for the work that uses them)
        mb = mh = 1
        if m is not None:
            ms = _canon4(m.shape)
            if ms[2:] != (Sq, Sk):
                raise TractRocmError(f"mask shape {m.shape} does not end in [q_len, kv_len]")
            mb, mh = ms[0], ms[1]
        if out is None:
            out = DeviceTensor(q.shape, q.dtype)
        elif tuple(out.shape) != tuple(q.shape) or out.dtype != q.dtype:
            raise TractRocmError("out must have Q's shape and datum type")
        if self._ws is None or self._ws_key != (B, Hq, D) or self._ws.nbytes < Workspace.bytes_for(B, Hq, Sq, D):
            self._ws, self._ws_key = Workspace(B, Hq, Sq, D, stream), (B, Hq, D)
        call("trocm_sdpa", q.ptr, k.ptr, v.ptr, None if m is None else m.ptr, out.ptr, dtype_code(q.dtype),
             B, Hq, Hkv, Sq, Sk, D, None, mb, mh, _scale_arg(self.scale), int(self.is_causal),
             self._ws.ptr, self._ws.nbytes, _sh(stream))
        return out


class StreamedSdpaOp:
    """The row-streaming attention operator (streamed_sdpa.rs:6-10): Q, K, V of rank 3 or 4 and an optional rank-2
    mask [q_len, kv_len] shared by every batch and head; the output has Q's shape and datum type.

    It is served by the same kernels as Sdpa; what differs is stated here as the reference states it:
    * a mask takes precedence and the causal flag is then not consulted (streamed_sdpa.rs:216-222);
    * `causal` hides key i_k > t_q counted from the FIRST key (:218), whatever kv_len is, where Sdpa aligns the
      diagonal with the last key: with kv_len > q_len only the first q_len keys are ever visible and the kernels
      are given exactly those (no copy: a shorter kv_len over the same strides); with kv_len < q_len the rule is
      passed as a mask;
    * `block_k` (:8) only sets the order of the f32 sums on the CPU and is not used.
    Scores that are NaN or +inf, which the CPU loop steps over (:231-234, :247-249), are not given that treatment."""

    def __init__(self, causal: bool = False, block_k: int = 64, scale=None):
        self.causal, self.block_k, self.scale = bool(causal), int(block_k), scale
        self._ws = None

    def name(self) -> str:
        return "StreamedSDPA"

    def info(self):
        return [f"causal={self.causal}, block_k={self.block_k}, scale={self.scale}"]

    def output_facts(self, q_shape, k_shape, v_shape, mask_shape=None):
        """streamed_sdpa.rs:29-91."""
        if not (len(q_shape) == len(k_shape) == len(v_shape)):
            raise TractRocmError(f"Q, K and V must have the same rank, found {len(q_shape)}, {len(k_shape)}, {len(v_shape)} resp.")
        if len(q_shape) not in (3, 4):
            raise TractRocmError(f"Inputs must be of rank 3 or 4, found {len(q_shape)}")
        if mask_shape is not None and len(mask_shape) != 2:
            raise TractRocmError(f"Mask must be of rank 2, found mask {tuple(mask_shape)}")
        (bq, hq, _tq, dq), (bk, hkv, tk, dk), (bv, hkv2, tk2, dv) = _canon4(q_shape), _canon4(k_shape), _canon4(v_shape)
        if not (bq == bk == bv):
            raise TractRocmError("Batch dims must match for Q/K/V")
        if hkv != hkv2:
            raise TractRocmError("K/V head counts must match")
        if tk != tk2:
            raise TractRocmError("K/V lengths must match")
        if not (dq == dk == dv):
            raise TractRocmError("Head dims (D) must match across Q/K/V")
        if hq % hkv:
            raise TractRocmError("num_q_heads must be a multiple of num_kv_heads for GQA")
        return tuple(q_shape)

    def eval(self, q, k, v, mask=None, stream=None, out=None) -> DeviceTensor:
        q, k, v = (_as_device(t, stream) for t in (q, k, v))
        m = None if mask is None else _as_device(mask, stream)
        self.output_facts(q.shape, k.shape, v.shape, None if m is None else m.shape)
        if q.dtype not in (np.float32, np.float16) or not (q.dtype == k.dtype == v.dtype):
            raise TractRocmError("Q, K and V must be f32 or f16 and share a datum type")
        B, Hq, Sq, D = _canon4(q.shape)
        _, Hkv, Sk, _ = _canon4(k.shape)
        causal, kv_len = 0, Sk
        if m is not None:
            if tuple(m.shape) != (Sq, Sk):
                raise TractRocmError(f"mask shape {tuple(m.shape)} is not [q_len, kv_len] = [{Sq}, {Sk}]")
            if m.dtype != q.dtype:   # the reference casts any float mask to f32 (:143-152); here to the kernels' type
                m = Cast(q.dtype).eval(m, stream)
        elif self.causal:
            if Sk >= Sq:
                causal, kv_len = 1, Sq   # keys past the q_len-th are hidden from every query
            else:
                rule = np.where(np.arange(Sk)[None, :] > np.arange(Sq)[:, None], -np.inf, 0.0).astype(q.dtype)
                m = DeviceTensor.from_numpy(rule, stream)
        if out is None:
            out = DeviceTensor(q.shape, q.dtype)
        elif tuple(out.shape) != tuple(q.shape) or out.dtype != q.dtype:
            raise TractRocmError("out must have Q's shape and datum type")
        if self._ws is None or self._ws_key != (B, Hq, D) or self._ws.nbytes < Workspace.bytes_for(B, Hq, Sq, D):
            self._ws, self._ws_key = Workspace(B, Hq, Sq, D, stream), (B, Hq, D)
        strides = (C.c_int64 * 3)(Hkv * Sk * D, Sk * D, D)
        call("trocm_sdpa", q.ptr, k.ptr, v.ptr, None if m is None else m.ptr, out.ptr, dtype_code(q.dtype),
             B, Hq, Hkv, Sq, kv_len, D, strides, 1, 1, _scale_arg(self.scale), causal,
             self._ws.ptr, self._ws.nbytes, _sh(stream))
        return out


class InPlaceKvSdpa:
    """Fused in-place KV-cache + attention op: inputs [Q, K_new, V_new], output Q-shaped."""

    def __init__(self, axis: int = 2, causal: bool = True, scale=None, storage_format: int | None = None):
        self.axis, self.causal, self.scale, self.storage_format = axis, causal, scale, storage_format

    def name(self) -> str:
        return "InPlaceKvSdpa"

    def is_stateless(self) -> bool:
        return False

    def state(self) -> "InPlaceKvSdpaState":
        return InPlaceKvSdpaState(self.axis, self.causal, self.scale, self.storage_format)

    def output_facts(self, *shapes):
        if len(shapes) != 3:
            raise TractRocmError("InPlaceKvSdpa expects [Q, K_new, V_new]")
        return tuple(shapes[0])


class InPlaceKvSdpaState:
    def __init__(self, axis, causal, scale, storage_format=None):
        self.axis, self.causal, self.scale, self.storage_format = axis, causal, scale, storage_format
        self.k = InPlaceKvCache(axis, storage_format)
        self.v = InPlaceKvCache(axis, storage_format)
        self._ws = None
        self._ws_key = None

    def eval(self, inputs, stream=None) -> DeviceTensor:
        if len(inputs) != 3:
            raise TractRocmError("InPlaceKvSdpa expects [Q, K_new, V_new]")
        q, k_new, v_new = (_as_device(t, stream) for t in inputs)
        return self.eval_into(q, k_new, v_new, None, stream)

    def eval_into(self, q: DeviceTensor, k_new: DeviceTensor, v_new: DeviceTensor, out: DeviceTensor | None = None,
                  stream=None) -> DeviceTensor:
        """`eval` on device tensors with a caller-provided output: one C call per step (the two
        pushes share a launch) once the caches exist."""
        fused = (self.k.handle is not None and self.v.handle is not None and k_new.shape == v_new.shape
                 and k_new.dtype == v_new.dtype == q.dtype and len(q.shape) == len(k_new.shape)
                 and q.shape[self.axis] == k_new.shape[self.axis])
        if not fused:
            self.k.push(k_new, stream=stream)
            self.v.push(v_new, stream=stream)
            return self.attend(q, stream, out)
        self.k._check_push_shape(k_new.shape)
        B, Hq, Sq, D = _canon4(q.shape)
        if out is None:
            out = DeviceTensor(q.shape, q.dtype)
        if self._ws is None or self._ws_key != (B, Hq, D) or self._ws.nbytes < Workspace.bytes_for(B, Hq, Sq, D):
            self._ws, self._ws_key = Workspace(B, Hq, Sq, D, stream), (B, Hq, D)
        call("trocm_inplace_kv_sdpa_eval", q.ptr, k_new.ptr, v_new.ptr, dtype_code(q.dtype), Hq, Sq, None,
             self.k.handle, self.v.handle, out.ptr, _scale_arg(self.scale), int(self.causal),
             self._ws.ptr, self._ws.nbytes, _sh(stream))
        return out

    def eval_rope_into(self, q: DeviceTensor, k_new: DeviceTensor, v_new: DeviceTensor, cos: DeviceTensor, sin: DeviceTensor,
                       out: DeviceTensor | None = None, stream=None) -> DeviceTensor:
        """ApplyRope on Q and K_new (Cos and Sin of shape [1 or batch, 1, n_new, head_dim]), then `eval`: one C call, and
        for a single-token step on an f16 cache one launch."""
        if not (q.dtype == k_new.dtype == v_new.dtype == cos.dtype == sin.dtype):
            raise TractRocmError("input, cos and sin must share a datum type")
        if tuple(cos.shape) != tuple(sin.shape):
            raise TractRocmError("cos and sin must have the same shape")
        B, Hq, Sq, D = _canon4(q.shape)
        Hkv = _canon4(k_new.shape)[1]
        cb = _canon4(cos.shape)
        if cb[1] != 1 or cb[2] != Sq or cb[3] != D or cb[0] not in (1, B):
            raise TractRocmError(f"cos / sin of shape {tuple(cos.shape)} do not broadcast against Q {tuple(q.shape)} over heads")
        if self.k.handle is None:   # first chunk: the caches take their shape from it
            rq = ApplyRope().eval(q, cos, sin, stream)
            rk = ApplyRope().eval(k_new, cos, sin, stream)
            return self.eval_into(rq, rk, v_new, out, stream)
        self.k._check_push_shape(k_new.shape)
        if out is None:
            out = DeviceTensor(q.shape, q.dtype)
        if self._ws is None or self._ws_key != (B, Hq, D) or self._ws.nbytes < Workspace.bytes_for(B, Hq, Sq, D):
            self._ws, self._ws_key = Workspace(B, Hq, Sq, D, stream), (B, Hq, D)
        es = np.dtype(q.dtype).itemsize
        need = ((B * Hq * Sq * D * es + 255) & ~255) + B * Hkv * Sq * D * es
        rot = getattr(self, "_rot", None)
        if rot is None or rot.nbytes < need:
            rot = self._rot = DeviceTensor((need,), np.uint8)
        call("trocm_inplace_kv_sdpa_eval_rope", q.ptr, k_new.ptr, v_new.ptr, cos.ptr, sin.ptr, 0 if cb[0] == 1 else Sq * D,
             dtype_code(q.dtype), Hq, Sq, self.k.handle, self.v.handle, out.ptr, _scale_arg(self.scale), int(self.causal),
             self._ws.ptr, self._ws.nbytes, rot.ptr, rot.nbytes, _sh(stream))
        return out

    def attend(self, q: DeviceTensor, stream=None, out: DeviceTensor | None = None) -> DeviceTensor:
        B, Hq, Sq, D = _canon4(q.shape)
        if out is None:
            out = DeviceTensor(q.shape, q.dtype)
        if self._ws is None or self._ws_key != (B, Hq, D) or self._ws.nbytes < Workspace.bytes_for(B, Hq, Sq, D):
            self._ws, self._ws_key = Workspace(B, Hq, Sq, D, stream), (B, Hq, D)
        if self.k.handle is None:
            raise TractRocmError("empty kv-cache")
        call("trocm_sdpa_cached", q.ptr, dtype_code(q.dtype), Hq, Sq, self.k.handle, self.v.handle, out.ptr,
             _scale_arg(self.scale), int(self.causal), self._ws.ptr, self._ws.nbytes, _sh(stream))
        return out

    def attend_noalloc(self, q: DeviceTensor, out: DeviceTensor, stream) -> DeviceTensor:
        """`attend` through the entry point that allocates nothing (the library's static split-K
        scratch): `out` and `stream` are the caller's; calls that overlap in time race on the scratch."""
        B, Hq, Sq, D = _canon4(q.shape)
        if self.k.handle is None:
            raise TractRocmError("empty kv-cache")
        call("trocm_sdpa_cached_noalloc", q.ptr, dtype_code(q.dtype), Hq, Sq, self.k.handle, self.v.handle, out.ptr,
             _scale_arg(self.scale), int(self.causal), _sh(stream))
        return out

    def save_to(self, states: list) -> None:
        if not self.k.is_empty():
            states.append(self.k.valid_contiguous())
            states.append(self.v.valid_contiguous())

    def load_from(self, states) -> None:
        it = iter(states)
        k = next(it, None)
        if k is not None:
            v = next(it, None)
            if v is None:
                raise TractRocmError("InPlaceKvSdpa load_from: expected V state after K")
            self.k = InPlaceKvCache(self.axis, self.storage_format)
            self.v = InPlaceKvCache(self.axis, self.storage_format)
            self.k.push(k)
            self.v.push(v)

    def freeze(self) -> "InPlaceKvSdpaState":
        f = InPlaceKvSdpaState(self.axis, self.causal, self.scale, self.storage_format)
        f.k, f.v = self.k.clone(), self.v.clone()
        return f

    def unfreeze(self) -> "InPlaceKvSdpaState":
        return self.freeze()


class WindowKvSdpa:
    """Fused sliding-window KV-cache + attention (decode): inputs [Q, K_new, V_new], each
    [B, H, S, D]; output has Q's shape.  The bounded cache is the sliding window."""

    def __init__(self, axis: int = 2, window: int = 4096, scale=None, storage_format: int | None = None):
        self.axis, self.window, self.scale, self.storage_format = axis, window, scale, storage_format

    def name(self) -> str:
        return "WindowKvSdpa"

    def is_stateless(self) -> bool:
        return False

    def state(self) -> "WindowKvSdpaState":
        return WindowKvSdpaState(self.axis, self.window, self.scale, self.storage_format)

    def output_facts(self, *shapes):
        if len(shapes) != 3:
            raise TractRocmError("WindowKvSdpa expects [Q, K_new, V_new]")
        return tuple(shapes[0])


class WindowKvSdpaState:
    def __init__(self, axis, window, scale, storage_format=None):
        self.axis, self.window, self.scale, self.storage_format = axis, window, scale, storage_format
        self.k = WindowKvCache(axis, window, storage_format)
        self.v = WindowKvCache(axis, window, storage_format)
        self._ws = None

    def eval(self, inputs, stream=None, out: DeviceTensor | None = None) -> DeviceTensor:
        if len(inputs) != 3:
            raise TractRocmError("WindowKvSdpa expects [Q, K_new, V_new]")
        q, k_new, v_new = (_as_device(t, stream) for t in inputs)
        if k_new.shape != v_new.shape or not (q.dtype == k_new.dtype == v_new.dtype):
            raise TractRocmError("K_new and V_new must share shape and datum type with Q's type")
        for c, t in ((self.k, k_new), (self.v, v_new)):
            if c.handle is None:
                c._create(t.shape, t.dtype)
            c._check_push_shape(t.shape)
        B, Hq, Sq, D = _canon4(q.shape)
        S = _canon4(k_new.shape)[2]
        if out is None:
            out = DeviceTensor(q.shape, q.dtype)
        if self._ws is None or self._ws.nbytes < Workspace.bytes_for(B, Hq, Sq, D):
            self._ws = Workspace(B, Hq, Sq, D, stream)
        call("trocm_window_kv_sdpa_eval", q.ptr, k_new.ptr, v_new.ptr, dtype_code(q.dtype), Hq, S, None,
             self.k.handle, self.v.handle, out.ptr, _scale_arg(self.scale), self._ws.ptr, self._ws.nbytes, _sh(stream))
        return out

    def freeze(self) -> "WindowKvSdpaState":
        f = WindowKvSdpaState(self.axis, self.window, self.scale, self.storage_format)
        f.k, f.v = self.k.clone(), self.v.clone()
        return f

    def unfreeze(self) -> "WindowKvSdpaState":
        return self.freeze()


class DynKeyValueCache:
    """The dynamic KV-cache op (dyn_kv_cache.rs:177-183): one input, output = whole cache."""

    def __init__(self, name: str, axis: int, storage_format: int | None = None):
        self.name, self.axis, self.storage_format = name, axis, storage_format

    def is_stateless(self) -> bool:
        return False

    def state(self) -> "DynKeyValueCacheState":
        return DynKeyValueCacheState(self.name, self.axis, self.storage_format)


class DynKeyValueCacheState:
    def __init__(self, name, axis, storage_format=None):
        self.name, self.axis = name, axis
        self.kv_cache = InPlaceKvCache(axis, storage_format)

    def eval(self, x, stream=None) -> InPlaceKvCache:
        """Appends in place and returns the cache itself: consumers read (buffer, capacity, len)
        instead of a freshly concatenated tensor."""
        self.kv_cache.push(x, stream=stream)
        return self.kv_cache

    def resolve_symbols(self) -> int:
        """The value bound to the past-length symbol P (dyn_kv_cache.rs:153-156)."""
        return self.kv_cache.len()

    def truncate(self, length: int) -> None:
        if self.kv_cache.handle is None:
            raise TractRocmError("Can not truncate a zero-len kv-cache value")
        self.kv_cache.truncate(length)

    def save_to(self, states: list) -> None:
        if self.kv_cache.handle is None:
            raise TractRocmError(f"KV cache {self.name} was never initialized")
        states.append(self.kv_cache.valid_contiguous())

    def load_from(self, states) -> None:
        it = iter(states)
        t = next(it, None)
        if t is None:
            raise TractRocmError("Not enough state initializers")
        self.kv_cache = InPlaceKvCache(self.axis, self.kv_cache.storage_format)
        self.kv_cache.push(t)

    def freeze(self) -> "DynKeyValueCacheState":
        f = DynKeyValueCacheState(self.name, self.axis, self.kv_cache.storage_format)
        f.kv_cache = self.kv_cache.clone()
        return f

    unfreeze = freeze


class BlockQuant:
    """A block-quantisation format as a tensor op (block_quant/mod.rs:36-108)."""

    def __init__(self, fmt: int, name: str, block_bytes: int):
        self.fmt, self.name, self._bb = fmt, name, block_bytes

    def block_len(self) -> int:
        return 32

    def block_bytes(self) -> int:
        return self._bb

    def _quant(self, x: np.ndarray, stream=None) -> np.ndarray:
        if x.size % 32:
            raise TractRocmError(f"{x.size} elements is not a multiple of the block length 32")
        src = DeviceTensor.from_numpy(x, stream)
        dst = DeviceTensor((x.size // 32 * self._bb,), np.uint8)
        call("trocm_block_quant", self.fmt, src.ptr, dtype_code(x.dtype), x.size, dst.ptr, _sh(stream))
        return dst.to_numpy(stream)

    def quant_f32(self, x, stream=None) -> np.ndarray:
        return self._quant(np.ascontiguousarray(x, dtype=np.float32), stream)

    def quant_f16(self, x, stream=None) -> np.ndarray:
        return self._quant(np.ascontiguousarray(x, dtype=np.float16), stream)

    def _dequant(self, blob, dtype, stream=None) -> np.ndarray:
        blob = np.ascontiguousarray(blob, dtype=np.uint8).reshape(-1)
        if blob.size % self._bb:
            raise TractRocmError(f"{blob.size} bytes is not a multiple of the block size {self._bb}")
        n = blob.size // self._bb * 32
        src = DeviceTensor.from_numpy(blob, stream)
        dst = DeviceTensor((n,), dtype)
        call("trocm_block_dequant", self.fmt, src.ptr, n, dst.ptr, dtype_code(dtype), _sh(stream))
        return dst.to_numpy(stream)

    def simulate_precision_loss(self, tensor, block_axis: int, stream=None) -> np.ndarray:
        """block_quant/mod.rs:130-154: the tensor after a round trip through the format, in its own type (f32 or
        f16); blocks run along `block_axis`, which must be the last axis."""
        x = np.ascontiguousarray(tensor)
        if x.dtype not in (np.float32, np.float16):
            raise TractRocmError(f"simulate_precision_loss takes f32 or f16 tensors, got {x.dtype}")
        if block_axis != x.ndim - 1:
            raise TractRocmError(f"block axis {block_axis} is not the last axis of a rank {x.ndim} tensor")
        if x.shape[-1] % 32:
            raise TractRocmError(f"{x.shape[-1]} elements along the block axis is not a multiple of the block length 32")
        t = DeviceTensor.from_numpy(x, stream)
        call("trocm_block_simulate_precision_loss", self.fmt, t.ptr, t.ptr, dtype_code(x.dtype), x.size, _sh(stream))
        return t.to_numpy(stream)

    def dequant_f32(self, blob, stream=None) -> np.ndarray:
        return self._dequant(blob, np.float32, stream)

    def dequant_f16(self, blob, stream=None) -> np.ndarray:
        return self._dequant(blob, np.float16, stream)


Q4_0_FORMAT = BlockQuant(Q4_0, "Q4_0", 18)
Q8_0_FORMAT = BlockQuant(Q8_0, "Q8_0", 34)


class Q40Weights:
    """Q4_0 weights [batch, n, k] resident on the device (BlockQuantStorage rows of k/32 blocks,
    block_quant/storage.rs:14-59), as the matrix-vector arm of GgmlGemm takes them."""

    def __init__(self, blocks, batch: int, n: int, k: int, stream=None):
        if k % 32:
            raise TractRocmError(f"k = {k} is not a whole number of 32-element blocks")
        if isinstance(blocks, DeviceTensor):
            src = blocks
        else:
            src = DeviceTensor.from_numpy(np.ascontiguousarray(blocks, dtype=np.uint8).reshape(-1), stream)
        if src.nbytes != batch * n * (k // 32) * 18:
            raise TractRocmError(f"{src.nbytes} bytes of blocks do not make a [{batch}, {n}, {k}] Q4_0 tensor")
        h = C.c_void_p()
        call("trocm_q4_0_weights_create", C.byref(h), src.ptr, batch, n, k, _sh(stream))
        self.handle, self.batch, self.n, self.k = h, batch, n, k
        synchronize() if stream is None else stream.synchronize()   # `src` may be released now

    @classmethod
    def quantize(cls, w: np.ndarray, stream=None) -> "Q40Weights":
        """Quantise a dense [batch, n, k] (or [n, k]) tensor with Q4_0 along k (BlockQuant::quant_f32)."""
        w = np.asarray(w)
        if w.ndim == 2:
            w = w[None]
        b, n, k = w.shape
        blob = Q4_0_FORMAT.quant_f16(w, stream) if w.dtype == np.float16 else Q4_0_FORMAT.quant_f32(w, stream)
        return cls(blob, b, n, k, stream)

    def blocks(self, stream=None) -> np.ndarray:
        """The canonical blocks, uint8 [batch, n, k/32 * 18]."""
        dst = DeviceTensor((self.batch, self.n, self.k // 32 * 18), np.uint8)
        call("trocm_q4_0_weights_export", self.handle, dst.ptr, _sh(stream))
        return dst.to_numpy(stream)

    def close(self):
        if getattr(self, "handle", None):
            call("trocm_q4_0_weights_destroy", self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class GgmlGemm:
    """Activations [b, m, k] x Q4_0 weights [b_w, n, k] -> [b, m, n]; built for m <= 8 (GgmlGemm::dispatch_eval,
    cuda/src/kernels/matmul/mod.rs:575-627; output_shape :536-545)."""

    def output_shape(self, act_shape, w_shape):
        return tuple(act_shape[:-2]) + (act_shape[-2], w_shape[-2])

    def eval(self, activs, weights: Q40Weights, stream=None, out=None) -> DeviceTensor:
        a = _as_device(activs, stream)
        if a.dtype not in (np.float32, np.float16):
            raise TractRocmError("activations must be f32 or f16")
        shape = tuple(a.shape)
        if len(shape) == 2:
            shape = (1,) + shape
        if len(shape) != 3 or shape[2] != weights.k:
            raise TractRocmError(f"activations {tuple(a.shape)} do not match weights [.., {weights.n}, {weights.k}]")
        b, m, _ = shape
        oshape = tuple(a.shape[:-1]) + (weights.n,)
        if out is None:
            out = DeviceTensor(oshape, a.dtype)
        elif tuple(out.shape) != oshape or out.dtype != a.dtype:
            raise TractRocmError("out must have shape [.., m, n] and the activations' datum type")
        call("trocm_q4_0_matvec", weights.handle, a.ptr, dtype_code(a.dtype), b, m, out.ptr, _sh(stream))
        return out


def sdpa_decode_ragged(q: DeviceTensor, k_caches, v_caches, scale=None, workspace: Workspace | None = None,
                       stream=None, out: DeviceTensor | None = None) -> DeviceTensor:
    """One decode step for `n_seq` independent sequences with their own caches and lengths.
    q: [n_seq, Hq, 1, D]."""
    n, Hq, _, D = q.shape
    if len(k_caches) != n or len(v_caches) != n:
        raise TractRocmError("ragged decode: one K and one V cache per sequence expected")
    if out is None:
        out = DeviceTensor(q.shape, q.dtype)
    ws = workspace or Workspace(n, Hq, 1, D, stream)
    ks = (C.c_void_p * n)(*[c.handle for c in k_caches])
    vs = (C.c_void_p * n)(*[c.handle for c in v_caches])
    call("trocm_sdpa_decode_ragged", q.ptr, dtype_code(q.dtype), Hq, n, ks, vs, out.ptr, _scale_arg(scale),
         ws.ptr, ws.nbytes, _sh(stream))
    return out


def inplace_kv_sdpa_eval_ragged(q: DeviceTensor, k_new: DeviceTensor, v_new: DeviceTensor, k_caches, v_caches,
                                scale=None, workspace: Workspace | None = None, stream=None,
                                out: DeviceTensor | None = None) -> DeviceTensor:
    """One decode step for `n_seq` independent sequences: append k_new[i], v_new[i]
    ([n_seq, Hkv, 1, D]) to sequence i's caches and attend q[i] ([n_seq, Hq, 1, D]) over them."""
    n, Hq, _, D = q.shape
    if len(k_caches) != n or len(v_caches) != n:
        raise TractRocmError("ragged decode: one K and one V cache per sequence expected")
    if k_new.shape != v_new.shape or k_new.shape[0] != n or k_new.shape[2] != 1:
        raise TractRocmError("ragged decode: k_new / v_new must be [n_seq, kv_heads, 1, head_dim]")
    if out is None:
        out = DeviceTensor(q.shape, q.dtype)
    ws = workspace or Workspace(n, Hq, 1, D, stream)
    ks = (C.c_void_p * n)(*[c.handle for c in k_caches])
    vs = (C.c_void_p * n)(*[c.handle for c in v_caches])
    call("trocm_inplace_kv_sdpa_eval_ragged", q.ptr, k_new.ptr, v_new.ptr, dtype_code(q.dtype), Hq, n, ks, vs,
         out.ptr, _scale_arg(scale), ws.ptr, ws.nbytes, _sh(stream))
    return out


def inplace_kv_sdpa_eval_ragged_rope(q: DeviceTensor, k_new: DeviceTensor, v_new: DeviceTensor, cos: DeviceTensor, sin: DeviceTensor,
                                     k_caches, v_caches, scale=None, workspace: Workspace | None = None, stream=None,
                                     out: DeviceTensor | None = None, rot_scratch: DeviceTensor | None = None) -> DeviceTensor:
    """`inplace_kv_sdpa_eval_ragged` with ApplyRope on q and k_new folded in; cos and sin are [n_seq, 1, 1, head_dim] (every
    sequence's own position)."""
    n, Hq, _, D = q.shape
    if len(k_caches) != n or len(v_caches) != n:
        raise TractRocmError("ragged decode: one K and one V cache per sequence expected")
    if k_new.shape != v_new.shape or k_new.shape[0] != n or k_new.shape[2] != 1:
        raise TractRocmError("ragged decode: k_new / v_new must be [n_seq, kv_heads, 1, head_dim]")
    if tuple(cos.shape) != tuple(sin.shape) or int(np.prod(cos.shape)) != n * D or cos.shape[0] != n or cos.shape[-1] != D:
        raise TractRocmError("ragged decode with RoPE: cos and sin must be [n_seq, 1, 1, head_dim]")
    if not (q.dtype == k_new.dtype == cos.dtype == sin.dtype):
        raise TractRocmError("input, cos and sin must share a datum type")
    if out is None:
        out = DeviceTensor(q.shape, q.dtype)
    ws = workspace or Workspace(n, Hq, 1, D, stream)
    es = np.dtype(q.dtype).itemsize
    need = ((n * Hq * D * es + 255) & ~255) + n * k_new.shape[1] * D * es
    if rot_scratch is None:
        rot_scratch = DeviceTensor((need,), np.uint8)
    ks = (C.c_void_p * n)(*[c.handle for c in k_caches])
    vs = (C.c_void_p * n)(*[c.handle for c in v_caches])
    call("trocm_inplace_kv_sdpa_eval_ragged_rope", q.ptr, k_new.ptr, v_new.ptr, cos.ptr, sin.ptr, dtype_code(q.dtype), Hq, n, ks, vs,
         out.ptr, _scale_arg(scale), ws.ptr, ws.nbytes, rot_scratch.ptr, rot_scratch.nbytes, _sh(stream))
    return out


def _broadcast_strides(x_shape, c_shape):
    """Element strides of a dense tensor of shape ``c_shape`` broadcast against ``x_shape``
    (0 on broadcast axes), for x's rank: cuda/src/kernels/utils.rs compute_broadcast_strides."""
    if len(c_shape) > len(x_shape):
        raise TractRocmError("cos/sin rank exceeds the input rank")
    pad = (1,) * (len(x_shape) - len(c_shape)) + tuple(c_shape)
    out, acc = [], 1
    for d in range(len(x_shape) - 1, -1, -1):
        if pad[d] not in (1, x_shape[d]):
            raise TractRocmError(f"cos/sin shape {tuple(c_shape)} does not broadcast against {tuple(x_shape)}")
        out.append(0 if pad[d] == 1 and x_shape[d] != 1 else acc)
        acc *= pad[d]
    return out[::-1]


class RotateHalf:
    """Y = Concat(Neg(Slice(X, h.., -1)), Slice(X, ..h, -1)), h = half the innermost axis."""

    def name(self) -> str:
        return "RotateHalf"

    def is_stateless(self) -> bool:
        return True

    def output_facts(self, shape):
        return tuple(shape)

    def eval(self, x, stream=None) -> DeviceTensor:
        x = _as_device(x, stream)
        out = DeviceTensor(x.shape, x.dtype)
        shp = (C.c_int64 * len(x.shape))(*x.shape)
        call("trocm_rotate_half", x.ptr, out.ptr, dtype_code(x.dtype), len(x.shape), shp, None, None, _sh(stream))
        return out


class ApplyRope:
    """Y = X * Cos + RotateHalf(X) * Sin, inputs [X, Cos, Sin]; Cos and Sin share a shape that
    broadcasts against X."""

    @staticmethod
    def is_supported_dt(dt) -> bool:
        return np.dtype(dt) in (np.dtype(np.float32), np.dtype(np.float16))

    def name(self) -> str:
        return "ApplyRope"

    def is_stateless(self) -> bool:
        return True

    def output_facts(self, x_shape, cos_shape=None, sin_shape=None):
        return tuple(x_shape)

    def eval(self, x, cos, sin, stream=None, out: DeviceTensor | None = None) -> DeviceTensor:
        x, cos, sin = (_as_device(t, stream) for t in (x, cos, sin))
        if not (x.dtype == cos.dtype == sin.dtype):
            raise TractRocmError("input, cos and sin must share a datum type")
        if tuple(cos.shape) != tuple(sin.shape):
            raise TractRocmError("cos and sin must have the same shape")
        cs = _broadcast_strides(x.shape, cos.shape)
        if out is None:
            out = DeviceTensor(x.shape, x.dtype)
        n = len(x.shape)
        call("trocm_apply_rope", x.ptr, cos.ptr, sin.ptr, out.ptr, dtype_code(x.dtype), n, (C.c_int64 * n)(*x.shape),
             None, (C.c_int64 * n)(*cs), None, _sh(stream))
        return out


class Cast:
    """Cast between f32 and f16 (round to nearest even on the way down)."""

    def __init__(self, to):
        self.to = np.dtype(to)

    def name(self) -> str:
        return "Cast"

    def eval(self, x, stream=None) -> DeviceTensor:
        x = _as_device(x, stream)
        out = DeviceTensor(x.shape, self.to)
        call("trocm_cast", x.ptr, dtype_code(x.dtype), out.ptr, dtype_code(self.to), int(np.prod(x.shape, dtype=np.int64)),
             _sh(stream))
        return out
