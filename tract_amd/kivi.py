"""Host-side mirror of tract's KIVI-style quantised cache operators over the rocm C ABI.

* ``QuantizedDynKeyValueCache``/State  transformers/src/ops/quant_dyn_kv_cache.rs:283-495 (Values per token,
  Keys per channel in frozen blocks of 32 tokens, 4 sink tokens in f32; the op's output is the whole cache
  dequantised to the input type)
* ``QuantizedKvSdpa``/State            transformers/src/ops/kv_quant.rs:242-355 (u8 codes, running per-channel
  key parameters, non-causal attention over the dequantised cache)
* ``quant_dequant``                    transformers/src/ops/kv_quant.rs:73-98 at 4 and 8 bits
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib
from ._lib import TractRocmError, call
from .runtime import DeviceTensor, Workspace, _sh, dtype_code

KIVI_PER_TOKEN, KIVI_BLOCK_CHANNEL, KIVI_RUNNING_CHANNEL = 0, 1, 2
SINK_TOKENS, KEY_BLOCK = 4, 32          # quant_dyn_kv_cache.rs:92, :153
_PARTS = {"sink": (0, np.float32), "packed": (1, np.uint8), "lo": (2, np.float32), "scale": (3, np.float32),
          "residual": (4, np.float32)}


def _as_device(x, stream=None) -> DeviceTensor:
    return x if isinstance(x, DeviceTensor) else DeviceTensor.from_numpy(np.asarray(x), stream)


class KiviCache:
    """One quantised tensor [batch, heads, len, head_dim] on the device: the HeadCache of every (batch, head)
    (quant_dyn_kv_cache.rs:252-281)."""

    def __init__(self, layout: int, bits: int, sink_tokens: int, batch: int, heads: int, head_dim: int, _handle=None):
        self.layout, self.bits, self.sink_tokens = layout, bits, sink_tokens
        self.batch, self.heads, self.head_dim = batch, heads, head_dim
        if _handle is None:
            _handle = C.c_void_p()
            call("trocm_kivi_cache_create", C.byref(_handle), layout, bits, sink_tokens, batch, heads, head_dim)
        self.handle = _handle

    def __del__(self):
        try:
            if self.handle:
                _lib.load().trocm_kivi_cache_destroy(self.handle)
                self.handle = None
        except Exception:
            pass

    def len(self) -> int:
        n = C.c_int64()
        call("trocm_kivi_cache_len", self.handle, C.byref(n))
        return n.value

    def reset(self, stream=None) -> None:
        """The empty state of a new session, keeping the device buffers."""
        call("trocm_kivi_cache_reset", self.handle, _sh(stream))

    def counts(self) -> dict:
        a, b, c, d = C.c_int64(), C.c_int64(), C.c_int64(), C.c_int64()
        call("trocm_kivi_cache_counts", self.handle, C.byref(a), C.byref(b), C.byref(c), C.byref(d))
        return {"n_sink": a.value, "n_rows": b.value, "n_res": c.value, "row_bytes": d.value}

    def memory_bytes(self) -> int:
        n = C.c_size_t()
        call("trocm_kivi_cache_memory_bytes", self.handle, C.byref(n))
        return n.value

    def append(self, x, stream=None) -> None:
        x = _as_device(x, stream)
        if len(x.shape) != 4:
            raise TractRocmError("quantized KV cache supports rank-4 [B, H, S, D] caches")
        if (x.shape[0], x.shape[1], x.shape[3]) != (self.batch, self.heads, self.head_dim):
            raise TractRocmError("cache shape changed between steps")
        call("trocm_kivi_cache_append", self.handle, x.ptr, dtype_code(x.dtype), x.shape[2], _sh(stream))

    def dequantize(self, dtype=np.float32, stream=None, out: DeviceTensor | None = None) -> DeviceTensor:
        if out is None:
            out = DeviceTensor((self.batch, self.heads, self.len(), self.head_dim), dtype)
        call("trocm_kivi_cache_dequantize", self.handle, out.ptr, dtype_code(out.dtype), _sh(stream))
        return out

    def state(self, stream=None) -> dict:
        """The raw state as numpy arrays, one leading row per (batch, head): sink [BH, n_sink, D] f32, packed
        [BH, n_rows, row_bytes] u8, lo / scale f32, residual [BH, n_res, D] f32."""
        bh, out = self.batch * self.heads, {}
        for name, (part, dt) in _PARTS.items():
            n = C.c_size_t()
            call("trocm_kivi_cache_export", self.handle, part, None, C.byref(n), _sh(stream))
            t = DeviceTensor((n.value // np.dtype(dt).itemsize,), dt)
            if n.value:
                call("trocm_kivi_cache_export", self.handle, part, t.ptr, C.byref(n), _sh(stream))
            out[name] = t.to_numpy(stream).reshape(bh, -1)
        c = self.counts()
        out["sink"] = out["sink"].reshape(bh, c["n_sink"], self.head_dim)
        out["packed"] = out["packed"].reshape(bh, c["n_rows"], c["row_bytes"])
        out["residual"] = out["residual"].reshape(bh, c["n_res"], self.head_dim)
        return out

    def clone(self, stream=None) -> "KiviCache":
        h = C.c_void_p()
        call("trocm_kivi_cache_clone", self.handle, C.byref(h), _sh(stream))
        return KiviCache(self.layout, self.bits, self.sink_tokens, self.batch, self.heads, self.head_dim, _handle=h)


class QuantizedDynKeyValueCache:
    """quant_dyn_kv_cache.rs:283-292: `per_channel` selects the KIVI layout (Keys: True, Values: False), `bits`
    is 4 or 8, the sequence axis must be 2 of [B, H, S, D]."""

    def __init__(self, name: str, axis: int = 2, bits: int = 8, per_channel: bool = False):
        if bits not in (4, 8):
            raise TractRocmError("KV quantization bits must be 4 or 8")
        self.name, self.axis, self.bits, self.per_channel = name, axis, bits, per_channel

    def op_name(self) -> str:
        return "QuantizedDynKeyValueCache"

    def info(self):
        return [f"bits={self.bits}, per_channel={str(self.per_channel).lower()}, axis={self.axis}"]

    def is_stateless(self) -> bool:
        return False

    def state(self) -> "QuantizedDynKvCacheState":
        return QuantizedDynKvCacheState(self.name, self.axis, self.bits, self.per_channel)

    def output_facts(self, input_shape, past_len: int):
        shape = list(input_shape)
        shape[self.axis] = past_len + input_shape[self.axis]
        return tuple(shape)

    def cost(self, shape):
        """quant_dyn_kv_cache.rs:318-336: values per token and resident bytes per token."""
        values = int(np.prod([d for a, d in enumerate(shape) if a != self.axis]))
        return {"KVCacheValuesPerToken": values, "KVCacheQuantBytesPerToken": values * max(self.bits, 1) // 8}


class QuantizedDynKvCacheState:
    def __init__(self, name, axis, bits, per_channel):
        self.name, self.axis, self.bits, self.per_channel = name, axis, bits, per_channel
        self.cache: KiviCache | None = None

    def _ingest(self, x: DeviceTensor, stream=None) -> None:
        if len(x.shape) != 4:
            raise TractRocmError("quantized KV cache supports rank-4 [B, H, S, D] caches")
        if self.axis != 2:
            raise TractRocmError("seq axis must be 2 ([B, H, S, D])")
        b, h, _, d = x.shape
        if self.cache is None:
            layout = KIVI_BLOCK_CHANNEL if self.per_channel else KIVI_PER_TOKEN
            self.cache = KiviCache(layout, self.bits, SINK_TOKENS, b, h, d)
        self.cache.append(x, stream)

    def eval(self, x, stream=None) -> DeviceTensor:
        """:477-494: ingest the new tokens, return the whole cache in the input's type."""
        x = _as_device(x, stream)
        self._ingest(x, stream)
        return self.cache.dequantize(x.dtype, stream)

    def resolve_symbols(self) -> int:
        return 0 if self.cache is None else self.cache.len()

    def load_from(self, states, stream=None) -> None:
        t = next(iter(states), None)
        if t is None:
            raise TractRocmError("Not enough state initializers")
        self._ingest(_as_device(t, stream), stream)

    def save_to(self, states: list, stream=None) -> None:
        states.append(self.cache.dequantize(np.float32, stream).to_numpy(stream))

    def freeze(self) -> "QuantizedDynKvCacheState":
        f = QuantizedDynKvCacheState(self.name, self.axis, self.bits, self.per_channel)
        f.cache = None if self.cache is None else self.cache.clone()
        return f

    unfreeze = freeze


class QuantizedKvSdpa:
    """kv_quant.rs:242-280: fused quantised KV cache + attention; inputs [Q, K_new, V_new] each [B, H, S, D]."""

    def __init__(self, axis: int = 2, scale=None):
        self.axis, self.scale = axis, scale

    def name(self) -> str:
        return "QuantizedKvSdpa"

    def info(self):
        return [f"axis={self.axis}, scale={self.scale}"]

    def is_stateless(self) -> bool:
        return False

    def state(self) -> "QuantizedKvSdpaState":
        return QuantizedKvSdpaState(self.scale)

    def output_facts(self, *shapes):
        if len(shapes) != 3:
            raise TractRocmError("QuantizedKvSdpa expects [Q, K_new, V_new]")
        return tuple(shapes[0])


class QuantizedKvSdpaState:
    def __init__(self, scale=None):
        self.scale = scale
        self.k: KiviCache | None = None
        self.v: KiviCache | None = None
        self._ws = None

    def eval(self, inputs, stream=None, out: DeviceTensor | None = None) -> DeviceTensor:
        if len(inputs) != 3:
            raise TractRocmError("QuantizedKvSdpa expects [Q, K_new, V_new]")
        q, k_new, v_new = (_as_device(t, stream) for t in inputs)
        b, kh, s_new, d = k_new.shape
        if self.k is None:
            self.k = KiviCache(KIVI_RUNNING_CHANNEL, 8, 0, b, kh, d)
            self.v = KiviCache(KIVI_PER_TOKEN, 8, 0, b, kh, d)
        if out is None:
            out = DeviceTensor(q.shape, q.dtype)
        hq, sq = q.shape[1], q.shape[2]
        need = Workspace.bytes_for(b, hq, sq, d)
        if self._ws is None or self._ws.nbytes < need:
            self._ws = Workspace(b, hq, sq, d, stream)
        scale = float("nan") if self.scale is None else float(self.scale)
        call("trocm_quantized_kv_sdpa_eval", q.ptr, k_new.ptr, v_new.ptr, dtype_code(q.dtype), hq, s_new,
             self.k.handle, self.v.handle, out.ptr, scale, self._ws.ptr, self._ws.nbytes, _sh(stream))
        return out

    def freeze(self) -> "QuantizedKvSdpaState":
        f = QuantizedKvSdpaState(self.scale)
        if self.k is not None:
            f.k, f.v = self.k.clone(), self.v.clone()
        return f

    unfreeze = freeze


def quant_dequant(x, bits: int, by_row: bool, stream=None) -> np.ndarray:
    """kv_quant.rs:73-98 for a [rows, cols] f32 matrix at 4 or 8 bits: one group per row (Values) or per
    column (Keys; run as one block-per-channel store over at most 32 rows, the size the cache op freezes)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    r, c = x.shape
    if by_row:
        cache = KiviCache(KIVI_PER_TOKEN, bits, 0, 1, 1, c)
        cache.append(x.reshape(1, 1, r, c), stream)
        return cache.dequantize(np.float32, stream).to_numpy(stream).reshape(r, c)
    if r > KEY_BLOCK:
        raise TractRocmError(f"per-channel quant_dequant takes at most {KEY_BLOCK} rows (one key block), got {r}")
    # per-column groups over r rows: pad the block to 32 rows by repeating the last row (min and max unchanged)
    pad = np.concatenate([x, np.repeat(x[-1:], KEY_BLOCK - r, axis=0)]) if r < KEY_BLOCK else x
    cache = KiviCache(KIVI_BLOCK_CHANNEL, bits, 0, 1, 1, c)
    cache.append(pad.reshape(1, 1, KEY_BLOCK, c), stream)
    return cache.dequantize(np.float32, stream).to_numpy(stream).reshape(KEY_BLOCK, c)[:r]
