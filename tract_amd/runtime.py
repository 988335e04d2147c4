"""Runtime plumbing over the C ABI: context, streams, device tensors, workspace.

Mirrors the pieces of tract's device layer that the KV-cache path touches:
``runtime_for_name`` (core/src/runtime.rs:223-250), ``DeviceContext`` (gpu/src/device.rs:13-35),
``DeviceTensor`` (gpu/src/tensor/mod.rs:21-24).
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib
from ._lib import F16, F32, TractRocmError, call

_DT = {np.dtype(np.float32): F32, np.dtype(np.float16): F16}


def dtype_code(dt) -> int:
    try:
        return _DT[np.dtype(dt)]
    except KeyError:
        raise TractRocmError(f"unsupported datum type {dt}: the rocm KV-cache path handles f32 and f16")


class RocmRuntime:
    """`Runtime` for name "rocm" (core/src/runtime.rs:23-34): `check()` tells whether the
    device is usable, `name()` returns the registry name."""

    _instance = None

    def __init__(self, device: int = 0):
        call("trocm_init", device)
        self.device = device
        cu, hbm = C.c_int(), C.c_size_t()
        name = C.create_string_buffer(256)
        call("trocm_device_info", C.byref(cu), C.byref(hbm), name, 256)
        self.compute_units, self.hbm_bytes, self.device_name = cu.value, hbm.value, name.value.decode()

    def name(self) -> str:
        return "rocm"

    def check(self) -> None:
        call("trocm_device_sync")


def runtime_for_name(name: str, device: int = 0) -> RocmRuntime:
    """core/src/runtime.rs:223-250: only "rocm" lives here; anything else is an error."""
    if name != "rocm":
        raise TractRocmError(f"Runtime {name!r} not found: this package registers only \"rocm\"")
    if RocmRuntime._instance is None:
        RocmRuntime._instance = RocmRuntime(device)
    return RocmRuntime._instance


def synchronize() -> None:
    call("trocm_device_sync")


class Stream:
    """One HIP stream (cuda/src/context.rs:37-43: one per host thread)."""

    def __init__(self):
        h = C.c_void_p()
        call("trocm_stream_create", C.byref(h))
        self.handle = h

    def synchronize(self):
        call("trocm_stream_sync", self.handle)

    def __del__(self):
        try:
            if self.handle:
                _lib.load().trocm_stream_destroy(self.handle)
                self.handle = None
        except Exception:
            pass


class Event:
    """A HIP event; `Event.elapsed_ms(a, b)` waits for b."""

    def __init__(self):
        h = C.c_void_p()
        call("trocm_event_create", C.byref(h))
        self.handle = h

    def record(self, stream=None):
        call("trocm_event_record", self.handle, _sh(stream))

    @staticmethod
    def elapsed_ms(start: "Event", stop: "Event") -> float:
        ms = C.c_float()
        call("trocm_event_elapsed_ms", start.handle, stop.handle, C.byref(ms))
        return ms.value

    def __del__(self):
        try:
            if self.handle:
                _lib.load().trocm_event_destroy(self.handle)
                self.handle = None
        except Exception:
            pass


def _sh(stream):
    return stream.handle if isinstance(stream, Stream) else stream


class DeviceTensor:
    """A dense device buffer with shape and numpy dtype (f32, f16 or u8 for block bytes)."""

    def __init__(self, shape, dtype, ptr=None, owner=None):
        self.shape = tuple(int(s) for s in shape)
        self.dtype = np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize
        self._owner = owner
        if ptr is None:
            p = C.c_void_p()
            call("trocm_malloc", C.byref(p), self.nbytes)
            self.ptr, self._owned = p, True
        else:
            self.ptr, self._owned = C.c_void_p(ptr) if not isinstance(ptr, C.c_void_p) else ptr, False

    @staticmethod
    def from_numpy(a: np.ndarray, stream=None) -> "DeviceTensor":
        a = np.ascontiguousarray(a)
        t = DeviceTensor(a.shape, a.dtype)
        if t.nbytes:
            call("trocm_h2d", t.ptr, a.ctypes.data_as(C.c_void_p), t.nbytes, _sh(stream))
            call("trocm_stream_sync", _sh(stream))  # the numpy temporary may die right after
        return t

    def to_numpy(self, stream=None) -> np.ndarray:
        out = np.empty(self.shape, dtype=self.dtype)
        if self.nbytes:
            call("trocm_d2h", out.ctypes.data_as(C.c_void_p), self.ptr, self.nbytes, _sh(stream))
            call("trocm_stream_sync", _sh(stream))
        return out

    def strides(self):
        """Element strides of the dense layout."""
        st, acc = [], 1
        for s in reversed(self.shape):
            st.append(acc)
            acc *= s
        return tuple(reversed(st))

    def __del__(self):
        try:
            if getattr(self, "_owned", False) and self.ptr:
                _lib.load().trocm_free(self.ptr)
                self.ptr = None
        except Exception:
            pass


class Workspace:
    """Persistent split-K scratch owned by an op state (the arena planner does not model
    scratch, gpu/src/memory/schema.rs:56-128)."""

    @staticmethod
    def bytes_for(batch: int, q_heads: int, q_len: int, head_dim: int) -> int:
        n = C.c_size_t()
        call("trocm_sdpa_workspace_bytes", batch, q_heads, q_len, head_dim, C.byref(n))
        return n.value

    def __init__(self, batch: int, q_heads: int, q_len: int, head_dim: int, stream=None):
        self.nbytes = Workspace.bytes_for(batch, q_heads, q_len, head_dim)
        self.buf = DeviceTensor((self.nbytes,), np.uint8)
        call("trocm_sdpa_workspace_init", self.buf.ptr, self.nbytes, _sh(stream))
        call("trocm_stream_sync", _sh(stream))

    @property
    def ptr(self):
        return self.buf.ptr
