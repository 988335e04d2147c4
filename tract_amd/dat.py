"""NNEF tensor files (``.dat``) for the tensors of the KV-cache path, over the library's host-side
header functions: the wire format of ``save_to`` / ``load_from`` for cache states
(nnef/src/tensors.rs:62-233 for plain tensors, :275-327 for block-quantised values)."""
from __future__ import annotations

import ctypes as C

import numpy as np

from ._lib import F16, F32, Q4_0, Q8_0, TractRocmError, call

LEGACY_Q4_PACKING, Q8_1_BLOCKS = 1, 2
_BLOCK_BYTES_ON_DISK = {Q4_0: 18, Q8_0: 36}


def write_tensor(a: np.ndarray) -> bytes:
    """write_tensor (tensors.rs:186-248) for an f32 / f16 array."""
    a = np.require(a, requirements="C")   # (ascontiguousarray would turn a rank-0 tensor into rank 1)
    item = {np.dtype(np.float32): F32, np.dtype(np.float16): F16}.get(a.dtype)
    if item is None:
        raise TractRocmError(f"Don't know how to serialize {a.dtype}")
    head = (C.c_uint8 * 128)()
    dims = (C.c_int64 * max(a.ndim, 1))(*a.shape)
    call("trocm_dat_header_write", head, item, a.ndim, dims, a.nbytes)
    return bytes(head) + a.tobytes()


def write_block_quant(fmt: int, blocks: np.ndarray, shape) -> bytes:
    """write_block_quant_value (tensors.rs:300-322): `blocks` are the canonical blocks of a value of
    logical `shape` (Q4_0: 18 bytes per 32 elements; Q8_0: 34, written as Q8_1 blocks of 36)."""
    blocks = np.ascontiguousarray(blocks).view(np.uint8).reshape(-1)
    n_elems = int(np.prod(shape, dtype=np.int64))
    if fmt == Q8_0:
        out = np.empty(n_elems // 32 * 36, np.uint8)
        if blocks.size != n_elems // 32 * 34:
            raise TractRocmError("block bytes do not match the shape")
        call("trocm_q8_0_to_q8_1", blocks.ctypes.data, out.ctypes.data, n_elems // 32)
        blocks = out
    head = (C.c_uint8 * 128)()
    dims = (C.c_int64 * len(shape))(*shape)
    call("trocm_dat_header_write", head, fmt, len(shape), dims, blocks.size)
    return bytes(head) + blocks.tobytes()


def read_tensor(data: bytes):
    """read_tensor (tensors.rs:62-185).  Returns (item, shape, payload): an f32 / f16 ndarray of `shape`,
    or for Q4_0 / Q8_0 the canonical blocks (uint8, Q8 already stripped of the Q8_1 sums) of a value
    of the rank-2 `shape` the file records."""
    if len(data) < 128:
        raise TractRocmError("truncated tensor file")
    buf = np.frombuffer(data, np.uint8)
    item, rank, nbytes, flags = C.c_int(), C.c_int(), C.c_size_t(), C.c_int()
    dims = (C.c_int64 * 8)()
    call("trocm_dat_header_read", buf.ctypes.data, C.byref(item), C.byref(rank), dims, C.byref(nbytes), C.byref(flags))
    shape = tuple(dims[i] for i in range(rank.value))
    if len(data) < 128 + nbytes.value:
        raise TractRocmError("truncated tensor file")
    payload = buf[128:128 + nbytes.value].copy()
    if item.value in (F32, F16):
        return item.value, shape, payload.view(np.float32 if item.value == F32 else np.float16).reshape(shape)
    if flags.value & LEGACY_Q4_PACKING:
        call("trocm_dat_q4_0_legacy_to_gguf", payload.ctypes.data, payload.size)
    if flags.value & Q8_1_BLOCKS:
        out = np.empty(payload.size // 36 * 34, np.uint8)
        call("trocm_q8_1_to_q8_0", payload.ctypes.data, out.ctypes.data, payload.size // 36)
        payload = out
    return item.value, shape, payload
