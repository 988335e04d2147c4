"""tract_amd — MI355X (gfx950) implementation of tract's KV-cache hot path.

The product is ``libtract_rocm.so`` (hand-written HIP behind the C ABI of
``include/tract_rocm.h``).  This package is the host-side mirror of the tract
operators on that path (``InPlaceKvCache``, ``InPlaceKvSdpa``, ``DynKeyValueCache``,
``Sdpa``, the Q4_0/Q8_0 ``BlockQuant`` formats) over that ABI, used by the tests and
the benchmark the way a ``tract-rocm`` crate would use it through FFI.
"""
from ._lib import F16, F32, Q4_0, Q8_0, TractRocmError  # noqa: F401
from .runtime import (DeviceTensor, Event, RocmRuntime, Stream, Workspace, runtime_for_name,  # noqa: F401
                      synchronize)
from .ops import (ApplyRope, BlockQuant, Cast, GgmlGemm, Q40Weights, RotateHalf, DynKeyValueCache, DynKeyValueCacheState, InPlaceKvCache, KvPool,  # noqa: F401
                  InPlaceKvSdpa, InPlaceKvSdpaState, Sdpa, StreamedSdpaOp, WindowKvCache, WindowKvSdpa, WindowKvSdpaState, Q4_0_FORMAT, Q8_0_FORMAT, inplace_kv_sdpa_eval_ragged, inplace_kv_sdpa_eval_ragged_rope,
                  sdpa_decode_ragged)
from .kivi import (KiviCache, QuantizedDynKeyValueCache, QuantizedDynKvCacheState, QuantizedKvSdpa,  # noqa: F401
                   QuantizedKvSdpaState, KIVI_BLOCK_CHANNEL, KIVI_PER_TOKEN, KIVI_RUNNING_CHANNEL)
