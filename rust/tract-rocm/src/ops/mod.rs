//! Device ops of the KV-cache path.  Every one is a thin typed op whose `eval` is one call of the C ABI.
pub mod dyn_kv_cache;
pub mod elementwise;
pub mod inplace_kv_sdpa;
pub mod q40_gemm;
pub mod quant_kv;
pub mod sdpa;

use std::os::raw::{c_int, c_void};

use tract_core::internal::*;
use tract_gpu::tensor::DeviceTensor;

use crate::ffi;
use crate::tensor::RocmBuffer;

pub use dyn_kv_cache::RocmDynKVCache;
pub use elementwise::{RocmApplyRope, RocmCast, RocmRotateHalf};
pub use inplace_kv_sdpa::{RocmInPlaceKvSdpa, RocmWindowKvSdpa};
pub use q40_gemm::{Q40DeviceWeights, RocmQ40Gemm};
pub use quant_kv::{RocmQuantDynKVCache, RocmQuantizedKvSdpa};
pub use sdpa::RocmSdpa;

/// Element type code of the C ABI (`trocm_dtype`).
pub(crate) fn dt_code(dt: DatumType) -> TractResult<c_int> {
    match dt {
        DatumType::F32 => Ok(ffi::TROCM_F32),
        DatumType::F16 => Ok(ffi::TROCM_F16),
        other => bail!("tract-rocm: no kernel for {other:?} (f32 and f16 only)"),
    }
}

/// `[B, H, S, D]` of a rank-4 tensor, or `[1, H, S, D]` of a rank-3 one (a single sequence: sdpa.rs:296-356
/// admits both).
pub(crate) fn bhsd(shape: &[usize]) -> TractResult<[i64; 4]> {
    match shape {
        [b, h, s, d] => Ok([*b as i64, *h as i64, *s as i64, *d as i64]),
        [h, s, d] => Ok([1, *h as i64, *s as i64, *d as i64]),
        _ => bail!("tract-rocm: attention operands are rank 3 or 4, got {shape:?}"),
    }
}

/// Element strides of the `[B, H, S, D]` reading of `t`, for the `*_strides` arguments of the C ABI.
pub(crate) fn strides4(t: &DeviceTensor) -> TractResult<[i64; 4]> {
    let s = t.strides();
    match s.len() {
        4 => Ok([s[0] as i64, s[1] as i64, s[2] as i64, s[3] as i64]),
        3 => Ok([0, s[0] as i64, s[1] as i64, s[2] as i64]),
        r => bail!("tract-rocm: rank {r} attention operand"),
    }
}

/// The split-K workspace an attention op state owns: partial records and arrival counters.  It lives in the
/// state (the arena planner models node outputs only, gpu/src/memory/schema.rs:56-128) and grows on demand;
/// a workspace that is too small only costs speed, none at all is allowed.
#[derive(Debug, Default)]
pub(crate) struct Workspace {
    buffer: Option<Arc<RocmBuffer>>,
}

/// A cloned state gets a workspace of its own (allocated at its first call): two states must never share one,
/// calls that overlap in time would race on the arrival counters.
impl Clone for Workspace {
    fn clone(&self) -> Self {
        Workspace::default()
    }
}

impl Workspace {
    /// Workspace for `batch` sequences of `q_heads` heads and `q_len` queries: `(pointer, bytes)`.
    pub fn for_shape(&mut self, batch: i64, q_heads: i64, q_len: i64, head_dim: i64, stream: *mut c_void) -> TractResult<(*mut c_void, usize)> {
        let mut need = 0usize;
        ffi::check(unsafe { ffi::trocm_sdpa_workspace_bytes(batch, q_heads, q_len, head_dim, &mut need) })?;
        if self.buffer.as_ref().map(|b| b.len() < need).unwrap_or(true) {
            // The old workspace may still be read by launches in flight on this stream: it is dropped (and
            // freed) only after the stream has drained.
            if self.buffer.is_some() {
                ffi::check(unsafe { ffi::trocm_stream_sync(stream) })?;
            }
            let fresh = RocmBuffer::alloc(need)?;
            ffi::check(unsafe { ffi::trocm_sdpa_workspace_init(fresh.ptr_mut(), need, stream) })?;
            self.buffer = Some(Arc::new(fresh));
        }
        let b = self.buffer.as_ref().unwrap();
        Ok((b.ptr_mut(), b.len()))
    }
}

/// NaN asks the library for the default `1 / sqrt(head_dim)` (sdpa.rs:177-181).
pub(crate) fn scale_arg(scale: Option<f32>) -> f32 {
    scale.unwrap_or(f32::NAN)
}
