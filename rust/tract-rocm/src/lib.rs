//! The `rocm` runtime: tract's dynamic KV-cache op and the Sdpa that reads it, on one MI355X (gfx950).
//!
//! Same plug-in shape as tract-cuda (cuda/src/lib.rs:18-59) and tract-metal (metal/src/lib.rs:24-56): a `Runtime`
//! registered by name, a `DeviceContext` behind tract-gpu's device tensors, and a translator that swaps the ops of
//! the path for device ops.  Everything on the device goes through the C ABI of libtract_rocm.so (`ffi`).
//!
//! Reachability needs two edits outside this crate: `"rocm"` in `GPU_RUNTIME_NAMES` (core/src/runtime.rs:221) and a
//! feature-gated `extern crate tract_rocm;` next to the cuda one in api/rs/src/lib.rs:4-5.
//!
//! Status: source only.  No Rust toolchain exists where this was written; the crate has not been compiled.

mod context;
pub mod ffi;
pub mod ops;
mod tensor;
mod transform;

use tract_core::internal::*;
use tract_core::transform::ModelTransform;

pub use context::{rocm_context, with_rocm_stream, RocmContext};
pub use tensor::{RocmBuffer, RocmTensor};
pub use transform::RocmTransform;

#[derive(Debug)]
struct RocmRuntime;

impl Runtime for RocmRuntime {
    fn name(&self) -> StaticName {
        "rocm".into()
    }

    /// OK when device 0 is a gfx950 part and the library could create its context.
    fn check(&self) -> TractResult<()> {
        ffi::check(unsafe { ffi::trocm_init(0) })
    }

    fn prepare_with_options(
        &self,
        mut model: TypedModel,
        options: &RunOptions,
    ) -> TractResult<Box<dyn Runnable>> {
        self.check()?;
        rocm_context()?; // installs the DeviceContext once per process (gpu/src/device.rs:129-137)
        // Device ops first, CPU codegen afterwards: model.optimize() turns a remaining Sdpa into FlashSdpaOp
        // (transformers/src/ops/sdpa.rs:377-409), so it must only see what stayed on the host.
        RocmTransform.transform(&mut model)?;
        model.optimize()?;

        let options = RunOptions { skip_order_opt_ram: true, ..options.clone() };
        let mut plan = TypedSimplePlan::build(model, &options)?;
        if let Some(hints) = options.memory_sizing_hints {
            let handler = tract_gpu::session_handler::DeviceSessionHandler::from_plan(&plan, &hints)
                .context("sizing the device arena (a symbol without a hint?)")?;
            plan = plan.with_session_handler(handler);
        }
        // Constants went to the device on this thread's stream; the threads that run the plan use their own.
        ffi::check(unsafe { ffi::trocm_device_sync() })?;
        Ok(Box::new(Arc::new(plan)))
    }
}

register_runtime!(RocmRuntime = RocmRuntime);
