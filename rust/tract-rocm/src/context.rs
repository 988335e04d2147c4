//! `DeviceContext` (gpu/src/device.rs:13-35) over the C ABI, and one stream per host thread
//! (the arrangement of cuda/src/context.rs:28-43).
use std::cell::OnceCell;
use std::os::raw::c_void;
use std::sync::OnceLock;

use tract_core::internal::*;
use tract_gpu::device::DeviceContext;
use tract_gpu::tensor::{DeviceTensor, OwnedDeviceTensor};

use crate::ffi;
use crate::tensor::RocmTensor;

/// The process-wide context: created on first use, installed as tract-gpu's device context.
pub fn rocm_context() -> TractResult<&'static RocmContext> {
    static INSTANCE: OnceLock<RocmContext> = OnceLock::new();
    if let Some(c) = INSTANCE.get() {
        return Ok(c);
    }
    ffi::check(unsafe { ffi::trocm_init(0) })?;
    let mut cus = 0;
    let mut hbm = 0usize;
    let mut name = [0 as std::os::raw::c_char; 128];
    ffi::check(unsafe { ffi::trocm_device_info(&mut cus, &mut hbm, name.as_mut_ptr(), name.len()) })?;
    let name = unsafe { std::ffi::CStr::from_ptr(name.as_ptr()) }.to_string_lossy().into_owned();
    log::info!("tract-rocm: device 0 = {name:?}, {cus} compute units, {} MiB", hbm >> 20);
    let ctx = INSTANCE.get_or_init(|| RocmContext { compute_units: cus as usize, hbm_bytes: hbm });
    // A second prepare() finds the context already set; that is not an error for this runtime.
    let _ = tract_gpu::device::set_context(Box::new(ctx.clone()));
    Ok(ctx)
}

#[derive(Debug, Clone)]
pub struct RocmContext {
    pub compute_units: usize,
    pub hbm_bytes: usize,
}

/// A HIP stream owned by one host thread.  Launches are asynchronous and ordered by the stream; nothing in the
/// library uses the NULL stream on the caller's behalf.
pub struct RocmStream(*mut c_void);

impl RocmStream {
    fn new() -> TractResult<RocmStream> {
        let mut s = std::ptr::null_mut();
        ffi::check(unsafe { ffi::trocm_stream_create(&mut s) })?;
        Ok(RocmStream(s))
    }
    pub fn raw(&self) -> *mut c_void {
        self.0
    }
    pub fn synchronize(&self) -> TractResult<()> {
        ffi::check(unsafe { ffi::trocm_stream_sync(self.0) })
    }
}

impl Drop for RocmStream {
    fn drop(&mut self) {
        unsafe { ffi::trocm_stream_destroy(self.0) };
    }
}

thread_local! {
    static STREAM: OnceCell<RocmStream> = const { OnceCell::new() };
}

/// Runs `f` with the calling thread's stream (created on the thread's first use).
pub fn with_rocm_stream<R>(f: impl FnOnce(&RocmStream) -> TractResult<R>) -> TractResult<R> {
    STREAM.with(|cell| {
        if cell.get().is_none() {
            let _ = cell.set(RocmStream::new()?);
        }
        f(cell.get().unwrap())
    })
}

/// Base pointer of a device tensor's data: the buffer plus the view's offset inside an arena.
pub fn data_ptr(t: &DeviceTensor) -> *const c_void {
    unsafe { (t.device_buffer_ptr() as *const u8).add(t.buffer_offset::<usize>()) as *const c_void }
}

impl DeviceContext for RocmContext {
    fn tensor_to_device(&self, tensor: TValue) -> TractResult<Box<dyn OwnedDeviceTensor>> {
        ensure!(DeviceTensor::is_supported_dt(tensor.datum_type()), "no device tensors of {:?}", tensor.datum_type());
        Ok(Box::new(RocmTensor::from_tensor(tensor.view().tensor)?))
    }

    fn uninitialized_device_tensor(&self, shape: &[usize], dt: DatumType) -> TractResult<Box<dyn OwnedDeviceTensor>> {
        Ok(Box::new(RocmTensor::uninitialized_dt(shape, dt)?))
    }

    fn uninitialized_device_exotic_tensor(&self, exotic_fact: Box<dyn ExoticFact>) -> TractResult<Box<dyn OwnedDeviceTensor>> {
        Ok(Box::new(RocmTensor::uninitialized_exotic(exotic_fact)?))
    }

    fn synchronize(&self) -> TractResult<()> {
        with_rocm_stream(|s| s.synchronize())
    }

    /// Element strides, byte offsets: the convention of trocm_copy_nd (and of gpu/src/device.rs:95-113).
    fn copy_nd(
        &self,
        input: &DeviceTensor,
        input_offset: usize,
        input_strides: &[isize],
        output: &DeviceTensor,
        output_offset: usize,
        output_shape: &[usize],
        output_strides: &[isize],
    ) -> TractResult<()> {
        ensure!(input.datum_type().size_of() == output.datum_type().size_of(), "copy_nd between element sizes");
        ensure!(input_strides.len() == output_shape.len() && output_strides.len() == output_shape.len());
        ensure!(output_shape.len() <= 6, "copy_nd: rank {} (at most 6)", output_shape.len());
        let shape: TVec<i64> = output_shape.iter().map(|d| *d as i64).collect();
        let src_strides: TVec<i64> = input_strides.iter().map(|s| *s as i64).collect();
        let dst_strides: TVec<i64> = output_strides.iter().map(|s| *s as i64).collect();
        with_rocm_stream(|s| {
            ffi::check(unsafe {
                ffi::trocm_copy_nd(
                    data_ptr(output) as *mut c_void,
                    output_offset,
                    dst_strides.as_ptr(),
                    data_ptr(input),
                    input_offset,
                    src_strides.as_ptr(),
                    shape.as_ptr(),
                    shape.len() as _,
                    input.datum_type().size_of() as _,
                    s.raw(),
                )
            })
        })
    }
}
