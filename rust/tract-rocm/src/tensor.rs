//! Device allocations and the owned device tensor (contract: gpu/src/tensor/owned.rs:12-32, gpu/src/device.rs:120-125).
use std::os::raw::c_void;

use tract_core::internal::*;
use tract_core::tract_linalg::block_quant::{BlockQuantFact, BlockQuantStorage};
use tract_gpu::device::DeviceBuffer;
use tract_gpu::tensor::{DeviceTensor, OwnedDeviceTensor};
use tract_gpu::utils::{as_q40_tensor, check_strides_validity};

use crate::context::with_rocm_stream;
use crate::ffi;

/// `len` bytes of device memory.  An owning buffer frees them on drop; a borrowed one (`owned == false`) names
/// memory that belongs to something else that outlives it -- the planes of a KV cache held by an op state.
#[derive(Debug)]
pub struct RocmBuffer {
    ptr: *mut c_void,
    len: usize,
    owned: bool,
}

// The pointer is device memory; the library is re-entrant across threads with distinct streams.
unsafe impl Send for RocmBuffer {}
unsafe impl Sync for RocmBuffer {}

impl RocmBuffer {
    pub fn alloc(len: usize) -> TractResult<RocmBuffer> {
        let mut ptr = std::ptr::null_mut();
        ffi::check(unsafe { ffi::trocm_malloc(&mut ptr, len.max(1)) })?;
        Ok(RocmBuffer { ptr, len, owned: true })
    }
    /// # Safety
    /// `ptr..ptr + len` must stay valid device memory for as long as the buffer (and every tensor over it) lives.
    pub unsafe fn borrowed(ptr: *mut c_void, len: usize) -> RocmBuffer {
        RocmBuffer { ptr, len, owned: false }
    }
    pub fn len(&self) -> usize {
        self.len
    }
    pub fn is_empty(&self) -> bool {
        self.len == 0
    }
    pub fn ptr_mut(&self) -> *mut c_void {
        self.ptr
    }
}

impl Drop for RocmBuffer {
    fn drop(&mut self) {
        if self.owned && !self.ptr.is_null() {
            unsafe { ffi::trocm_free(self.ptr) };
        }
    }
}

impl DeviceBuffer for Arc<RocmBuffer> {
    fn ptr(&self) -> *const c_void {
        self.ptr
    }
}

#[derive(Clone)]
pub struct RocmTensor {
    buffer: Arc<RocmBuffer>,
    datum_type: DatumType,
    shape: TVec<usize>,
    strides: TVec<isize>,
    exotic_fact: Option<Box<dyn ExoticFact>>,
}

impl PartialEq for RocmTensor {
    fn eq(&self, other: &Self) -> bool {
        self.buffer.ptr == other.buffer.ptr
            && self.buffer.len == other.buffer.len
            && self.datum_type == other.datum_type
            && self.shape == other.shape
            && self.strides == other.strides
    }
}
impl Eq for RocmTensor {}

impl std::hash::Hash for RocmTensor {
    fn hash<H: std::hash::Hasher>(&self, state: &mut H) {
        (self.buffer.ptr as usize).hash(state);
        self.datum_type.hash(state);
        self.shape.hash(state);
    }
}

impl std::fmt::Debug for RocmTensor {
    fn fmt(&self, f: &mut std::fmt::Formatter<'_>) -> std::fmt::Result {
        write!(f, "RocmTensor({:?} {:?} strides {:?}, {} bytes", self.datum_type, self.shape, self.strides, self.buffer.len)?;
        if let Some(e) = &self.exotic_fact {
            write!(f, ", {e:?}")?;
        }
        write!(f, ")")
    }
}

fn upload(bytes: &[u8]) -> TractResult<Arc<RocmBuffer>> {
    let buffer = RocmBuffer::alloc(bytes.len())?;
    if !bytes.is_empty() {
        with_rocm_stream(|s| {
            ffi::check(unsafe { ffi::trocm_h2d(buffer.ptr, bytes.as_ptr() as _, bytes.len(), s.raw()) })?;
            // the host slice may be gone when the call returns
            s.synchronize()
        })?;
    }
    Ok(Arc::new(buffer))
}

impl RocmTensor {
    pub fn from_tensor(tensor: &Tensor) -> TractResult<Self> {
        // Q4_0 constants (block-quantised weights) travel as their canonical blocks with the fact beside them,
        // like cuda/src/tensor.rs:60-80; every other tensor as its plain bytes.
        if let Some(bqs) = as_q40_tensor(tensor) {
            let fact = BlockQuantFact::new(tract_core::dyn_clone::clone_box(bqs.format()), tensor.shape().into());
            Ok(RocmTensor {
                buffer: upload(bqs.value().as_bytes())?,
                datum_type: tensor.datum_type(),
                shape: tensor.shape().into(),
                strides: tensor.strides().into(),
                exotic_fact: Some(Box::new(fact)),
            })
        } else {
            Ok(RocmTensor {
                buffer: upload(tensor.as_bytes())?,
                datum_type: tensor.datum_type(),
                shape: tensor.shape().into(),
                strides: tensor.strides().into(),
                exotic_fact: None,
            })
        }
    }

    pub fn uninitialized_dt(shape: &[usize], dt: DatumType) -> TractResult<Self> {
        let bytes = shape.iter().product::<usize>() * dt.size_of();
        Ok(RocmTensor {
            buffer: Arc::new(RocmBuffer::alloc(bytes)?),
            datum_type: dt,
            shape: shape.into(),
            strides: Tensor::natural_strides(shape),
            exotic_fact: None,
        })
    }

    pub fn uninitialized_exotic(exotic_fact: Box<dyn ExoticFact>) -> TractResult<Self> {
        let Some(bqf) = exotic_fact.downcast_ref::<BlockQuantFact>() else {
            bail!("tract-rocm: no device storage for {exotic_fact:?}")
        };
        let len: usize = bqf.shape().iter().product();
        ensure!(len % bqf.format.block_len() == 0);
        let bytes = len / bqf.format.block_len() * bqf.format.block_bytes();
        Ok(RocmTensor {
            buffer: Arc::new(RocmBuffer::alloc(bytes)?),
            datum_type: f32::datum_type(),
            shape: tvec!(),
            strides: tvec!(),
            exotic_fact: Some(Box::new(bqf.clone())),
        })
    }

    /// A tensor over memory this crate does not own: the valid region of a KV cache, with the cache's pitch in
    /// its strides.
    ///
    /// # Safety
    /// See `RocmBuffer::borrowed`.
    pub unsafe fn view_of(ptr: *mut c_void, bytes: usize, dt: DatumType, shape: &[usize], strides: &[isize]) -> Self {
        RocmTensor {
            buffer: Arc::new(unsafe { RocmBuffer::borrowed(ptr, bytes) }),
            datum_type: dt,
            shape: shape.into(),
            strides: strides.into(),
            exotic_fact: None,
        }
    }

    fn download(&self, offset: usize, out: &mut [u8]) -> TractResult<()> {
        ensure!(offset + out.len() <= self.buffer.len);
        with_rocm_stream(|s| {
            let src = unsafe { (self.buffer.ptr as *const u8).add(offset) };
            ffi::check(unsafe { ffi::trocm_d2h(out.as_mut_ptr() as _, src as _, out.len(), s.raw()) })?;
            s.synchronize()
        })
    }
}

impl OwnedDeviceTensor for RocmTensor {
    fn datum_type(&self) -> DatumType {
        self.datum_type
    }
    fn shape(&self) -> &[usize] {
        &self.shape
    }
    fn strides(&self) -> &[isize] {
        &self.strides
    }

    fn reshaped(&self, shape: TVec<usize>) -> TractResult<DeviceTensor> {
        ensure!(self.len() == shape.iter().product::<usize>(), "reshape {:?} to {:?}", self.shape, shape);
        ensure!(self.strides == Tensor::natural_strides(&self.shape), "reshape of a strided device tensor");
        let strides = Tensor::natural_strides(&shape);
        Ok(DeviceTensor::Owned(Box::new(RocmTensor { shape, strides, ..self.clone() })))
    }

    fn restrided(&self, strides: TVec<isize>) -> TractResult<DeviceTensor> {
        check_strides_validity(self.shape.clone(), strides.clone())?;
        Ok(DeviceTensor::Owned(Box::new(RocmTensor { strides, ..self.clone() })))
    }

    fn exotic_fact(&self) -> Option<&dyn ExoticFact> {
        self.exotic_fact.as_deref()
    }

    fn get_bytes_slice(&self, offset: usize, len: usize) -> Vec<u8> {
        let mut out = vec![0u8; len];
        self.download(offset, &mut out).expect("device to host copy");
        out
    }

    fn device_buffer(&self) -> &dyn DeviceBuffer {
        &self.buffer
    }

    fn to_host(&self) -> TractResult<Arc<Tensor>> {
        if let Some(fact) = &self.exotic_fact {
            let bqf = fact.downcast_ref::<BlockQuantFact>().context("unknown exotic fact on a device tensor")?;
            let mut blob = unsafe { Blob::new_for_size_and_align(self.buffer.len, vector_size()) };
            self.download(0, blob.as_bytes_mut())?;
            let storage = BlockQuantStorage::new(bqf.format.clone(), bqf.m(), bqf.k(), Arc::new(blob))?;
            return Ok(Arc::new(storage.into_tensor_with_shape(self.datum_type, &self.shape)));
        }
        if self.strides == Tensor::natural_strides(&self.shape) {
            let mut t = unsafe { Tensor::uninitialized_dt(self.datum_type, &self.shape)? };
            self.download(0, t.as_bytes_mut())?;
            return Ok(Arc::new(t));
        }
        // a strided view (a cache's valid region): gather on the device first, then one dense copy
        let dense = RocmTensor::uninitialized_dt(&self.shape, self.datum_type)?;
        let src = DeviceTensor::Owned(Box::new(self.clone()));
        let dst = DeviceTensor::Owned(Box::new(dense.clone()));
        tract_gpu::device::get_context()?.copy_nd(&src, 0, &self.strides, &dst, 0, &self.shape, &dense.strides)?;
        dense.to_host()
    }
}
