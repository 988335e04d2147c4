//! `GgmlGemm` with Q4_0 weights on the device (cuda/src/kernels/matmul/mod.rs:575-627): activations `[.., m, k]` of f32
//! or f16 times a constant weight matrix `[n, k]` (or `[batch, n, k]`) kept as Q4_0 blocks along k.  The weights are
//! handed to the library once, when the model is translated (`trocm_q4_0_weights_create` re-lays the canonical 18-byte
//! blocks out as a code plane and a scale plane); every `eval` is one `trocm_q4_0_matvec`, which picks the kernel by the
//! number of activation rows (vector ALUs up to 3 rows, the matrix cores from 4 rows on, a matrix-matrix kernel above
//! 16).  Unlike the reference's kernel, which quantises the activations to Q8_1 first (`CudaGgmlQuantQ81`,
//! cuda/src/transform.rs:262-267), this one multiplies them as they are: the product with the dequantised weights, the
//! definition the reference's own test holds its kernel to (mod.rs:864-890).
use std::sync::Arc;

use tract_core::internal::*;
use tract_core::tract_linalg::block_quant::{BlockQuantStorage, Q4_0};
use tract_gpu::tensor::DeviceTensorExt;

use super::dt_code;
use crate::context::{data_ptr, with_rocm_stream};
use crate::ffi;
use crate::tensor::RocmBuffer;

/// The library's copy of a Q4_0 weight matrix.
pub struct Q40DeviceWeights {
    raw: *mut ffi::trocm_q4_weights,
    pub batch: usize,
    pub n: usize,
    pub k: usize,
}
unsafe impl Send for Q40DeviceWeights {}
unsafe impl Sync for Q40DeviceWeights {} // read-only after creation

impl Q40DeviceWeights {
    /// From a constant tensor whose storage is `BlockQuantStorage` in Q4_0 and whose shape is `[n, k]` or `[batch, n, k]`.
    pub fn from_konst(weights: &Tensor) -> TractResult<Arc<Self>> {
        let storage = weights
            .storage_as::<BlockQuantStorage>()
            .filter(|s| s.format().dyn_eq(&Q4_0))
            .context("Q4_0 block-quantised weights expected")?;
        let shape = weights.shape();
        ensure!(shape.len() == 2 || shape.len() == 3, "Q4_0 weights of rank 2 or 3, got {shape:?}");
        let (batch, n, k) = if shape.len() == 2 { (1, shape[0], shape[1]) } else { (shape[0], shape[1], shape[2]) };
        ensure!(k % 32 == 0, "Q4_0 rows of k = {k}: not whole blocks");
        let blocks = storage.value();
        ensure!(blocks.len() == batch * n * (k / 32) * 18, "{} bytes of blocks for {batch} x {n} x {k}", blocks.len());
        let staging = RocmBuffer::alloc(blocks.len())?;
        let mut raw = std::ptr::null_mut();
        with_rocm_stream(|s| {
            ffi::check(unsafe { ffi::trocm_h2d(staging.ptr_mut(), blocks.as_ptr() as *const _, blocks.len(), s.raw()) })?;
            ffi::check(unsafe { ffi::trocm_q4_0_weights_create(&mut raw, staging.ptr_mut(), batch as i64, n as i64, k as i64, s.raw()) })?;
            s.synchronize() // `staging` is dropped when this block ends
        })?;
        Ok(Arc::new(Q40DeviceWeights { raw, batch, n, k }))
    }
}

impl Drop for Q40DeviceWeights {
    fn drop(&mut self) {
        unsafe { ffi::trocm_q4_0_weights_destroy(self.raw) };
    }
}

impl std::fmt::Debug for Q40DeviceWeights {
    fn fmt(&self, f: &mut std::fmt::Formatter<'_>) -> std::fmt::Result {
        write!(f, "Q40DeviceWeights({} x {} x {})", self.batch, self.n, self.k)
    }
}

#[derive(Debug, Clone)]
pub struct RocmQ40Gemm {
    pub weights: Arc<Q40DeviceWeights>,
}

// Two ops are the same op when they share their device weights.
impl PartialEq for RocmQ40Gemm {
    fn eq(&self, other: &Self) -> bool {
        Arc::ptr_eq(&self.weights, &other.weights)
    }
}
impl Eq for RocmQ40Gemm {}
impl std::hash::Hash for RocmQ40Gemm {
    fn hash<H: std::hash::Hasher>(&self, state: &mut H) {
        (Arc::as_ptr(&self.weights) as usize).hash(state)
    }
}

impl RocmQ40Gemm {
    /// `[.., m, k]` -> (act_batch, m): every leading axis is a batch of the activations.
    fn rows(&self, shape: &[usize]) -> TractResult<(usize, usize)> {
        ensure!(shape.len() >= 2, "activations of rank >= 2, got {shape:?}");
        ensure!(shape[shape.len() - 1] == self.weights.k, "activations {shape:?} against weights of k = {}", self.weights.k);
        let act_batch: usize = shape[..shape.len() - 2].iter().product();
        ensure!(act_batch % self.weights.batch == 0, "{act_batch} activation batches over {} weight matrices", self.weights.batch);
        Ok((act_batch, shape[shape.len() - 2]))
    }

    fn output_shape<D: DimLike>(&self, act: &[D]) -> TVec<D> {
        let mut out: TVec<D> = act.iter().cloned().collect();
        let last = out.len() - 1;
        out[last] = D::from(self.weights.n);
        out
    }
}

impl Op for RocmQ40Gemm {
    fn name(&self) -> StaticName {
        "RocmQ40Gemm".into()
    }
    fn info(&self) -> TractResult<Vec<String>> {
        Ok(vec![format!("{:?}", self.weights)])
    }
    op_as_typed_op!();
}

impl EvalOp for RocmQ40Gemm {
    fn is_stateless(&self) -> bool {
        true
    }
    fn eval_with_session(&self, node_id: usize, session: &TurnState, inputs: TVec<TValue>) -> TractResult<TVec<TValue>> {
        ensure!(inputs.len() == 1, "RocmQ40Gemm expects the activations (the weights live in the op)");
        let act = inputs[0].to_device_tensor()?;
        ensure!(act.strides() == Tensor::natural_strides(act.shape()).as_slice(), "activations must be dense");
        let (act_batch, m) = self.rows(act.shape())?;
        let out_shape = self.output_shape(act.shape());
        let out = tract_gpu::session_handler::make_tensor_for_node(session, node_id, act.datum_type(), &out_shape)?;
        let dt = dt_code(act.datum_type())?;
        with_rocm_stream(|s| {
            ffi::check(unsafe {
                ffi::trocm_q4_0_matvec(self.weights.raw, data_ptr(act), dt, act_batch as i64, m as i64, data_ptr(&out) as *mut _, s.raw())
            })
        })?;
        Ok(tvec!(out.into_tensor().into_tvalue()))
    }
}

impl TypedOp for RocmQ40Gemm {
    fn output_facts(&self, inputs: &[&TypedFact]) -> TractResult<TVec<TypedFact>> {
        ensure!(inputs.len() == 1, "RocmQ40Gemm expects the activations");
        tract_gpu::utils::facts_to_device_facts(inputs, |facts| {
            let act = facts[0];
            ensure!(matches!(act.datum_type, DatumType::F32 | DatumType::F16), "f32 or f16 activations");
            ensure!(act.rank() >= 2 && act.shape[act.rank() - 1] == self.weights.k.to_dim(), "activations {:?} against k = {}", act.shape, self.weights.k);
            let shape = self.output_shape(&act.shape.to_tvec());
            Ok(tvec!(act.datum_type.fact(shape)))
        })
        .with_context(|| format!("Error while computing facts for {:?}", self.name()))
    }
    as_op!();
}
