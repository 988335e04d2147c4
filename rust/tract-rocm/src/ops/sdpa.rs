//! `Sdpa` on the device (transformers/src/ops/sdpa.rs:83-89, :296-356): stateless, inputs `[Q, K, V]` or
//! `[Q, K, V, mask]`.  K and V arrive at `kv_heads` (the reference's `fuse_kv_cache_broadcast_rule`, sdpa.rs:414-502,
//! has removed the repeat-interleave) and may be strided views of a cache (`RocmDynKVCache`).
//!
//! Unlike the reference's CUDA translator (cuda/src/transform.rs:301-409) nothing is cast to f16 here: f32
//! operands run on f32 kernels.  A translator that wants the MFMA prefill for f32 prompts wires `RocmCast`s
//! around this op itself.
use std::os::raw::c_int;

use tract_core::internal::*;
use tract_gpu::tensor::DeviceTensorExt;
use tract_transformers::ops::sdpa::Sdpa;

use super::{bhsd, dt_code, scale_arg, strides4, Workspace};
use crate::context::{data_ptr, with_rocm_stream};
use crate::ffi;

#[derive(Debug, Clone, PartialEq, Eq, Hash)]
pub struct RocmSdpa {
    pub scale_bits: Option<u32>,
    pub is_causal: bool,
}

impl RocmSdpa {
    pub fn from_tract_transformers(op: &Sdpa) -> TractResult<Self> {
        let scale = op.scale.as_ref().map(|t| t.cast_to_scalar::<f32>()).transpose()?;
        Ok(Self { scale_bits: scale.map(f32::to_bits), is_causal: op.is_causal })
    }
}

impl Op for RocmSdpa {
    fn name(&self) -> StaticName {
        "RocmSdpa".into()
    }
    fn info(&self) -> TractResult<Vec<String>> {
        Ok(vec![format!("scale={:?}, causal={}", self.scale_bits.map(f32::from_bits), self.is_causal)])
    }
    op_as_typed_op!();
}

impl EvalOp for RocmSdpa {
    fn is_stateless(&self) -> bool {
        false // it owns a split-K workspace
    }
    fn state(&self, _session: &TurnState, node_id: usize) -> TractResult<Option<Box<dyn OpState>>> {
        Ok(Some(Box::new(RocmSdpaState { node_id, op: self.clone(), workspace: Workspace::default() })))
    }
}

impl TypedOp for RocmSdpa {
    fn output_facts(&self, inputs: &[&TypedFact]) -> TractResult<TVec<TypedFact>> {
        ensure!(inputs.len() == 3 || inputs.len() == 4, "Sdpa expects [Q, K, V] or [Q, K, V, mask]");
        ensure!(!(self.is_causal && inputs.len() == 4), "a causal Sdpa takes no mask input (sdpa.rs:297-299)");
        tract_gpu::utils::facts_to_device_facts(inputs, |facts| {
            // Q's shape with V's last dimension, Q's type (sdpa.rs:296-356)
            let (q, v) = (facts[0], facts[2]);
            let mut out = q.without_value();
            out.shape.set(q.rank() - 1, v.shape.dims()[v.rank() - 1].clone());
            Ok(tvec!(out))
        })
        .with_context(|| format!("Error while computing facts for {:?}", self.name()))
    }
    as_op!();
}

#[derive(Debug, Clone)]
struct RocmSdpaState {
    node_id: usize,
    op: RocmSdpa,
    workspace: Workspace,
}

impl OpState for RocmSdpaState {
    fn eval(&mut self, session: &mut TurnState, _op: &dyn Op, inputs: TVec<TValue>) -> TractResult<TVec<TValue>> {
        let (q, k, v) = (inputs[0].to_device_tensor()?, inputs[1].to_device_tensor()?, inputs[2].to_device_tensor()?);
        let mask = inputs.get(3).map(|m| m.to_device_tensor()).transpose()?;
        ensure!(k.datum_type() == q.datum_type() && v.datum_type() == q.datum_type(), "Q, K and V of one type");
        ensure!(k.shape() == v.shape() && k.strides() == v.strides(), "K and V of one layout");
        ensure!(q.strides() == Tensor::natural_strides(q.shape()).as_slice(), "Q must be dense");
        let [b, hq, sq, d] = bhsd(q.shape())?;
        let [_, hkv, sk, _] = bhsd(k.shape())?;
        ensure!(hq % hkv == 0, "{hq} query heads over {hkv} kv heads");
        let (mask_ptr, mask_b, mask_h) = match mask {
            Some(m) => {
                ensure!(m.datum_type() == q.datum_type(), "mask of Q's type");
                ensure!(m.strides() == Tensor::natural_strides(m.shape()).as_slice(), "mask must be dense");
                let ms = m.shape();
                ensure!(ms.len() >= 2 && ms[ms.len() - 2] as i64 == sq && ms[ms.len() - 1] as i64 == sk, "mask {ms:?} for {sq} x {sk}");
                let lead: i64 = ms[..ms.len() - 2].iter().product::<usize>() as i64;
                let (mb, mh) = if lead == 1 { (1, 1) } else if lead == b { (b, 1) } else if lead == hq { (1, hq) } else { (b, hq) };
                ensure!(mb * mh == lead, "mask {ms:?} does not broadcast over [{b}, {hq}]");
                (data_ptr(m), mb, mh)
            }
            None => (std::ptr::null(), 1, 1),
        };
        let out = tract_gpu::session_handler::make_tensor_for_node(session, self.node_id, q.datum_type(), q.shape())?;
        let kv_strides = strides4(k)?;
        let (scale, causal) = (scale_arg(self.op.scale_bits.map(f32::from_bits)), self.op.is_causal as c_int);
        let dt = dt_code(q.datum_type())?;
        let workspace = &mut self.workspace;
        with_rocm_stream(|s| {
            let (ws, ws_bytes) = workspace.for_shape(b, hq, sq, d, s.raw())?;
            ffi::check(unsafe {
                ffi::trocm_sdpa(
                    data_ptr(q), data_ptr(k), data_ptr(v), mask_ptr, data_ptr(&out) as *mut _, dt, b, hq, hkv, sq, sk, d,
                    kv_strides.as_ptr(), mask_b, mask_h, scale, causal, ws, ws_bytes, s.raw(),
                )
            })
        })?;
        Ok(tvec!(out.into_tensor().into_tvalue()))
    }
}

impl tract_core::ops::OpStateFreeze for RocmSdpaState {
    fn freeze(&self) -> Box<dyn FrozenOpState> {
        Box::new(FrozenRocmSdpaState { node_id: self.node_id, op: self.op.clone() })
    }
}

#[derive(Debug, Clone)]
struct FrozenRocmSdpaState {
    node_id: usize,
    op: RocmSdpa,
}

impl FrozenOpState for FrozenRocmSdpaState {
    fn unfreeze(&self) -> Box<dyn OpState> {
        Box::new(RocmSdpaState { node_id: self.node_id, op: self.op.clone(), workspace: Workspace::default() })
    }
}
