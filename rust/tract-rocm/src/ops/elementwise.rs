//! The ops either side of attention that keep a decoder layer on the device: `Cast` f32 <-> f16
//! (cuda/src/kernels/array/cast.rs:21-47), `ApplyRope` and `RotateHalf` (transformers/src/ops/apply_rope.rs:58-76,
//! :169-176).  Stateless: one launch each.
use tract_core::internal::*;
use tract_gpu::tensor::{DeviceTensor, DeviceTensorExt};

use super::dt_code;
use crate::context::{data_ptr, with_rocm_stream};
use crate::ffi;

fn strides_i64(t: &DeviceTensor) -> TVec<i64> {
    t.strides().iter().map(|s| *s as i64).collect()
}

fn shape_i64(t: &DeviceTensor) -> TVec<i64> {
    t.shape().iter().map(|d| *d as i64).collect()
}

/// Strides of `small` read at `big`'s rank, 0 on the axes along which it is broadcast (what
/// compute_broadcast_strides gives, cuda/src/kernels/nn/apply_rope.rs:75-81).
fn broadcast_strides(small: &DeviceTensor, big: &DeviceTensor) -> TractResult<TVec<i64>> {
    let lead = big.rank().checked_sub(small.rank()).context("cos / sin of a higher rank than the input")?;
    let mut out: TVec<i64> = tvec!(0; big.rank());
    for (ax, (dim, stride)) in small.shape().iter().zip(small.strides()).enumerate() {
        ensure!(*dim == 1 || *dim == big.shape()[lead + ax], "cos / sin {:?} against {:?}", small.shape(), big.shape());
        out[lead + ax] = if *dim == 1 { 0 } else { *stride as i64 };
    }
    Ok(out)
}

macro_rules! stateless_device_op {
    ($ty:ident, $name:literal) => {
        impl Op for $ty {
            fn name(&self) -> StaticName {
                $name.into()
            }
            op_as_typed_op!();
        }
        impl EvalOp for $ty {
            fn is_stateless(&self) -> bool {
                true
            }
            fn eval_with_session(&self, node_id: usize, session: &TurnState, inputs: TVec<TValue>) -> TractResult<TVec<TValue>> {
                self.run(node_id, session, inputs)
            }
        }
    };
}

// ---- Cast -----------------------------------------------------------------------------------------------

#[derive(Debug, Clone, PartialEq, Eq, Hash)]
pub struct RocmCast {
    pub to: DatumType,
}

impl RocmCast {
    pub fn new(to: DatumType) -> Option<Self> {
        matches!(to, DatumType::F32 | DatumType::F16).then_some(Self { to })
    }
    fn run(&self, node_id: usize, session: &TurnState, inputs: TVec<TValue>) -> TractResult<TVec<TValue>> {
        let x = inputs[0].to_device_tensor()?;
        ensure!(x.strides() == Tensor::natural_strides(x.shape()).as_slice(), "cast of a dense tensor");
        let out = tract_gpu::session_handler::make_tensor_for_node(session, node_id, self.to, x.shape())?;
        with_rocm_stream(|s| {
            ffi::check(unsafe { ffi::trocm_cast(data_ptr(x), dt_code(x.datum_type())?, data_ptr(&out) as *mut _, dt_code(self.to)?, x.len(), s.raw()) })
        })?;
        Ok(tvec!(out.into_tensor().into_tvalue()))
    }
}
stateless_device_op!(RocmCast, "RocmCast");

impl TypedOp for RocmCast {
    fn output_facts(&self, inputs: &[&TypedFact]) -> TractResult<TVec<TypedFact>> {
        tract_gpu::utils::facts_to_device_facts(inputs, |facts| Ok(tvec!(self.to.fact(facts[0].shape.clone()))))
            .with_context(|| format!("Error while computing facts for {:?}", self.name()))
    }
    as_op!();
}

// ---- RotateHalf / ApplyRope ---------------------------------------------------------------------------------

#[derive(Debug, Clone, PartialEq, Eq, Hash)]
pub struct RocmRotateHalf;

impl RocmRotateHalf {
    fn run(&self, node_id: usize, session: &TurnState, inputs: TVec<TValue>) -> TractResult<TVec<TValue>> {
        let x = inputs[0].to_device_tensor()?;
        let out = tract_gpu::session_handler::make_tensor_for_node(session, node_id, x.datum_type(), x.shape())?;
        let (shape, xs, os) = (shape_i64(x), strides_i64(x), strides_i64(&out));
        with_rocm_stream(|s| {
            ffi::check(unsafe {
                ffi::trocm_rotate_half(data_ptr(x), data_ptr(&out) as *mut _, dt_code(x.datum_type())?, x.rank() as _, shape.as_ptr(), xs.as_ptr(), os.as_ptr(), s.raw())
            })
        })?;
        Ok(tvec!(out.into_tensor().into_tvalue()))
    }
}
stateless_device_op!(RocmRotateHalf, "RocmRotateHalf");

impl TypedOp for RocmRotateHalf {
    fn output_facts(&self, inputs: &[&TypedFact]) -> TractResult<TVec<TypedFact>> {
        tract_gpu::utils::facts_to_device_facts(inputs, |facts| Ok(tvec!(facts[0].without_value())))
            .with_context(|| format!("Error while computing facts for {:?}", self.name()))
    }
    as_op!();
}

#[derive(Debug, Clone, PartialEq, Eq, Hash)]
pub struct RocmApplyRope;

impl RocmApplyRope {
    fn run(&self, node_id: usize, session: &TurnState, inputs: TVec<TValue>) -> TractResult<TVec<TValue>> {
        ensure!(inputs.len() == 3, "ApplyRope expects [input, cos, sin]");
        let (x, cos, sin) = (inputs[0].to_device_tensor()?, inputs[1].to_device_tensor()?, inputs[2].to_device_tensor()?);
        ensure!(cos.shape() == sin.shape() && cos.strides() == sin.strides(), "cos and sin of one layout");
        ensure!(cos.datum_type() == x.datum_type() && sin.datum_type() == x.datum_type());
        let out = tract_gpu::session_handler::make_tensor_for_node(session, node_id, x.datum_type(), x.shape())?;
        let (shape, xs, os) = (shape_i64(x), strides_i64(x), strides_i64(&out));
        let cs = broadcast_strides(cos, x)?;
        with_rocm_stream(|s| {
            ffi::check(unsafe {
                ffi::trocm_apply_rope(
                    data_ptr(x), data_ptr(cos), data_ptr(sin), data_ptr(&out) as *mut _, dt_code(x.datum_type())?, x.rank() as _,
                    shape.as_ptr(), xs.as_ptr(), cs.as_ptr(), os.as_ptr(), s.raw(),
                )
            })
        })?;
        Ok(tvec!(out.into_tensor().into_tvalue()))
    }
}
stateless_device_op!(RocmApplyRope, "RocmApplyRope");

impl TypedOp for RocmApplyRope {
    fn output_facts(&self, inputs: &[&TypedFact]) -> TractResult<TVec<TypedFact>> {
        tract_gpu::utils::facts_to_device_facts(inputs, |facts| Ok(tvec!(facts[0].without_value())))
            .with_context(|| format!("Error while computing facts for {:?}", self.name()))
    }
    as_op!();
}
