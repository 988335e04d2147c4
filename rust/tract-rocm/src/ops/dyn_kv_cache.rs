//! `DynKeyValueCache` on the device (transformers/src/ops/dyn_kv_cache.rs:158-224), for graphs in which the cache
//! was not fused into an `InPlaceKvSdpa`.  The reference's device op (gpu/src/ops/dyn_kv_cache.rs:58-113)
//! allocates a new tensor and copies the whole past every step; this one appends in place into a
//! capacity-doubling cache (`InPlaceKvCache::push`, inplace_kv_cache.rs:55-83) and hands the consumer a strided
//! *view* of the valid region `[B, H, len, D]` whose token-axis pitch is the cache's.
use tract_core::internal::*;
use tract_core::ops::OpStateFreeze;
use tract_gpu::fact::DeviceTypedFactExt;
use tract_gpu::tensor::{DeviceTensor, DeviceTensorExt, IntoDevice};
use tract_transformers::ops::dyn_kv_cache::{DynKeyValueCache, DynKeyValueCacheState};

use super::inplace_kv_sdpa::CacheHandle;
use super::{bhsd, dt_code, strides4};
use crate::context::{data_ptr, with_rocm_stream};
use crate::ffi;
use crate::tensor::RocmTensor;

#[derive(Clone, PartialEq, Eq)]
pub struct RocmDynKVCache {
    pub name: String,
    pub axis: usize,
    pub past_sequence_fact: TypedFact,
    pub input_sequence_fact: TypedFact,
}

impl RocmDynKVCache {
    pub fn from_tract_transformers(op: &DynKeyValueCache) -> Self {
        Self {
            name: op.name.clone(),
            axis: op.axis,
            past_sequence_fact: op.past_sequence_fact.clone(),
            input_sequence_fact: op.input_sequence_fact.clone(),
        }
    }
}

impl std::fmt::Debug for RocmDynKVCache {
    fn fmt(&self, f: &mut std::fmt::Formatter) -> std::fmt::Result {
        write!(f, "RocmDynKVCache({}, axis={})", self.name, self.axis)
    }
}

impl std::hash::Hash for RocmDynKVCache {
    fn hash<H: std::hash::Hasher>(&self, state: &mut H) {
        self.name.hash(state);
        self.axis.hash(state);
    }
}

impl Op for RocmDynKVCache {
    fn name(&self) -> StaticName {
        "RocmDynKVCache".into()
    }
    fn info(&self) -> TractResult<Vec<String>> {
        Ok(vec![format!("axis: {}, in-place append", self.axis)])
    }
    op_as_typed_op!();
}

impl EvalOp for RocmDynKVCache {
    fn is_stateless(&self) -> bool {
        false
    }
    fn state(&self, _session: &TurnState, _node_id: usize) -> TractResult<Option<Box<dyn OpState>>> {
        ensure!(self.axis == 2, "tract-rocm caches grow along axis 2 of [B, H, S, D], got axis {}", self.axis);
        Ok(Some(Box::new(RocmDynKVCacheState { name: self.name.clone(), past_sequence_fact: self.past_sequence_fact.clone(), cache: None })))
    }
}

impl TypedOp for RocmDynKVCache {
    fn output_facts(&self, inputs: &[&TypedFact]) -> TractResult<TVec<TypedFact>> {
        ensure!(inputs.len() == 1);
        let mut facts = tract_gpu::utils::facts_to_device_facts(inputs, |facts| {
            let mut fact = facts[0].without_value();
            fact.shape.set(
                self.axis,
                self.past_sequence_fact.shape.dims()[self.axis].clone() + self.input_sequence_fact.shape.dims()[self.axis].clone(),
            );
            Ok(tvec!(fact))
        })
        .with_context(|| format!("Error while computing facts for {:?}", self.name()))?;
        // the output is the op's own cache: keep it out of the arena (gpu/src/ops/dyn_kv_cache.rs:254)
        facts[0].as_device_fact_mut().unwrap().state_owned = true;
        Ok(facts)
    }
    as_op!();
}

#[derive(Debug)]
pub struct RocmDynKVCacheState {
    name: String,
    past_sequence_fact: TypedFact,
    cache: Option<CacheHandle>,
}

impl Clone for RocmDynKVCacheState {
    fn clone(&self) -> Self {
        Self {
            name: self.name.clone(),
            past_sequence_fact: self.past_sequence_fact.clone(),
            cache: self.cache.as_ref().map(|c| c.try_clone().expect("cloning a device KV cache")),
        }
    }
}

impl RocmDynKVCacheState {
    fn push(&mut self, new: &DeviceTensor) -> TractResult<()> {
        let [b, h, n, d] = bhsd(new.shape())?;
        if self.cache.is_none() {
            self.cache = Some(CacheHandle::create(dt_code(new.datum_type())?, new.datum_type(), None, b, h, d)?);
        }
        let strides = strides4(new)?;
        let cache = self.cache.as_ref().unwrap();
        with_rocm_stream(|s| {
            ffi::check(unsafe { ffi::trocm_kv_append(cache.raw, data_ptr(new), dt_code(new.datum_type())?, strides.as_ptr(), n, s.raw()) })
        })
    }

    /// The valid region as a device tensor over the cache's own memory.
    fn view(&self) -> TractResult<DeviceTensor> {
        let c = self.cache.as_ref().context("empty cache")?;
        let (mut data, mut scales, mut pitch) = (std::ptr::null_mut(), std::ptr::null_mut(), 0i64);
        ffi::check(unsafe { ffi::trocm_kv_cache_raw(c.raw, &mut data, &mut scales, &mut pitch) })?;
        let (b, h, d, len) = (c.batch as usize, c.kv_heads as usize, c.head_dim as usize, c.len()?);
        let pitch = pitch as usize;
        let shape = [b, h, len, d];
        let strides = [(h * pitch * d) as isize, (pitch * d) as isize, d as isize, 1];
        let bytes = b * h * pitch * d * c.dt.size_of();
        // The view is consumed by this run's Sdpa; the next append may move the planes (growth), which the
        // library orders behind the stream's pending work.
        Ok(DeviceTensor::Owned(Box::new(unsafe { RocmTensor::view_of(data, bytes, c.dt, &shape, &strides) })))
    }

    pub fn truncate(&mut self, len: usize) -> TractResult<()> {
        if let Some(c) = &self.cache {
            ffi::check(unsafe { ffi::trocm_kv_cache_truncate(c.raw, len as i64) })?;
        }
        Ok(())
    }
}

impl OpState for RocmDynKVCacheState {
    fn eval(&mut self, _session: &mut TurnState, _op: &dyn Op, inputs: TVec<TValue>) -> TractResult<TVec<TValue>> {
        ensure!(inputs.len() == 1);
        self.push(inputs[0].to_device_tensor()?)?;
        Ok(tvec!(self.view()?.into_tensor().into_tvalue()))
    }

    fn load_from(&mut self, state: &mut TurnState, states: &mut dyn Iterator<Item = TValue>) -> TractResult<()> {
        let kv = states.next().context("Not enough state initializers")?;
        DynKeyValueCacheState::resolve_symbols(state, self.past_sequence_fact.clone(), Some(kv.shape()))?;
        self.cache = None;
        if kv.shape()[2] > 0 {
            let dev = kv.into_tensor().into_device()?;
            self.push(&dev)?;
            with_rocm_stream(|s| s.synchronize())?; // `dev` goes away here
        }
        Ok(())
    }

    fn save_to(&self, states: &mut Vec<TValue>) -> TractResult<()> {
        match &self.cache {
            Some(c) => {
                states.push(c.to_host()?.into_tvalue());
                Ok(())
            }
            None => bail!("KV cache {} was never initialized", self.name),
        }
    }

    fn init_tensor_fact(&self) -> Option<(String, TypedFact)> {
        Some((self.name.clone(), self.past_sequence_fact.clone()))
    }

    fn has_init_tensor_fact(&self) -> bool {
        true
    }

    /// Binds the past-length symbol to the cache's current length (dyn_kv_cache.rs:78-106).
    fn resolve_symbols(&mut self, state: &mut TurnState) -> TractResult<()> {
        let shape: Option<TVec<usize>> = match &self.cache {
            Some(c) => Some(tvec!(c.batch as usize, c.kv_heads as usize, c.len()?, c.head_dim as usize)),
            None => None,
        };
        DynKeyValueCacheState::resolve_symbols(state, self.past_sequence_fact.clone(), shape.as_deref())
    }
}

#[derive(Debug, Clone)]
struct FrozenRocmDynKVCacheState(RocmDynKVCacheState);
unsafe impl Sync for FrozenRocmDynKVCacheState {}

impl OpStateFreeze for RocmDynKVCacheState {
    fn freeze(&self) -> Box<dyn FrozenOpState> {
        Box::new(FrozenRocmDynKVCacheState(self.clone()))
    }
}

impl FrozenOpState for FrozenRocmDynKVCacheState {
    fn unfreeze(&self) -> Box<dyn OpState> {
        Box::new(self.0.clone())
    }
}
