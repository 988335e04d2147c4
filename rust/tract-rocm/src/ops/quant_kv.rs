//! The reference's own storage-quantised caches on the device (KIVI: affine u8 / u4 codes with f32 `lo` / `scale`):
//! `QuantizedDynKeyValueCache` (transformers/src/ops/quant_dyn_kv_cache.rs:283-495: Values per token, Keys per
//! channel in frozen 32-token blocks, the first 4 tokens kept in f32) and `QuantizedKvSdpa`
//! (transformers/src/ops/kv_quant.rs:242-349: u8, running per-channel Keys).  Not to be confused with the Q8_0 /
//! Q4_0 block formats of `RocmInPlaceKvSdpa`'s `KvStorage`.
use tract_core::internal::*;
use tract_core::ops::OpStateFreeze;
use tract_gpu::tensor::DeviceTensorExt;
use tract_transformers::ops::kv_quant::QuantizedKvSdpa;
use tract_transformers::ops::quant_dyn_kv_cache::QuantizedDynKeyValueCache;

use super::{bhsd, dt_code, scale_arg, Workspace};
use crate::context::{data_ptr, with_rocm_stream};
use crate::ffi;

/// Tokens kept unquantised at the head of a `QuantizedDynKeyValueCache` store (SINK_TOKENS, quant_dyn_kv_cache.rs:92).
const SINK_TOKENS: i64 = 4;

#[derive(Debug)]
struct KiviHandle(*mut ffi::trocm_kivi_cache);
unsafe impl Send for KiviHandle {}

impl KiviHandle {
    fn create(layout: std::os::raw::c_int, bits: u32, sink: i64, batch: i64, heads: i64, head_dim: i64) -> TractResult<Self> {
        let mut h = std::ptr::null_mut();
        ffi::check(unsafe { ffi::trocm_kivi_cache_create(&mut h, layout, bits as _, sink, batch, heads, head_dim) })?;
        Ok(KiviHandle(h))
    }
    fn len(&self) -> TractResult<i64> {
        let mut n = 0;
        ffi::check(unsafe { ffi::trocm_kivi_cache_len(self.0, &mut n) })?;
        Ok(n)
    }
    fn try_clone(&self) -> TractResult<Self> {
        let mut h = std::ptr::null_mut();
        with_rocm_stream(|s| ffi::check(unsafe { ffi::trocm_kivi_cache_clone(self.0, &mut h, s.raw()) }))?;
        Ok(KiviHandle(h))
    }
}

impl Drop for KiviHandle {
    fn drop(&mut self) {
        unsafe { ffi::trocm_kivi_cache_destroy(self.0) };
    }
}

// ---- QuantizedDynKeyValueCache ------------------------------------------------------------------------------

#[derive(Clone, PartialEq, Eq)]
pub struct RocmQuantDynKVCache {
    pub name: String,
    pub axis: usize,
    pub bits: u32,
    pub per_channel: bool,
    pub past_sequence_fact: TypedFact,
    pub input_sequence_fact: TypedFact,
}

impl RocmQuantDynKVCache {
    pub fn from_tract_transformers(op: &QuantizedDynKeyValueCache) -> Self {
        Self {
            name: op.name.clone(),
            axis: op.axis,
            bits: op.bits,
            per_channel: op.per_channel,
            past_sequence_fact: op.past_sequence_fact.clone(),
            input_sequence_fact: op.input_sequence_fact.clone(),
        }
    }
}

impl std::fmt::Debug for RocmQuantDynKVCache {
    fn fmt(&self, f: &mut std::fmt::Formatter) -> std::fmt::Result {
        write!(f, "RocmQuantDynKVCache({}, {} bits, per_channel={})", self.name, self.bits, self.per_channel)
    }
}

impl std::hash::Hash for RocmQuantDynKVCache {
    fn hash<H: std::hash::Hasher>(&self, state: &mut H) {
        self.name.hash(state);
        self.bits.hash(state);
        self.per_channel.hash(state);
    }
}

impl Op for RocmQuantDynKVCache {
    fn name(&self) -> StaticName {
        "RocmQuantDynKVCache".into()
    }
    op_as_typed_op!();
}

impl EvalOp for RocmQuantDynKVCache {
    fn is_stateless(&self) -> bool {
        false
    }
    fn state(&self, _session: &TurnState, node_id: usize) -> TractResult<Option<Box<dyn OpState>>> {
        ensure!(self.axis == 2 && (self.bits == 4 || self.bits == 8));
        Ok(Some(Box::new(RocmQuantDynKVCacheState { node_id, op: self.clone(), store: None })))
    }
}

impl TypedOp for RocmQuantDynKVCache {
    fn output_facts(&self, inputs: &[&TypedFact]) -> TractResult<TVec<TypedFact>> {
        ensure!(inputs.len() == 1);
        tract_gpu::utils::facts_to_device_facts(inputs, |facts| {
            let mut fact = facts[0].without_value();
            fact.shape.set(
                self.axis,
                self.past_sequence_fact.shape.dims()[self.axis].clone() + self.input_sequence_fact.shape.dims()[self.axis].clone(),
            );
            Ok(tvec!(fact))
        })
        .with_context(|| format!("Error while computing facts for {:?}", self.name()))
    }
    as_op!();
}

#[derive(Debug)]
struct RocmQuantDynKVCacheState {
    node_id: usize,
    op: RocmQuantDynKVCache,
    store: Option<KiviHandle>,
}

impl Clone for RocmQuantDynKVCacheState {
    fn clone(&self) -> Self {
        Self { node_id: self.node_id, op: self.op.clone(), store: self.store.as_ref().map(|s| s.try_clone().expect("cloning a quantised store")) }
    }
}

impl OpState for RocmQuantDynKVCacheState {
    /// Appends the new tokens to the store and returns the whole cache dequantised, as the CPU op does every step
    /// (quant_dyn_kv_cache.rs:432-449, :483-494).
    fn eval(&mut self, session: &mut TurnState, _op: &dyn Op, inputs: TVec<TValue>) -> TractResult<TVec<TValue>> {
        let new = inputs[0].to_device_tensor()?;
        ensure!(new.strides() == Tensor::natural_strides(new.shape()).as_slice(), "dense [B, H, S, D] input");
        let [b, h, n, d] = bhsd(new.shape())?;
        if self.store.is_none() {
            let layout = if self.op.per_channel { ffi::TROCM_KIVI_BLOCK_CHANNEL } else { ffi::TROCM_KIVI_PER_TOKEN };
            self.store = Some(KiviHandle::create(layout, self.op.bits, SINK_TOKENS, b, h, d)?);
        }
        let store = self.store.as_ref().unwrap();
        let dt = dt_code(new.datum_type())?;
        with_rocm_stream(|s| ffi::check(unsafe { ffi::trocm_kivi_cache_append(store.0, data_ptr(new), dt, n, s.raw()) }))?;
        let len = store.len()? as usize;
        let out = tract_gpu::session_handler::make_tensor_for_node(session, self.node_id, new.datum_type(), &[b as usize, h as usize, len, d as usize])?;
        with_rocm_stream(|s| ffi::check(unsafe { ffi::trocm_kivi_cache_dequantize(store.0, data_ptr(&out) as *mut _, dt, s.raw()) }))?;
        Ok(tvec!(out.into_tensor().into_tvalue()))
    }

    fn init_tensor_fact(&self) -> Option<(String, TypedFact)> {
        Some((self.op.name.clone(), self.op.past_sequence_fact.clone()))
    }
    fn has_init_tensor_fact(&self) -> bool {
        true
    }
    fn resolve_symbols(&mut self, state: &mut TurnState) -> TractResult<()> {
        let len = self.store.as_ref().map(|s| s.len()).transpose()?;
        let shape: Option<TVec<usize>> = len.map(|l| {
            let mut dims: TVec<usize> = self.op.past_sequence_fact.shape.dims().iter().map(|d| d.to_usize().unwrap_or(0)).collect();
            dims[self.op.axis] = l as usize;
            dims
        });
        tract_transformers::ops::dyn_kv_cache::DynKeyValueCacheState::resolve_symbols(state, self.op.past_sequence_fact.clone(), shape.as_deref())
    }
}

#[derive(Debug, Clone)]
struct FrozenRocmQuantDynKVCacheState(RocmQuantDynKVCacheState);
unsafe impl Sync for FrozenRocmQuantDynKVCacheState {}

impl OpStateFreeze for RocmQuantDynKVCacheState {
    fn freeze(&self) -> Box<dyn FrozenOpState> {
        Box::new(FrozenRocmQuantDynKVCacheState(self.clone()))
    }
}
impl FrozenOpState for FrozenRocmQuantDynKVCacheState {
    fn unfreeze(&self) -> Box<dyn OpState> {
        Box::new(self.0.clone())
    }
}

// ---- QuantizedKvSdpa ----------------------------------------------------------------------------------------

#[derive(Debug, Clone, PartialEq, Eq, Hash)]
pub struct RocmQuantizedKvSdpa {
    pub axis: usize,
    pub scale_bits: Option<u32>,
}

impl RocmQuantizedKvSdpa {
    pub fn from_tract_transformers(op: &QuantizedKvSdpa) -> Self {
        Self { axis: op.axis, scale_bits: op.scale.map(f32::to_bits) }
    }
}

impl Op for RocmQuantizedKvSdpa {
    fn name(&self) -> StaticName {
        "RocmQuantizedKvSdpa".into()
    }
    op_as_typed_op!();
}

impl EvalOp for RocmQuantizedKvSdpa {
    fn is_stateless(&self) -> bool {
        false
    }
    fn state(&self, _session: &TurnState, node_id: usize) -> TractResult<Option<Box<dyn OpState>>> {
        Ok(Some(Box::new(RocmQuantizedKvSdpaState { node_id, op: self.clone(), k: None, v: None, workspace: Workspace::default() })))
    }
}

impl TypedOp for RocmQuantizedKvSdpa {
    fn output_facts(&self, inputs: &[&TypedFact]) -> TractResult<TVec<TypedFact>> {
        ensure!(inputs.len() == 3, "QuantizedKvSdpa expects [Q, K_new, V_new]");
        tract_gpu::utils::facts_to_device_facts(inputs, |facts| Ok(tvec!(facts[0].without_value())))
            .with_context(|| format!("Error while computing facts for {:?}", self.name()))
    }
    as_op!();
}

#[derive(Debug)]
struct RocmQuantizedKvSdpaState {
    node_id: usize,
    op: RocmQuantizedKvSdpa,
    k: Option<KiviHandle>,
    v: Option<KiviHandle>,
    workspace: Workspace,
}

impl Clone for RocmQuantizedKvSdpaState {
    fn clone(&self) -> Self {
        let dup = |c: &Option<KiviHandle>| c.as_ref().map(|c| c.try_clone().expect("cloning a quantised store"));
        Self { node_id: self.node_id, op: self.op.clone(), k: dup(&self.k), v: dup(&self.v), workspace: Workspace::default() }
    }
}

impl OpState for RocmQuantizedKvSdpaState {
    /// Keys into the running per-channel store, Values into the per-token store, then attention straight over the
    /// codes (one f16 query token, head_dim 128) or over dequantised copies (kv_quant.rs:296-349).
    fn eval(&mut self, session: &mut TurnState, _op: &dyn Op, inputs: TVec<TValue>) -> TractResult<TVec<TValue>> {
        ensure!(inputs.len() == 3, "QuantizedKvSdpa expects [Q, K_new, V_new]");
        let (q, k_new, v_new) = (inputs[0].to_device_tensor()?, inputs[1].to_device_tensor()?, inputs[2].to_device_tensor()?);
        let dense = |t: &tract_gpu::tensor::DeviceTensor| t.strides() == Tensor::natural_strides(t.shape()).as_slice();
        ensure!(dense(q) && dense(k_new) && dense(v_new), "dense [B, H, S, D] inputs");
        let [b, hq, _sq, d] = bhsd(q.shape())?;
        let [_, hkv, n_new, _] = bhsd(k_new.shape())?;
        if self.k.is_none() {
            self.k = Some(KiviHandle::create(ffi::TROCM_KIVI_RUNNING_CHANNEL, 8, 0, b, hkv, d)?);
            self.v = Some(KiviHandle::create(ffi::TROCM_KIVI_PER_TOKEN, 8, 0, b, hkv, d)?);
        }
        let out = tract_gpu::session_handler::make_tensor_for_node(session, self.node_id, q.datum_type(), q.shape())?;
        let (kc, vc) = (self.k.as_ref().unwrap().0, self.v.as_ref().unwrap().0);
        let scale = scale_arg(self.op.scale_bits.map(f32::from_bits));
        let dt = dt_code(q.datum_type())?;
        let workspace = &mut self.workspace;
        with_rocm_stream(|s| {
            let (ws, ws_bytes) = workspace.for_shape(b, hq, 1, d, s.raw())?;
            ffi::check(unsafe {
                ffi::trocm_quantized_kv_sdpa_eval(
                    data_ptr(q), data_ptr(k_new), data_ptr(v_new), dt, hq, n_new, kc, vc, data_ptr(&out) as *mut _, scale, ws,
                    ws_bytes, s.raw(),
                )
            })
        })?;
        Ok(tvec!(out.into_tensor().into_tvalue()))
    }
}

#[derive(Debug, Clone)]
struct FrozenRocmQuantizedKvSdpaState(RocmQuantizedKvSdpaState);
unsafe impl Sync for FrozenRocmQuantizedKvSdpaState {}

impl OpStateFreeze for RocmQuantizedKvSdpaState {
    fn freeze(&self) -> Box<dyn FrozenOpState> {
        Box::new(FrozenRocmQuantizedKvSdpaState(self.clone()))
    }
}
impl FrozenOpState for FrozenRocmQuantizedKvSdpaState {
    fn unfreeze(&self) -> Box<dyn OpState> {
        Box::new(self.0.clone())
    }
}
