//! `InPlaceKvSdpa` and `WindowKvSdpa` on the device (transformers/src/ops/inplace_kv_cache.rs:131-290,
//! window_kv_cache.rs:161-237): one stateful op, inputs `[Q, K_new, V_new]`, output Q-shaped.  The two caches
//! never leave the state; a decode step is ONE launch that stores the new token and attends over the cache.
//! With `rope` set the op has the inputs `[Q, K_new, V_new, Cos, Sin]` and stands for ApplyRope(Q), ApplyRope(K_new),
//! InPlaceKvSdpa (the translator folds the two rotations in, transform.rs): still one launch per decode step.
use std::os::raw::c_int;

use tract_core::internal::*;
use tract_core::ops::OpStateFreeze;
use tract_gpu::fact::DeviceTypedFactExt;
use tract_gpu::tensor::{DeviceTensorExt, IntoDevice};
use tract_transformers::ops::inplace_kv_cache::InPlaceKvSdpa;
use tract_transformers::ops::window_kv_cache::WindowKvSdpa;

use super::{bhsd, dt_code, scale_arg, strides4, Workspace};
use crate::context::{data_ptr, with_rocm_stream};
use crate::ffi;

/// An owned `trocm_kv_cache` handle together with the geometry it was created for.
#[derive(Debug)]
pub(crate) struct CacheHandle {
    pub raw: *mut ffi::trocm_kv_cache,
    pub fmt: c_int,
    pub dt: DatumType, // type of the tokens that are appended (and of a dense export)
    pub batch: i64,
    pub kv_heads: i64,
    pub head_dim: i64,
    pub window: Option<usize>,
}
unsafe impl Send for CacheHandle {}

impl CacheHandle {
    pub fn create(fmt: c_int, dt: DatumType, window: Option<usize>, batch: i64, kv_heads: i64, head_dim: i64) -> TractResult<Self> {
        let mut raw = std::ptr::null_mut();
        match window {
            Some(w) => ffi::check(unsafe { ffi::trocm_kv_cache_create_window(&mut raw, fmt, batch, kv_heads, head_dim, w as i64) })?,
            None => ffi::check(unsafe { ffi::trocm_kv_cache_create(&mut raw, fmt, batch, kv_heads, head_dim) })?,
        }
        Ok(CacheHandle { raw, fmt, dt, batch, kv_heads, head_dim, window })
    }
    pub fn len(&self) -> TractResult<usize> {
        let mut n = 0i64;
        ffi::check(unsafe { ffi::trocm_kv_cache_len(self.raw, &mut n) })?;
        Ok(n as usize)
    }
    pub fn try_clone(&self) -> TractResult<Self> {
        let mut raw = std::ptr::null_mut();
        with_rocm_stream(|s| ffi::check(unsafe { ffi::trocm_kv_cache_clone(self.raw, &mut raw, s.raw()) }))?;
        Ok(CacheHandle { raw, fmt: self.fmt, dt: self.dt, batch: self.batch, kv_heads: self.kv_heads, head_dim: self.head_dim, window: self.window })
    }
    /// The valid region on the host: `[B, H, len, D]` in the cache's element type, or, for a block-quantised
    /// cache, its canonical blocks as u8 `[B, H, len, D / 32 * block_bytes]` (what trocm_kv_export writes).
    pub fn to_host(&self) -> TractResult<Tensor> {
        let len = self.len()?;
        let mut row = 0usize;
        ffi::check(unsafe { ffi::trocm_kv_row_bytes(self.raw, &mut row) })?;
        let quantised = self.fmt == ffi::TROCM_Q8_0 || self.fmt == ffi::TROCM_Q4_0;
        let (dt, last) = if quantised { (DatumType::U8, row) } else { (self.dt, self.head_dim as usize) };
        let shape = [self.batch as usize, self.kv_heads as usize, len, last];
        let mut host = unsafe { Tensor::uninitialized_dt(dt, &shape)? };
        let staging = crate::tensor::RocmBuffer::alloc(host.as_bytes().len())?;
        with_rocm_stream(|s| {
            ffi::check(unsafe { ffi::trocm_kv_export(self.raw, staging.ptr_mut(), s.raw()) })?;
            ffi::check(unsafe { ffi::trocm_d2h(host.as_bytes_mut().as_mut_ptr() as _, staging.ptr_mut(), host.as_bytes().len(), s.raw()) })?;
            s.synchronize()
        })?;
        Ok(host)
    }
}

impl Drop for CacheHandle {
    fn drop(&mut self) {
        unsafe { ffi::trocm_kv_cache_destroy(self.raw) };
    }
}

/// Storage format of the caches: the dtype of K/V, or a block-quantised format chosen by the translator
/// (`TRACT_ROCM_KV_FORMAT` = f16 | q8_0 | q4_0, read in transform.rs).
#[derive(Debug, Clone, Copy, PartialEq, Eq, Hash)]
pub enum KvStorage {
    AsInput,
    Q8_0,
    Q4_0,
}

#[derive(Debug, Clone, PartialEq, Eq, Hash)]
pub struct RocmInPlaceKvSdpa {
    pub axis: usize,
    pub causal: bool,
    pub scale_bits: Option<u32>, // f32 bits: the op must be Eq + Hash
    pub window: Option<usize>,
    pub storage: KvStorage,
    /// Inputs 3 and 4 are Cos and Sin: Q and K_new are rotated (apply_rope.rs:169-176) before the append.
    pub rope: bool,
}

pub type RocmWindowKvSdpa = RocmInPlaceKvSdpa;

impl RocmInPlaceKvSdpa {
    pub fn from_inplace(op: &InPlaceKvSdpa, storage: KvStorage) -> Self {
        Self { axis: op.axis, causal: op.causal, scale_bits: op.scale.map(f32::to_bits), window: None, storage, rope: false }
    }
    /// The same op with ApplyRope on Q and K_new folded in (growing caches of any storage format).
    pub fn with_rope(mut self) -> Self {
        self.rope = true;
        self
    }
    pub fn from_window(op: &WindowKvSdpa, storage: KvStorage) -> Self {
        // the ring buffer is the mask: window_kv_cache.rs:212-237 attends over every token it still holds
        Self { axis: op.axis, causal: false, scale_bits: op.scale.map(f32::to_bits), window: Some(op.window), storage, rope: false }
    }
    fn scale(&self) -> Option<f32> {
        self.scale_bits.map(f32::from_bits)
    }
}

impl Op for RocmInPlaceKvSdpa {
    fn name(&self) -> StaticName {
        if self.window.is_some() {
            "RocmWindowKvSdpa".into()
        } else if self.rope {
            "RocmRopeInPlaceKvSdpa".into()
        } else {
            "RocmInPlaceKvSdpa".into()
        }
    }
    fn info(&self) -> TractResult<Vec<String>> {
        Ok(vec![format!(
            "axis={}, causal={}, scale={:?}, window={:?}, storage={:?}, rope={}",
            self.axis, self.causal, self.scale(), self.window, self.storage, self.rope
        )])
    }
    op_as_typed_op!();
}

impl EvalOp for RocmInPlaceKvSdpa {
    fn is_stateless(&self) -> bool {
        false
    }
    fn state(&self, _session: &TurnState, node_id: usize) -> TractResult<Option<Box<dyn OpState>>> {
        ensure!(self.axis == 2, "tract-rocm caches grow along axis 2 of [B, H, S, D], got axis {}", self.axis);
        ensure!(!self.rope || self.window.is_none(), "the rotation is folded into growing caches only");
        Ok(Some(Box::new(RocmInPlaceKvSdpaState { node_id, op: self.clone(), k: None, v: None, workspace: Workspace::default(), rot_scratch: None })))
    }
}

impl TypedOp for RocmInPlaceKvSdpa {
    fn output_facts(&self, inputs: &[&TypedFact]) -> TractResult<TVec<TypedFact>> {
        if self.rope {
            ensure!(inputs.len() == 5, "{} expects [Q, K_new, V_new, Cos, Sin]", self.name());
        } else {
            ensure!(inputs.len() == 3, "{} expects [Q, K_new, V_new]", self.name());
        }
        // Q's shape and dtype, as a device fact.  The caches are op state: nothing here is `state_owned`.
        tract_gpu::utils::facts_to_device_facts(inputs, |facts| Ok(tvec!(facts[0].without_value())))
            .with_context(|| format!("Error while computing facts for {:?}", self.name()))
    }
    as_op!();
}

#[derive(Debug)]
pub struct RocmInPlaceKvSdpaState {
    node_id: usize,
    op: RocmInPlaceKvSdpa,
    k: Option<CacheHandle>,
    v: Option<CacheHandle>,
    workspace: Workspace,
    /// `rope` only: where a call that has no fused kernel (several tokens, f32, one head per kv head) rotates Q and K_new
    rot_scratch: Option<crate::tensor::RocmBuffer>,
}

impl Clone for RocmInPlaceKvSdpaState {
    fn clone(&self) -> Self {
        let dup = |c: &Option<CacheHandle>| c.as_ref().map(|c| c.try_clone().expect("cloning a device KV cache"));
        Self { node_id: self.node_id, op: self.op.clone(), k: dup(&self.k), v: dup(&self.v), workspace: Workspace::default(), rot_scratch: None }
    }
}

impl RocmInPlaceKvSdpaState {
    fn ensure_caches(&mut self, kv_dt: DatumType, batch: i64, kv_heads: i64, head_dim: i64) -> TractResult<()> {
        if self.k.is_none() {
            let fmt = match self.op.storage {
                KvStorage::AsInput => dt_code(kv_dt)?,
                KvStorage::Q8_0 => ffi::TROCM_Q8_0,
                KvStorage::Q4_0 => ffi::TROCM_Q4_0,
            };
            self.k = Some(CacheHandle::create(fmt, kv_dt, self.op.window, batch, kv_heads, head_dim)?);
            self.v = Some(CacheHandle::create(fmt, kv_dt, self.op.window, batch, kv_heads, head_dim)?);
        }
        Ok(())
    }

    /// Rollback to `len` tokens (speculative decoding): metadata only, the tail is never read.
    pub fn truncate(&mut self, len: usize) -> TractResult<()> {
        for c in [&self.k, &self.v].into_iter().flatten() {
            ffi::check(unsafe { ffi::trocm_kv_cache_truncate(c.raw, len as i64) })?;
        }
        Ok(())
    }

    pub fn len(&self) -> TractResult<usize> {
        self.k.as_ref().map(|c| c.len()).unwrap_or(Ok(0))
    }
}

impl OpState for RocmInPlaceKvSdpaState {
    fn eval(&mut self, session: &mut TurnState, _op: &dyn Op, inputs: TVec<TValue>) -> TractResult<TVec<TValue>> {
        ensure!(inputs.len() == if self.op.rope { 5 } else { 3 }, "{}: wrong number of inputs", self.op.name());
        let (q, k_new, v_new) = (inputs[0].to_device_tensor()?, inputs[1].to_device_tensor()?, inputs[2].to_device_tensor()?);
        ensure!(k_new.datum_type() == q.datum_type() && v_new.datum_type() == q.datum_type(), "Q, K and V of one type");
        ensure!(k_new.shape() == v_new.shape() && k_new.strides() == v_new.strides(), "K_new and V_new of one layout");
        let [b, hq, sq, d] = bhsd(q.shape())?;
        let [_, hkv, n_new, _] = bhsd(k_new.shape())?;
        ensure!(sq == n_new, "{}: {sq} queries for {n_new} new tokens", self.op.name());
        ensure!(q.strides() == Tensor::natural_strides(q.shape()).as_slice(), "Q must be dense");
        self.ensure_caches(k_new.datum_type(), b, hkv, d)?;
        let out = tract_gpu::session_handler::make_tensor_for_node(session, self.node_id, q.datum_type(), q.shape())?;
        let kv_strides = strides4(k_new)?;
        let (kc, vc) = (self.k.as_ref().unwrap().raw, self.v.as_ref().unwrap().raw);
        let (scale, causal, window) = (scale_arg(self.op.scale()), self.op.causal as c_int, self.op.window);
        let dt = dt_code(q.datum_type())?;
        let workspace = &mut self.workspace;
        if self.op.rope {
            // Cos and Sin: [1 or B, 1, n_new, D] of Q's type, dense (what an exported decoder slices out of its tables)
            let (cos, sin) = (inputs[3].to_device_tensor()?, inputs[4].to_device_tensor()?);
            ensure!(cos.datum_type() == q.datum_type() && sin.datum_type() == q.datum_type(), "Cos and Sin of Q's type");
            ensure!(cos.shape() == sin.shape(), "Cos and Sin of one shape");
            let [cb, ch, cn, cd] = bhsd(cos.shape())?;
            ensure!(ch == 1 && cn == n_new && cd == d && (cb == 1 || cb == b), "Cos / Sin {:?} do not broadcast over the heads of Q {:?}", cos.shape(), q.shape());
            for t in [cos, sin, k_new] {
                ensure!(t.strides() == Tensor::natural_strides(t.shape()).as_slice(), "the rotating step takes dense operands");
            }
            let es = q.datum_type().size_of();
            let q_room = ((b * hq * n_new * d) as usize * es + 255) & !255;
            let need = q_room + (b * hkv * n_new * d) as usize * es;
            if self.rot_scratch.as_ref().map(|r| r.len() < need).unwrap_or(true) {
                // (an older, smaller scratch may still be read by launches in flight: drain the stream before it is dropped)
                if self.rot_scratch.is_some() {
                    with_rocm_stream(|s| s.synchronize())?;
                }
                self.rot_scratch = Some(crate::tensor::RocmBuffer::alloc(need)?);
            }
            let rot = self.rot_scratch.as_ref().unwrap();
            let batch_stride = if cb == 1 { 0 } else { n_new * d };
            with_rocm_stream(|s| {
                let (ws, ws_bytes) = workspace.for_shape(b, hq, sq, d, s.raw())?;
                ffi::check(unsafe {
                    ffi::trocm_inplace_kv_sdpa_eval_rope(
                        data_ptr(q), data_ptr(k_new), data_ptr(v_new), data_ptr(cos), data_ptr(sin), batch_stride, dt, hq, n_new, kc, vc,
                        data_ptr(&out) as *mut _, scale, causal, ws, ws_bytes, rot.ptr_mut(), rot.len(), s.raw(),
                    )
                })
            })?;
            return Ok(tvec!(out.into_tensor().into_tvalue()));
        }
        with_rocm_stream(|s| {
            let (ws, ws_bytes) = workspace.for_shape(b, hq, sq, d, s.raw())?;
            ffi::check(unsafe {
                if window.is_some() {
                    ffi::trocm_window_kv_sdpa_eval(
                        data_ptr(q), data_ptr(k_new), data_ptr(v_new), dt, hq, n_new, kv_strides.as_ptr(), kc, vc,
                        data_ptr(&out) as *mut _, scale, ws, ws_bytes, s.raw(),
                    )
                } else {
                    ffi::trocm_inplace_kv_sdpa_eval(
                        data_ptr(q), data_ptr(k_new), data_ptr(v_new), dt, hq, n_new, kv_strides.as_ptr(), kc, vc,
                        data_ptr(&out) as *mut _, scale, causal, ws, ws_bytes, s.raw(),
                    )
                }
            })
        })?;
        Ok(tvec!(out.into_tensor().into_tvalue()))
    }

    /// `[K_valid, V_valid]` on the host, K then V, nothing when empty (inplace_kv_cache.rs:222-228).  Quantised
    /// caches export their canonical blocks as a u8 tensor `[B, H, len, row_bytes]`.
    fn save_to(&self, states: &mut Vec<TValue>) -> TractResult<()> {
        let (Some(k), Some(v)) = (&self.k, &self.v) else { return Ok(()) };
        if k.len()? == 0 {
            return Ok(());
        }
        for c in [k, v] {
            states.push(c.to_host()?.into_tvalue());
        }
        Ok(())
    }

    /// Re-seeds both caches from a saved `[K, V]` pair; with no initialisers they stay empty
    /// (inplace_kv_cache.rs:232-245).
    fn load_from(&mut self, _: &mut TurnState, states: &mut dyn Iterator<Item = TValue>) -> TractResult<()> {
        let Some(k) = states.next() else { return Ok(()) };
        let v = states.next().context("InPlaceKvSdpa load_from: expected V state after K")?;
        ensure!(k.shape() == v.shape() && k.rank() == 4, "saved K and V of one rank-4 shape");
        self.k = None;
        self.v = None;
        let blocks = k.datum_type() == DatumType::U8; // the canonical blocks of a quantised cache, as save_to wrote them
        let [b, h, n, last] = bhsd(k.shape())?;
        if blocks {
            let block_bytes = match self.op.storage {
                KvStorage::Q8_0 => 34,
                KvStorage::Q4_0 => 18,
                KvStorage::AsInput => bail!("saved block-quantised caches need a quantised storage format"),
            };
            ensure!(last % block_bytes == 0, "rows of {last} bytes are not whole {block_bytes}-byte blocks");
            self.ensure_caches(DatumType::F16, b, h, last / block_bytes * 32)?;
        } else {
            self.ensure_caches(k.datum_type(), b, h, last)?;
        }
        for (cache, t) in [(self.k.as_ref().unwrap(), k), (self.v.as_ref().unwrap(), v)] {
            let dev = t.into_tensor().into_device()?;
            let strides = strides4(&dev)?;
            with_rocm_stream(|s| {
                ffi::check(unsafe {
                    if blocks {
                        ffi::trocm_kv_import_blocks(cache.raw, data_ptr(&dev), n, s.raw())
                    } else {
                        ffi::trocm_kv_append(cache.raw, data_ptr(&dev), dt_code(dev.datum_type())?, strides.as_ptr(), n, s.raw())
                    }
                })?;
                s.synchronize() // `dev` is dropped when this block ends
            })?;
        }
        Ok(())
    }
}

#[derive(Debug, Clone)]
struct FrozenRocmInPlaceKvSdpaState(RocmInPlaceKvSdpaState);
// A frozen state is only ever cloned or thawed; the handles are not touched concurrently.
unsafe impl Sync for FrozenRocmInPlaceKvSdpaState {}

impl OpStateFreeze for RocmInPlaceKvSdpaState {
    fn freeze(&self) -> Box<dyn FrozenOpState> {
        Box::new(FrozenRocmInPlaceKvSdpaState(self.clone())) // device-to-device copies of both caches
    }
}

impl FrozenOpState for FrozenRocmInPlaceKvSdpaState {
    fn unfreeze(&self) -> Box<dyn OpState> {
        Box::new(self.0.clone())
    }
}
