//! The translator: which ops of a typed model go to the device (contract: core/src/model/translator.rs:7-63;
//! the reference's CUDA one is cuda/src/transform.rs:411-527).
//!
//! Only the KV-cache path and its neighbours move: the fused cache + attention op, bare `Sdpa`, bare
//! `DynKeyValueCache`, the reference's own quantised cache ops, RoPE, f32 <-> f16 casts, and the view / concat ops
//! tract-gpu implements on `copy_nd`.  Everything else stays a CPU op between `DeviceSync` nodes.
use std::collections::HashMap;

use tract_core::internal::*;
use tract_core::model::translator::Translate;
use tract_core::ops::cast::Cast;
use tract_core::ops::einsum::prefix_matmul::{rewrite_einsum_to_prefix_matmul, PrefixMatMul};
use tract_core::tract_linalg::block_quant::Q4_0;
use tract_core::transform::ModelTransform;
use tract_gpu::fact::DeviceTypedFactExt;
use tract_gpu::rewrite_rules::rewire_syncs::rewire_syncs;
use tract_gpu::sync::{sync_inputs_if_required, sync_model_outputs_if_required, DeviceSyncKind};
use tract_gpu::tensor::DeviceTensor;
use tract_transformers::ops::apply_rope::{ApplyRope, RotateHalf};
use tract_transformers::ops::dyn_kv_cache::DynKeyValueCache;
use tract_transformers::ops::inplace_kv_cache::{fuse_inplace_kv_sdpa_rule, InPlaceKvSdpa};
use tract_transformers::ops::kv_quant::QuantizedKvSdpa;
use tract_transformers::ops::quant_dyn_kv_cache::QuantizedDynKeyValueCache;
use tract_transformers::ops::sdpa::{fuse_kv_cache_broadcast_rule, Sdpa};
use tract_transformers::ops::window_kv_cache::WindowKvSdpa;

use crate::ops::inplace_kv_sdpa::KvStorage;
use crate::ops::*;

tract_core::declare_knob!(
    TRACT_ROCM_KV_FORMAT,
    String,
    String::new(),
    "Storage of the fused KV caches: empty = the dtype of K/V, q8_0 or q4_0 = quantise on append (32-element blocks, f16 scale)."
);
tract_core::declare_knob!(
    TRACT_ROCM_FORCE_CPU,
    String,
    String::new(),
    "Comma-separated node-name substrings kept on the CPU."
);

tract_core::declare_knob!(
    TRACT_ROCM_FUSE_ROPE,
    bool,
    true,
    "Fold ApplyRope on Q and K_new into the fused cache + attention op when both rotations share their Cos and Sin."
);

fn kv_storage() -> TractResult<KvStorage> {
    match TRACT_ROCM_KV_FORMAT.get().as_str() {
        "" | "f16" | "f32" => Ok(KvStorage::AsInput),
        "q8_0" => Ok(KvStorage::Q8_0),
        "q4_0" => Ok(KvStorage::Q4_0),
        other => bail!("TRACT_ROCM_KV_FORMAT={other}: expected q8_0 or q4_0"),
    }
}

#[derive(Debug, Default)]
pub struct RocmTransform;

impl ModelTransform for RocmTransform {
    fn name(&self) -> StaticName {
        "rocm-transform".into()
    }

    fn transform(&self, model: &mut TypedModel) -> TractResult<()> {
        self.transform_up_to_phase(model, usize::MAX)
    }
}

impl RocmTransform {
    /// Phase 0: the reference's own graph rewrites; 1: translation; 2: sync clean-up.  (The test runner stops
    /// early to look at intermediate graphs, as test-rt/test-cuda does.)
    pub fn transform_up_to_phase(&self, model: &mut TypedModel, stop_at_phase: usize) -> TractResult<()> {
        crate::context::rocm_context()?;
        // {DynKeyValueCache(K), DynKeyValueCache(V), Sdpa} -> InPlaceKvSdpa, after the repeat-interleave of GQA has
        // been folded away (transformers/src/ops/inplace_kv_cache.rs:336-350).  Models whose caches were already
        // rewritten (window, KIVI) arrive with those ops in place and are left alone.
        // matrix products as PrefixMatMul, the form in which the Q4_0-weight ones are recognised (cuda/src/transform.rs:92)
        rewrite_einsum_to_prefix_matmul(model, false)?;
        Rewriter::default()
            .with_rule_for("fuse-kv-broadcast", fuse_kv_cache_broadcast_rule)
            .with_rule_for("fuse-inplace-kv-sdpa", fuse_inplace_kv_sdpa_rule)
            .rewrite(&(), model)?;
        model.compact()?;
        if stop_at_phase == 0 {
            return Ok(());
        }
        *model = self.translate_model(model)?;
        model.compact()?; // (drops the rotations whose work moved into a fused op)
        if stop_at_phase == 1 {
            return Ok(());
        }
        rewire_syncs(model)
    }
}

/// `InPlaceKvSdpa` whose Q and K_new both come out of `ApplyRope` nodes that share their Cos and Sin (what an exported
/// decoder's attention block looks like, sdpa.rs:453-458): the outlets `[Q, K, V_new, Cos, Sin]` of the fused device op,
/// Q and K as they enter the rotations.  The rotations must feed nothing else, or they would run anyway.
fn rope_feeding(source: &TypedModel, node: &TypedNode) -> Option<TVec<OutletId>> {
    let op = node.op_as::<InPlaceKvSdpa>()?;
    if op.axis != 2 {
        return None;
    }
    let (rq, rk) = (source.node(node.inputs[0].node), source.node(node.inputs[1].node));
    if !rq.op_is::<ApplyRope>() || !rk.op_is::<ApplyRope>() || rq.id == rk.id {
        return None;
    }
    if rq.inputs[1] != rk.inputs[1] || rq.inputs[2] != rk.inputs[2] {
        return None;
    }
    if rq.outputs[0].successors.len() != 1 || rk.outputs[0].successors.len() != 1 {
        return None;
    }
    if source.outputs.iter().any(|o| o.node == rq.id || o.node == rk.id) {
        return None;
    }
    // Cos / Sin that broadcast over the heads: [1 or B, 1, S, D] against Q [B, H, S, D]
    let (qf, cf) = (source.outlet_fact(rq.inputs[0]).ok()?, source.outlet_fact(rq.inputs[1]).ok()?);
    if qf.rank() != 4 || cf.rank() != 4 || cf.shape[1] != 1.to_dim() || cf.shape[3] != qf.shape[3] || cf.shape[2] != qf.shape[2] {
        return None;
    }
    if cf.shape[0] != 1.to_dim() && cf.shape[0] != qf.shape[0] {
        return None;
    }
    Some(tvec!(rq.inputs[0], rk.inputs[0], node.inputs[2], rq.inputs[1], rq.inputs[2]))
}

/// The device op for `node`, or None when the node stays on the CPU.
fn try_make_rocm_op(source: &TypedModel, node: &TypedNode) -> TractResult<Option<Box<dyn TypedOp>>> {
    let facts = source.node_input_facts(node.id)?;
    let float = |f: &&TypedFact| matches!(f.datum_type, DatumType::F32 | DatumType::F16);
    if let Some(op) = node.op_as::<InPlaceKvSdpa>() {
        rule_if!(facts.iter().all(float) && op.axis == 2);
        return Ok(Some(Box::new(RocmInPlaceKvSdpa::from_inplace(op, kv_storage()?))));
    }
    if let Some(op) = node.op_as::<WindowKvSdpa>() {
        rule_if!(facts.iter().all(float) && op.axis == 2);
        return Ok(Some(Box::new(RocmWindowKvSdpa::from_window(op, kv_storage()?))));
    }
    if let Some(op) = node.op_as::<QuantizedKvSdpa>() {
        rule_if!(facts.iter().all(float) && op.axis == 2);
        return Ok(Some(Box::new(RocmQuantizedKvSdpa::from_tract_transformers(op))));
    }
    if let Some(op) = node.op_as::<QuantizedDynKeyValueCache>() {
        rule_if!(facts.iter().all(float) && op.axis == 2);
        return Ok(Some(Box::new(RocmQuantDynKVCache::from_tract_transformers(op))));
    }
    if let Some(op) = node.op_as::<Sdpa>() {
        // operands of one float type; rank 3 (one sequence) or 4
        rule_if!(facts.iter().all(float) && facts.iter().all(|f| f.datum_type == facts[0].datum_type));
        rule_if!(facts[0].rank() == facts[1].rank() && (facts[0].rank() == 3 || facts[0].rank() == 4));
        return Ok(Some(Box::new(RocmSdpa::from_tract_transformers(op)?)));
    }
    // Before the generic copy-based ops: try_make_copy_based_op would hand a DynKeyValueCache to the
    // reallocate-and-copy GpuDynKVCache (gpu/src/ops/copy_based.rs:32-34).
    if let Some(op) = node.op_as::<DynKeyValueCache>() {
        rule_if!(facts.iter().all(float) && op.axis == 2 && facts[0].rank() == 4);
        return Ok(Some(Box::new(RocmDynKVCache::from_tract_transformers(op))));
    }
    if node.op_is::<ApplyRope>() {
        rule_if!(facts.iter().all(float));
        return Ok(Some(Box::new(RocmApplyRope)));
    }
    if node.op_is::<RotateHalf>() {
        rule_if!(facts.iter().all(float));
        return Ok(Some(Box::new(RocmRotateHalf)));
    }
    if let Some(op) = node.op_as::<Cast>() {
        rule_if!(facts.iter().all(float));
        return Ok(RocmCast::new(op.to).map(|c| Box::new(c) as Box<dyn TypedOp>));
    }
    rule_if!(facts.iter().all(|f| DeviceTensor::is_supported_dt(f.datum_type)));
    tract_gpu::ops::copy_based::try_make_copy_based_op(source, node)
}

impl Translate<TypedFact, Box<dyn TypedOp>, TypedFact, Box<dyn TypedOp>> for RocmTransform {
    fn translate_node(
        &self,
        source: &TypedModel,
        node: &TypedNode,
        target: &mut TypedModel,
        mapping: &HashMap<OutletId, OutletId>,
    ) -> TractResult<TVec<OutletId>> {
        // (constant inputs of a device op are uploaded by sync_inputs_if_required itself, gpu/src/sync.rs:117-128)
        let forced_cpu = TRACT_ROCM_FORCE_CPU.get().split(',').any(|pat| !pat.is_empty() && node.name.contains(pat));
        // activations x constant Q4_0 weights [n, k] (PrefixMatMul with transpose_b, the shape exported decoders have,
        // cuda/src/transform.rs:204-270): the weights go to the library now, the node keeps the activations as its input
        if !forced_cpu {
            if let Some(op) = node.op_as::<PrefixMatMul>() {
                let facts = source.node_input_facts(node.id)?;
                let weights = facts[1].konst.as_ref().filter(|_| tract_gpu::utils::as_quant_fact(facts[1], &Q4_0).is_some());
                if let (Some(weights), true, false, true) = (
                    weights,
                    matches!(facts[0].datum_type, DatumType::F32 | DatumType::F16),
                    op.transpose_a || op.transpose_c,
                    op.transpose_b && op.quantize_output.is_none(),
                ) {
                    let device_op = RocmQ40Gemm { weights: Q40DeviceWeights::from_konst(weights)? };
                    let mut as_unary = node.clone();
                    as_unary.inputs = tvec!(node.inputs[0]);
                    let inputs = sync_inputs_if_required(target, &as_unary, mapping, DeviceSyncKind::ToDevice)?;
                    let mut outlets = target.wire_node(node.name.clone(), device_op, &inputs)?;
                    // (the CPU op may promise another float type than the activations': cast, as the reference does at :287-297)
                    let want = source.node_output_facts(node.id)?[0].datum_type;
                    if want != facts[0].datum_type {
                        if let Some(cast) = RocmCast::new(want) {
                            outlets = target.wire_node(format!("{}.out_cast", node.name), cast, &outlets)?;
                        }
                    }
                    return sync_model_outputs_if_required(source, node, target, outlets);
                }
            }
        }
        // ApplyRope(Q), ApplyRope(K_new), InPlaceKvSdpa as one device op (one launch per decode step).  The two rotation
        // nodes were translated when the walk passed them; with their only consumer gone they are dead and the
        // compaction that follows the translation drops them.
        if !forced_cpu && TRACT_ROCM_FUSE_ROPE.get() {
            if let Some(fused_inputs) = rope_feeding(source, node) {
                let facts: TVec<&TypedFact> = fused_inputs.iter().map(|o| source.outlet_fact(*o)).collect::<TractResult<_>>()?;
                if facts.iter().all(|f| matches!(f.datum_type, DatumType::F32 | DatumType::F16)) && facts.iter().all(|f| f.datum_type == facts[0].datum_type) {
                    let op = RocmInPlaceKvSdpa::from_inplace(node.op_as::<InPlaceKvSdpa>().unwrap(), kv_storage()?).with_rope();
                    let mut as_fused = node.clone();
                    as_fused.inputs = fused_inputs;
                    let inputs = sync_inputs_if_required(target, &as_fused, mapping, DeviceSyncKind::ToDevice)?;
                    let outlets = target.wire_node(node.name.clone(), op, &inputs)?;
                    return sync_model_outputs_if_required(source, node, target, outlets);
                }
            }
        }
        let device_op = if forced_cpu { None } else { try_make_rocm_op(source, node)? };
        // The op must accept the facts it will really see: every input as a device fact (what the ToDevice syncs
        // produce).  An op that refuses them stays on the CPU instead of aborting the translation.
        if let Some(op) = device_op {
            let as_device: TVec<TypedFact> = node
                .inputs
                .iter()
                .map(|i| {
                    let f = target.outlet_fact(mapping[i])?.clone();
                    if f.as_device_fact().is_some() { Ok(f) } else { Ok(tract_gpu::fact::DeviceFact::from_host(f)?.into_exotic_fact()) }
                })
                .collect::<TractResult<_>>()?;
            let refs: TVec<&TypedFact> = as_device.iter().collect();
            if op.output_facts(&refs).is_ok() {
                let inputs = sync_inputs_if_required(target, node, mapping, DeviceSyncKind::ToDevice)?;
                let outlets = target.wire_node(node.name.clone(), op, &inputs)?;
                return sync_model_outputs_if_required(source, node, target, outlets);
            }
            log::debug!("tract-rocm: {} stays on the CPU (its device op refused the input facts)", node.name);
        }
        let inputs = sync_inputs_if_required(target, node, mapping, DeviceSyncKind::ToHost)?;
        target.wire_node(&node.name, node.op.clone(), &inputs)
    }
}
