#![cfg(test)]
//! The suites of test-rt run through the `rocm` runtime, in three arrangements: the registered runtime as users
//! get it, the same with the device arena sized from the resolved symbols, and the translation alone without
//! tract's optimiser (so that a failure can be told apart from an optimiser interaction).

use std::sync::Arc;

use pastey::paste;
use tract_core::internal::*;
use tract_core::runtime::Runtime;
use tract_core::transform::ModelTransform;

#[path = "../suite.rs"]
mod suite;

#[derive(Clone, Debug)]
struct ArenaState {
    state: TypedSimpleState,
    use_arena: bool,
}

impl State for ArenaState {
    fn run(&mut self, inputs: TVec<TValue>) -> TractResult<TVec<TValue>> {
        if !self.use_arena {
            return self.state.run(inputs);
        }
        // a fresh plan whose node outputs live in one device arena (gpu/src/session_handler.rs)
        let handler = tract_gpu::session_handler::DeviceSessionHandler::from_plan(
            self.state.plan(),
            &self.state.turn_state.resolved_symbols,
        )?;
        let plan = Arc::new(Arc::unwrap_or_clone(self.state.plan().clone()).with_session_handler(handler));
        plan.spawn()?.run(inputs)
    }
    fn input_count(&self) -> usize {
        self.state.input_count()
    }
    fn output_count(&self) -> usize {
        self.state.output_count()
    }
    fn runnable(&self) -> &dyn Runnable {
        self.state.runnable()
    }
    fn freeze(&self) -> Box<dyn FrozenState> {
        Box::new(self.state.freeze())
    }
}

#[derive(Debug)]
struct ArenaRunnable {
    runnable: Arc<TypedRunnableModel>,
    use_arena: bool,
}

impl Runnable for ArenaRunnable {
    fn spawn(&self) -> TractResult<Box<dyn State>> {
        Ok(Box::new(ArenaState { state: self.runnable.spawn()?, use_arena: self.use_arena }))
    }
    fn input_count(&self) -> usize {
        self.runnable.input_count()
    }
    fn output_count(&self) -> usize {
        self.runnable.output_count()
    }
    fn typed_model(&self) -> Option<&Arc<TypedModel>> {
        self.runnable.typed_model()
    }
    fn typed_plan(&self) -> Option<&Arc<TypedSimplePlan>> {
        self.runnable.typed_plan()
    }
}

#[derive(Debug)]
struct RocmTestRuntime {
    name: &'static str,
    optimize: bool,
    use_arena: bool,
}

impl Runtime for RocmTestRuntime {
    fn name(&self) -> StaticName {
        self.name.into()
    }
    fn prepare_with_options(&self, mut model: TypedModel, options: &RunOptions) -> TractResult<Box<dyn Runnable>> {
        tract_rocm::RocmTransform.transform(&mut model)?;
        if self.optimize {
            model = model.into_optimized()?;
        }
        Ok(Box::new(ArenaRunnable { runnable: model.into_runnable_with_options(options)?, use_arena: self.use_arena }))
    }
    fn check(&self) -> TractResult<()> {
        tract_core::runtime::runtime_for_name("rocm")?.context("No rocm runtime found")?.check()
    }
}

macro_rules! rocm_test_suite {
    ($id: ident, $optimize: expr, $use_arena: expr) => {
        paste! {
            mod [<$id>] {
                use super::*;

                fn runtime() -> &'static RocmTestRuntime {
                    lazy_static::lazy_static! {
                        static ref RT: RocmTestRuntime = RocmTestRuntime { name: stringify!([<$id>]), optimize: $optimize, use_arena: $use_arena };
                    };
                    &RT
                }

                include!(concat!(env!("OUT_DIR"), "/tests/tests.rs"));
            }
        }
    };
}

rocm_test_suite!(optimized_rocm, true, false);
rocm_test_suite!(optimized_rocm_with_arena, true, true);
rocm_test_suite!(translated_rocm, false, false);

/// ApplyRope(Q), ApplyRope(K_new), InPlaceKvSdpa with shared Cos / Sin becomes ONE device op (the rotations fold into
/// the fused cache + attention op), and a decode loop through it matches the same graph on the CPU.
mod rope_fusion {
    use super::*;
    use tract_transformers::ops::apply_rope::ApplyRope;
    use tract_transformers::ops::inplace_kv_cache::InPlaceKvSdpa;

    fn block(dt: DatumType, b: usize, hq: usize, hkv: usize, d: usize) -> TractResult<TypedModel> {
        let mut m = TypedModel::default();
        let s = m.sym("S");
        let q = m.add_source("q", dt.fact(dims!(b, hq, s.clone(), d)))?;
        let k = m.add_source("k", dt.fact(dims!(b, hkv, s.clone(), d)))?;
        let v = m.add_source("v", dt.fact(dims!(b, hkv, s.clone(), d)))?;
        let cos = m.add_source("cos", dt.fact(dims!(1, 1, s.clone(), d)))?;
        let sin = m.add_source("sin", dt.fact(dims!(1, 1, s, d)))?;
        let rq = m.wire_node("rope_q", ApplyRope, &[q, cos, sin])?[0];
        let rk = m.wire_node("rope_k", ApplyRope, &[k, cos, sin])?[0];
        let o = m.wire_node("attn", InPlaceKvSdpa { axis: 2, causal: true, scale: None }, &[rq, rk, v])?;
        m.set_output_outlets(&o)?;
        Ok(m)
    }

    #[test]
    fn rotations_fold_into_the_fused_op() -> TractResult<()> {
        let mut m = block(DatumType::F16, 2, 8, 2, 128)?;
        tract_rocm::RocmTransform.transform(&mut m)?;
        let names: Vec<String> = m.eval_order()?.into_iter().map(|n| m.node(n).op.name().to_string()).collect();
        assert!(names.iter().any(|n| n == "RocmRopeInPlaceKvSdpa"), "{names:?}");
        assert!(!names.iter().any(|n| n.contains("ApplyRope")), "{names:?}");
        Ok(())
    }

    #[test]
    fn decode_loop_matches_the_cpu_graph() -> TractResult<()> {
        let (b, hq, hkv, d) = (2, 8, 2, 128);
        let cpu = block(DatumType::F16, b, hq, hkv, d)?.into_runnable()?;
        let mut dev_model = block(DatumType::F16, b, hq, hkv, d)?;
        tract_rocm::RocmTransform.transform(&mut dev_model)?;
        let dev = dev_model.into_runnable()?;
        let (mut cpu_state, mut dev_state) = (cpu.spawn()?, dev.spawn()?);
        for (step, n) in [5usize, 1, 1, 1].into_iter().enumerate() {
            let rnd = |shape: &[usize], seed: usize| -> TractResult<TValue> {
                let len: usize = shape.iter().product();
                let data: Vec<f32> = (0..len).map(|i| (((i * 2654435761 + seed * 40503) % 2001) as f32 / 1000.0) - 1.0).collect();
                Ok(tensor1(&data).into_shape(shape)?.cast_to::<f16>()?.into_owned().into_tvalue())
            };
            let inputs = tvec!(
                rnd(&[b, hq, n, d], step)?,
                rnd(&[b, hkv, n, d], step + 10)?,
                rnd(&[b, hkv, n, d], step + 20)?,
                rnd(&[1, 1, n, d], step + 30)?,
                rnd(&[1, 1, n, d], step + 40)?
            );
            let want = cpu_state.run(inputs.clone())?;
            let got = dev_state.run(inputs)?;
            got[0].close_enough(&want[0], Approximation::Approximate)?;
        }
        Ok(())
    }
}
