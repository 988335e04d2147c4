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
