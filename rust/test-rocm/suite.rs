use infra::Test;
use suite_unit::sdpa::{SdpaProblem, SdpaProblemParams};
use tract_core::num_traits::Float;
use tract_core::prelude::Datum;
use tract_core::tract_data::half;

pub fn suite() -> &'static infra::TestSuite {
    lazy_static::lazy_static! {
        static ref SUITE: infra::TestSuite = mk_suite();
    };
    &SUITE
}

fn mk_suite() -> infra::TestSuite {
    // Everything the translator leaves on the CPU must still give the right answer through the DeviceSync
    // nodes, so the whole of both suites runs; only the attention cases decide which kernels are exercised.
    let onnx = suite_onnx::suite().clone();
    let mut unit = suite_unit::suite().unwrap().clone();
    unit.ignore_case(&ignore_unit);
    // Head sizes with a fast kernel (64 and 128) and a few that fall to the generic one.
    unit.get_sub_mut("sdpa").add_arbitrary::<SdpaProblem<half::f16>>(
        "proptest_f16",
        SdpaProblemParams { embed_dims: vec![64, 128] },
    );
    unit.get_sub_mut("sdpa").add_arbitrary::<SdpaProblem<f32>>(
        "proptest_f32_generic",
        SdpaProblemParams { embed_dims: vec![16, 64, 80] },
    );
    infra::TestSuite::default().with("onnx", onnx).with("unit", unit)
}

/// Unlike the CUDA runner (test-rt/test-cuda/suite.rs:42-61) no head size is excluded: what the MFMA kernels do
/// not take runs on the generic kernel.  Skipped: cases whose K and V differ in their last dimension, which no
/// kernel here handles (the translator leaves them on the CPU, where the plain suite already covers them).
fn ignore_unit(_t: &[String], case: &dyn Test) -> bool {
    fn square<F: Datum + Float>(p: &SdpaProblem<F>) -> bool {
        p.k.shape().last() == p.v.shape().last()
    }
    if let Some(p) = case.downcast_ref::<SdpaProblem<f32>>() {
        return !square(p);
    }
    if let Some(p) = case.downcast_ref::<SdpaProblem<half::f16>>() {
        return !square(p);
    }
    false
}
