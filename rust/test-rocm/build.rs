#[path = "suite.rs"]
mod suite;

fn main() {
    // The attention kernels accumulate in f32 and round once to the output type; the suite's closed-form
    // reference is compared with the tolerance the CUDA and Metal runners use.
    suite::suite().test_runtime("tests", "suite::suite()", "runtime()", "Approximation::VeryApproximate");
}
