// The backend-generic acceptance tests of ug-core/src/common_tests.rs, as ug-cuda/tests/lb_tests.rs
// runs them.  `cat` can run on the device too: ughip_alloc zero-fills like the CPU backend.
use ug::Result;

#[test]
fn lb_hip_add() -> Result<()> {
    let dev = ug_hip::Device::new(0)?;
    ug::common_tests::lb::add(&dev)
}

#[test]
fn lb_hip_mm() -> Result<()> {
    let dev = ug_hip::Device::new(0)?;
    ug::common_tests::lb::mm(&dev)
}

#[test]
fn lb_hip_cat() -> Result<()> {
    let dev = ug_hip::Device::new(0)?;
    ug::common_tests::lb::cat(&dev)
}
