//! `HIP<Mods>`: an MI355X (gfx950) device for sliced, written the way the reference's own
//! devices are - one `impl` of every op trait under `src/ops2/` - with each method a single call
//! into libsliced_hip.so (`ffi.rs`, `include/sliced_hip.h`).  With these impls sliced's blanket
//! `*MayGrad` wrappers (`src/ops.rs`), `Matrix` and the examples run unchanged with
//! `D = HIP<Autograd<Cached<Base>>>`.
//!
//! NOT COMPILED: see README.md.  custos is named the way the reference's sources use it
//! (`src/ops.rs:6-11`, `src/ops2/gemm/opencl.rs:1-5`); where a custos item's exact shape could
//! only be inferred from that usage, a `// custos:` comment says what is assumed.
pub mod device;
pub mod ffi;
pub mod graph;
pub mod ops;
pub mod probe;

pub use device::{HipError, HipPtr, HIP};
pub use graph::Graph;

/// Turns a status of the C ABI into a `Result`, carrying `slhip_last_error_string()`.
pub fn check(status: i32) -> Result<(), HipError> {
    if status == ffi::SLHIP_OK {
        return Ok(());
    }
    let msg = unsafe { std::ffi::CStr::from_ptr(ffi::slhip_last_error_string()) }
        .to_string_lossy()
        .into_owned();
    Err(HipError { status, msg })
}
