//! Record once, replay many: the device-side form of the reference's lazy mode
//! (`Autograd<Lazy<Base>>` + `dev.run()`, examples/sine_net.rs:178-220).  Everything the body issues
//! on the device lands in a HIP graph; `run()` replays it as one launch.  The body must not
//! allocate, read back or wait: run the same sequence eagerly once before (a `Cached` device then
//! owns every output and gradient buffer), and keep the buffers alive while the graph is in use.
use crate::{check, ffi, HipError, HIP};

pub struct Graph {
    ctx: *mut ffi::SlhipCtx,
    g: *mut ffi::SlhipGraph,
}

impl<Mods> HIP<Mods> {
    pub fn record(&self, body: impl FnOnce()) -> Result<Graph, HipError> {
        check(unsafe { ffi::slhip_graph_begin(self.ctx) })?;
        body();
        let mut g = core::ptr::null_mut();
        check(unsafe { ffi::slhip_graph_end(self.ctx, &mut g) })?;
        Ok(Graph { ctx: self.ctx, g })
    }
}

impl Graph {
    pub fn run(&self) -> Result<(), HipError> {
        check(unsafe { ffi::slhip_graph_launch(self.ctx, self.g) })
    }
    /// Kernels in the recording.
    pub fn nodes(&self) -> usize {
        let mut n = 0usize;
        unsafe { ffi::slhip_graph_node_count(self.g, &mut n) };
        n
    }
}

impl Drop for Graph {
    fn drop(&mut self) {
        unsafe { ffi::slhip_graph_destroy(self.g) };
    }
}
