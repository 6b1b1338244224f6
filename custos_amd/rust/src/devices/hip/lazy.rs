use crate::HIP;

use super::api::{custos_hip_capture_begin, custos_hip_capture_end_reuse, custos_hip_graph_destroy, custos_hip_graph_launch};

/// `Lazy::run` calls every recorded operation and then the device's `run`
/// (`src/modules/lazy.rs:190-197`).  The device records while those operations are called
/// (nothing is launched), so `run` ends the recording, gets a graph for it, launches the
/// graph once and starts recording again for the next run.  The graph is built from the
/// first recording; later runs record the same program, get the same graph back without
/// any build, and launch it once -- the CUDA device runs every operation eagerly and then
/// the graph again from the second run on (`src/devices/cuda/lazy.rs:31-49`).  A changed
/// program (a new operation, another buffer) builds a new graph by itself.  The reference's
/// wait after the launch is deferred (`HipDevice::run_waits`): beginning the next recording
/// takes no wait either, and the first read, write, allocation or `sync` while it is open does.
impl<Mods> crate::LazyRun for HIP<Mods> {
    fn run(&self) -> crate::Result<()> {
        let previous = self.graph.get();
        let mut graph = core::ptr::null_mut();
        self.check(unsafe { custos_hip_capture_end_reuse(self.handle, previous, &mut graph) })?;
        if graph != previous && !previous.is_null() {
            self.check(unsafe { custos_hip_graph_destroy(self.handle, previous) })?;
        }
        self.graph.set(graph);
        self.check(unsafe { custos_hip_graph_launch(self.handle, graph) })?;
        if self.run_waits.get() {
            self.sync()?;
        }
        self.check(unsafe { custos_hip_capture_begin(self.handle) })?;
        Ok(())
    }
}

impl<Mods: crate::RunModule<Self>> crate::Run for HIP<Mods> {
    #[inline]
    fn run(&self) -> crate::Result<()> {
        self.modules.run(self)
    }
}

impl<Mods> crate::LazySetup for HIP<Mods> {
    /// From here on launches, clears and copies are recorded; allocation, reads and writes
    /// stay legal and execute at once (`src/devices/cuda/lazy.rs:57-72` opens a global
    /// stream capture, under which `cuMemAlloc` fails).
    #[inline]
    fn lazy_setup(&mut self) -> crate::Result<()> {
        self.check(unsafe { custos_hip_capture_begin(self.handle) })?;
        Ok(())
    }
}
