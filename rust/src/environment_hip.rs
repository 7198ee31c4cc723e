//! The device-facing half of `src/environment.rs`, rewritten over `device::hip`.
//!
//! What this file replaces in `src/environment.rs` (everything else in that file -- parameter construction,
//! `reset_parameter`, `scope`, `build_graph`, the random initialisers -- stays as it is and only ever reaches the
//! device through `writer` / `reader`):
//!
//!   lines  42-76   `ParameterWriter` / `ParameterReader` (wrappers of StagingWriter / StagingReader)
//!   lines  84-124  `struct Environment` and `Environment::new`
//!   lines 160-188  `writer`, `reader`
//!   lines 241-324  `run_kernel` (descriptor sets, pipeline bind, push constant, dispatch, barrier): gone -- a whole
//!                  graph is handed to the library once and `dsc_schedule_run` performs the launches
//!   lines 326-516  `run`
//!   lines 518-528  `print_timings`, `Drop`
//!
//! `Cargo.toml`: drop `spark` and `shaderc` (lines 12-13); nothing is added (the binding is `extern "C"`).
//! `src/lib.rs`: `mod device;` keeps its name and now contains `pub mod hip;` only; add `mod kernel_marshal;`.
//! `src/kernel.rs`: keep the descriptor types (lines 6-35, 146-149, 196-201, 386-391, 560-565, 645-650, 713-717,
//! 813-818, 878-886) and `label_name`; delete the `Kernel` trait's `generate_source`, `KernelModule`,
//! `KernelCacheWorker` and `KernelCache` (lines 925-1070) together with the two `.glsl` files.

use crate::common::*;
use crate::device::hip::*;
use crate::kernel_marshal::{graph_fingerprint, MarshalledSchedule};
use slotmap::SlotMap;
use std::{
    cell::RefCell,
    collections::HashMap,
    io::{self, prelude::*},
    rc::Rc,
};

/// `io::Write` into a parameter's buffer.  As in the reference, what has not been written when the writer is dropped
/// is zero-filled (src/device/staging.rs:181-187), which is also what `zero_fill` relies on.
pub struct ParameterWriter<'a> {
    device: &'a mut HipDevice,
    buffer: BufferId,
    offset: usize,
    size: usize,
}

impl<'a> ParameterWriter<'a> {
    pub fn zero_fill(self) {
        // consumed here; Drop zeroes from the current offset to the end
    }
}

impl<'a> io::Write for ParameterWriter<'a> {
    fn write(&mut self, buf: &[u8]) -> io::Result<usize> {
        let count = buf.len().min(self.size - self.offset);
        if count > 0 {
            // the library copies through its pinned staging ring; `buf` may be reused as soon as this returns
            self.device.write(self.buffer, self.offset, &buf[..count]);
            self.offset += count;
        }
        Ok(count)
    }

    fn flush(&mut self) -> io::Result<()> {
        Ok(())
    }
}

impl<'a> Drop for ParameterWriter<'a> {
    fn drop(&mut self) {
        if self.offset < self.size {
            self.device.fill_zero(self.buffer, self.offset, self.size - self.offset);
        }
    }
}

/// `io::Read` / `io::BufRead` of a parameter's buffer.  The reference streams through two mapped staging regions; here
/// the read-back lands in one host vector first (`dsc_buf_read` blocks until the data is there).
pub struct ParameterReader {
    bytes: Vec<u8>,
    next: usize,
}

impl io::Read for ParameterReader {
    fn read(&mut self, buf: &mut [u8]) -> io::Result<usize> {
        let count = buf.len().min(self.bytes.len() - self.next);
        buf[..count].copy_from_slice(&self.bytes[self.next..self.next + count]);
        self.next += count;
        Ok(count)
    }
}

impl io::BufRead for ParameterReader {
    fn fill_buf(&mut self) -> io::Result<&[u8]> {
        Ok(&self.bytes[self.next..])
    }

    fn consume(&mut self, amt: usize) {
        self.next += amt;
    }
}

/// One schedule per distinct graph, created the first time such a graph runs (graphs are built once and run many
/// times: examples/fashion_mnist/main.rs:360-448).  The key is `graph_fingerprint`, a hash of the graph's content:
/// nothing of the `Graph` is held, so a graph that is dropped and rebuilt finds its schedule again, and a different
/// graph that happens to reuse the old one's memory cannot be mistaken for it.
struct GraphSchedule {
    marshalled: Box<MarshalledSchedule>,
    schedule: HipSchedule,
    slots: Vec<dsc_buf>,
}

pub struct Environment {
    device: HipDevice,
    parameters: SharedParameters,
    schedules: HashMap<u64, GraphSchedule>,
}

impl Default for Environment {
    fn default() -> Self {
        Self::new()
    }
}

impl Environment {
    pub fn new() -> Self {
        Self {
            device: HipDevice::new(),
            parameters: Rc::new(RefCell::new(SlotMap::with_key())),
            schedules: HashMap::new(),
        }
    }

    pub fn writer(&mut self, parameter: &Parameter) -> ParameterWriter {
        let parameter_id = parameter.checked_id(&self.parameters);
        let mut parameters = self.parameters.borrow_mut();
        let param = parameters.get_mut(parameter_id).unwrap();
        if let Some(buffer_id) = param.buffer_id.take() {
            self.device.free(buffer_id);
        }
        let size = param.shape.buffer_size();
        let buffer_id = self.device.alloc(size).unwrap();
        param.buffer_id = Some(buffer_id);
        ParameterWriter { device: &mut self.device, buffer: buffer_id, offset: 0, size }
    }

    pub fn reader(&mut self, parameter: &Parameter) -> ParameterReader {
        let parameter_id = parameter.checked_id(&self.parameters);
        let parameters = self.parameters.borrow();
        let param = parameters.get(parameter_id).unwrap();
        let buffer_id = param.buffer_id.unwrap();
        let mut bytes = vec![0u8; param.shape.buffer_size()];
        self.device.read(buffer_id, 0, &mut bytes);
        ParameterReader { bytes, next: 0 }
    }

    /// `Environment::run` (src/environment.rs:326-516).  The use-count bookkeeping, the lazy allocation and release of
    /// node buffers, the ScatterAdd accumulator hand-off and the move of output buffers into parameters all happen
    /// inside `dsc_schedule_run`, over the fused launch list; this side only passes the parameters' buffers in and
    /// takes the new ones back.
    pub fn run(&mut self, graph: &Graph, rand_seed: u32) {
        let key = graph_fingerprint(graph);
        let device = &self.device;
        let entry = self.schedules.entry(key).or_insert_with(|| {
            let marshalled = MarshalledSchedule::new(graph);
            let schedule = HipSchedule::new(device, &marshalled.desc, 0);
            let slots = vec![0; marshalled.params.len()];
            GraphSchedule { marshalled, schedule, slots }
        });
        let mut parameters = self.parameters.borrow_mut();
        for (slot, parameter_id) in entry.slots.iter_mut().zip(entry.marshalled.params.iter()) {
            *slot = parameters[*parameter_id].buffer_id.map_or(0, |id| id.0);
        }
        entry.schedule.run(&mut entry.slots, rand_seed);
        for (slot, parameter_id) in entry.slots.iter().zip(entry.marshalled.params.iter()) {
            parameters[*parameter_id].buffer_id = if *slot != 0 { Some(BufferId(*slot)) } else { None };
        }
    }

    pub fn print_timings(&mut self, label: &str) {
        self.device.print_timings(label, 5);
    }
}
/// `Drop for Environment` (src/environment.rs:523-528) waited for the device.  Here the schedules go first, while the
/// context they were created on is still alive; `HipDevice::drop` then waits for the stream and frees everything.
impl Drop for Environment {
    fn drop(&mut self) {
        self.schedules.clear();
    }
}
