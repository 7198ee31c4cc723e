//! `src/device/hip.rs` -- binding of `libdescent_hip.so` (C ABI: `include/descent_hip.h`) for the descent crate.
//!
//! It takes the place of the crate's Vulkan device layer (`src/device/{context,buffer_heap,heap,staging,
//! command_buffer,fence,descriptor_pool,timestamp}.rs`) and of the shader side of `src/kernel.rs`
//! (`KernelCache`, `KernelModule`, every `generate_source`).  The graph builder, autodiff, `Module`s and optimisers
//! are untouched: `Environment` keeps its public API and calls `HipDevice` where it called `spark`.
//!
//! Every `#[repr(C)]` type below mirrors the struct of the same name in the header, field for field and in order;
//! every `extern "C"` item is one export of the library.  `tests/test_rust_shim.py` of the backend's repository checks
//! both against the header mechanically (names, order, types, sizes, offsets, and that no export is missing).
#![allow(non_camel_case_types, dead_code)]

use std::ffi::{c_void, CStr};
use std::os::raw::{c_char, c_int};

pub const DSC_MAX_DIM: usize = 7;
pub const DSC_STATIC_SCRATCH_BYTES: usize = 64 << 20;

// dsc_status
pub const DSC_OK: c_int = 0;
pub const DSC_ERR_INVALID: c_int = 1;
pub const DSC_ERR_OOM: c_int = 2;
pub const DSC_ERR_HIP: c_int = 3;
pub const DSC_ERR_COMPILE: c_int = 4;
pub const DSC_ERR_UNSUPPORTED: c_int = 5;
pub const DSC_ERR_NO_DEVICE: c_int = 6;

// dsc_kernel_kind
pub const DSC_KERNEL_FILL: i32 = 0;
pub const DSC_KERNEL_PER_ELEMENT: i32 = 1;
pub const DSC_KERNEL_REDUCE: i32 = 2;
pub const DSC_KERNEL_MATMUL: i32 = 3;
pub const DSC_KERNEL_UNPAD: i32 = 4;
pub const DSC_KERNEL_WINDOWS_TO_IMAGE: i32 = 5;
pub const DSC_KERNEL_SCATTER_ADD: i32 = 6;

// dsc_pe_kind
pub const DSC_PE_LOAD: i32 = 0;
pub const DSC_PE_LITERAL_F32: i32 = 1;
pub const DSC_PE_LITERAL_U32: i32 = 2;
pub const DSC_PE_COORD: i32 = 3;
pub const DSC_PE_RAND: i32 = 4;
pub const DSC_PE_UNARY: i32 = 5;
pub const DSC_PE_BINARY: i32 = 6;
pub const DSC_PE_SELECT: i32 = 7;
pub const DSC_PE_GATHER: i32 = 8;

// dsc_schedule_create flags
pub const DSC_SCHEDULE_NO_FUSION: u32 = 1;
pub const DSC_SCHEDULE_NO_CONV_KERNELS: u32 = 2;
pub const DSC_SCHEDULE_GRAPH_REPLAY: u32 = 4;
pub const DSC_SCHEDULE_SPLIT_CONV_GRADS: u32 = 8;

#[repr(C)]
#[derive(Clone, Copy)]
pub struct dsc_shape {
    pub rank: i32,
    pub dims: [i64; DSC_MAX_DIM],
}

#[repr(C)]
#[derive(Clone, Copy)]
pub struct dsc_view {
    pub in_shape: dsc_shape,
    pub in_offset: [i64; DSC_MAX_DIM],
    pub out_shape: dsc_shape,
    pub map_axis: [i32; DSC_MAX_DIM],
    pub map_step: [i64; DSC_MAX_DIM],
}

#[repr(C)]
#[derive(Clone, Copy)]
pub struct dsc_pe_op {
    pub kind: i32,
    pub op: i32,
    pub args: [i32; 4],
    pub bits: u32,
    pub input_index: i32,
    pub view_index: i32,
    pub axis: i32,
    pub gather_shape: dsc_shape,
}

#[repr(C)]
#[derive(Clone, Copy)]
pub struct dsc_kernel_desc {
    pub kind: i32,
    pub shape: dsc_shape,
    pub n_inputs: i32,
    pub inputs: *const dsc_view,
    pub n_ops: i32,
    pub ops: *const dsc_pe_op,
    pub n_outputs: i32,
    pub outputs: *const i32,
    pub n_builtin_views: i32,
    pub builtin_views: *const dsc_view,
    pub fill_bits: u32,
    pub reduce_op: i32,
    pub axis: i32,
    pub pad: i32,
    pub stride_w: i32,
    pub stride_h: i32,
    pub output_mode: i32,
}

#[repr(C)]
#[derive(Clone, Copy)]
pub struct dsc_caps {
    pub has_float_atomic_add: i32,
    pub compute_units: i32,
    pub wavefront_size: i32,
    pub device_memory_bytes: i64,
    pub arch: [c_char; 32],
}

#[repr(C)]
#[derive(Clone, Copy)]
pub struct dsc_cluster_output {
    pub node: i32,
    pub copy_from: i32,
    pub copy_from_is_literal: i32,
    pub literal_bits: u32,
}

#[repr(C)]
#[derive(Clone, Copy)]
pub struct dsc_cluster {
    pub kernel: dsc_kernel_desc,
    pub n_inputs: i32,
    pub inputs: *const i32,
    pub n_outputs: i32,
    pub outputs: *const dsc_cluster_output,
}

#[repr(C)]
#[derive(Clone, Copy)]
pub struct dsc_param_io {
    pub node: i32,
    pub param: i32,
}

#[repr(C)]
#[derive(Clone, Copy)]
pub struct dsc_schedule_desc {
    pub n_nodes: i32,
    pub node_elements: *const i64,
    pub n_clusters: i32,
    pub clusters: *const dsc_cluster,
    pub n_inputs: i32,
    pub inputs: *const dsc_param_io,
    pub n_outputs: i32,
    pub outputs: *const dsc_param_io,
    pub n_params: i32,
}

/// Opaque handles of the library.
#[repr(C)]
pub struct dsc_ctx {
    _private: [u8; 0],
}
#[repr(C)]
pub struct dsc_kernel {
    _private: [u8; 0],
}
#[repr(C)]
pub struct dsc_schedule {
    _private: [u8; 0],
}
/// `BufferId` of `src/device/buffer_heap.rs:10-12` becomes this handle; 0 = none.
pub type dsc_buf = u64;

#[link(name = "descent_hip")]
extern "C" {
    pub fn dsc_last_error() -> *const c_char;
    pub fn dsc_ctx_create(device_ordinal: c_int, out: *mut *mut dsc_ctx) -> c_int;
    pub fn dsc_ctx_destroy(ctx: *mut dsc_ctx) -> c_int;
    pub fn dsc_ctx_caps(ctx: *mut dsc_ctx, out: *mut dsc_caps) -> c_int;
    pub fn dsc_ctx_sync(ctx: *mut dsc_ctx) -> c_int;
    pub fn dsc_fence_record(ctx: *mut dsc_ctx, out_fence: *mut u64) -> c_int;
    pub fn dsc_fence_wait(ctx: *mut dsc_ctx, fence: u64) -> c_int;
    pub fn dsc_fence_query(ctx: *mut dsc_ctx, fence: u64, out_finished: *mut c_int) -> c_int;
    pub fn dsc_ctx_stream(ctx: *mut dsc_ctx, out_stream: *mut *mut c_void) -> c_int;

    pub fn dsc_buf_alloc(ctx: *mut dsc_ctx, bytes: usize, out: *mut dsc_buf) -> c_int;
    pub fn dsc_buf_free(ctx: *mut dsc_ctx, buf: dsc_buf) -> c_int;
    pub fn dsc_buf_info(ctx: *mut dsc_ctx, buf: dsc_buf, out_device_ptr: *mut *mut c_void, out_bytes: *mut usize) -> c_int;
    pub fn dsc_heap_stats(ctx: *mut dsc_ctx, out_live_buffers: *mut i64, out_live_bytes: *mut i64, out_arena_bytes: *mut i64) -> c_int;
    pub fn dsc_buf_write(ctx: *mut dsc_ctx, buf: dsc_buf, offset: usize, src: *const c_void, bytes: usize) -> c_int;
    pub fn dsc_buf_fill_zero(ctx: *mut dsc_ctx, buf: dsc_buf, offset: usize, bytes: usize) -> c_int;
    pub fn dsc_buf_read(ctx: *mut dsc_ctx, buf: dsc_buf, offset: usize, dst: *mut c_void, bytes: usize) -> c_int;
    pub fn dsc_buf_alloc_io(ctx: *mut dsc_ctx, bytes: usize, out: *mut dsc_buf) -> c_int;
    pub fn dsc_host_alloc(ctx: *mut dsc_ctx, bytes: usize, out_ptr: *mut *mut c_void) -> c_int;
    pub fn dsc_host_free(ctx: *mut dsc_ctx, ptr: *mut c_void) -> c_int;
    pub fn dsc_buf_write_async(ctx: *mut dsc_ctx, buf: dsc_buf, offset: usize, src: *const c_void, bytes: usize, out_fence: *mut u64) -> c_int;
    pub fn dsc_buf_read_async(ctx: *mut dsc_ctx, buf: dsc_buf, offset: usize, dst: *mut c_void, bytes: usize, out_fence: *mut u64) -> c_int;

    pub fn dsc_kernel_get(ctx: *mut dsc_ctx, desc: *const dsc_kernel_desc, out: *mut *mut dsc_kernel) -> c_int;
    pub fn dsc_kernel_buffer_count(k: *const dsc_kernel) -> c_int;
    pub fn dsc_kernel_reference_group_count(k: *const dsc_kernel) -> i64;
    pub fn dsc_kernel_label(k: *const dsc_kernel) -> *const c_char;
    pub fn dsc_kernel_source(k: *const dsc_kernel) -> *const c_char;
    pub fn dsc_kernel_launch(ctx: *mut dsc_ctx, k: *mut dsc_kernel, bufs: *const dsc_buf, n: c_int, rand_seed: u32) -> c_int;
    pub fn dsc_codegen_source(desc: *const dsc_kernel_desc, out_source: *mut *mut c_char) -> c_int;
    pub fn dsc_codegen_compile(desc: *const dsc_kernel_desc, arch: *const c_char, out_code_bytes: *mut usize) -> c_int;
    pub fn dsc_codegen_check_schedule(desc: *const dsc_schedule_desc, flags: u32, arch: *const c_char, out_text: *mut *mut c_char) -> c_int;
    pub fn dsc_cache_stats(out_hits: *mut i64, out_compiles: *mut i64, out_rejected: *mut i64) -> c_int;
    pub fn dsc_free_string(s: *mut c_char);

    pub fn dsc_schedule_create(ctx: *mut dsc_ctx, desc: *const dsc_schedule_desc, flags: u32, out: *mut *mut dsc_schedule) -> c_int;
    pub fn dsc_schedule_destroy(ctx: *mut dsc_ctx, s: *mut dsc_schedule) -> c_int;
    pub fn dsc_schedule_run(ctx: *mut dsc_ctx, s: *mut dsc_schedule, params: *mut dsc_buf, rand_seed: u32) -> c_int;
    pub fn dsc_schedule_run_static(ctx: *mut dsc_ctx, s: *mut dsc_schedule, params: *mut dsc_buf, spare: *mut dsc_buf, rand_seed: u32) -> c_int;
    pub fn dsc_schedule_launch_count(s: *const dsc_schedule, out_launches: *mut i32, out_clusters: *mut i32) -> c_int;
    pub fn dsc_schedule_describe(s: *const dsc_schedule, out_text: *mut *mut c_char) -> c_int;
    pub fn dsc_schedule_dot(s: *const dsc_schedule, out_text: *mut *mut c_char) -> c_int;

    pub fn dsc_prof_enable(ctx: *mut dsc_ctx, enabled: c_int) -> c_int;
    pub fn dsc_prof_markers(ctx: *mut dsc_ctx, enabled: c_int) -> c_int;
    pub fn dsc_prof_reset(ctx: *mut dsc_ctx) -> c_int;
    pub fn dsc_prof_report(ctx: *mut dsc_ctx, top_n: c_int, out_text: *mut *mut c_char) -> c_int;
    pub fn dsc_prof_query(ctx: *mut dsc_ctx, prefix: *const c_char, out_avg_us: *mut f64, out_launches: *mut i64) -> c_int;
    pub fn dsc_prof_work(ctx: *mut dsc_ctx, prefix: *const c_char, out_total_us: *mut f64, out_algo_bytes: *mut f64, out_algo_flops: *mut f64, out_launches: *mut i64) -> c_int;
}

// ------------------------------------------------------------------------------------------------------------
// Safe layer: what `Environment` holds instead of SharedContext + FenceSet + CommandBuffers + BufferHeap +
// StagingBuffer + KernelCache + DescriptorPools + TimestampSets (src/environment.rs:84-124).

/// The reference unwraps every Vulkan result (`.unwrap()`, `assert!`, `panic!`); the shim keeps that behaviour and
/// panics with the library's message.
fn check(status: c_int, what: &str) {
    if status != DSC_OK {
        let msg = unsafe { CStr::from_ptr(dsc_last_error()) }.to_string_lossy().into_owned();
        panic!("descent_hip: {} failed with status {}: {}", what, status, msg);
    }
}

fn take_string(p: *mut c_char) -> String {
    let s = unsafe { CStr::from_ptr(p) }.to_string_lossy().into_owned();
    unsafe { dsc_free_string(p) };
    s
}

/// `BufferId` of the reference (`src/device/buffer_heap.rs:10-12`): the parameter storage and `run`'s node storage
/// keep these; ownership stays with the caller and a double free is a caller bug, as there.
#[derive(Debug, Clone, Copy, PartialEq, Eq, Hash)]
pub struct BufferId(pub dsc_buf);

/// Owner of the library context.  `HipDevice` and every `HipSchedule` created on it share one of these, so the
/// context is destroyed after the last of them: `dsc_schedule_destroy` hands a schedule's buffers back to the
/// context's heap and must find it alive.
struct ContextHandle(*mut dsc_ctx);

impl Drop for ContextHandle {
    /// `Drop for Environment` waits for the device (src/environment.rs:523-528); dsc_ctx_destroy does and frees all.
    fn drop(&mut self) {
        unsafe { dsc_ctx_destroy(self.0) };
    }
}

pub struct HipDevice {
    ctx: *mut dsc_ctx,
    owner: std::rc::Rc<ContextHandle>,
}

impl HipDevice {
    /// `Context::new()` + the device objects of `Environment::new` (src/environment.rs:104-124).
    pub fn new() -> Self {
        let mut ctx = std::ptr::null_mut();
        check(unsafe { dsc_ctx_create(0, &mut ctx) }, "dsc_ctx_create");
        let mut caps = std::mem::MaybeUninit::<dsc_caps>::uninit();
        check(unsafe { dsc_ctx_caps(ctx, caps.as_mut_ptr()) }, "dsc_ctx_caps");
        // src/kernel.rs:954 asserts shader float atomics when a ScatterAdd module is built; always present here
        assert_eq!(unsafe { caps.assume_init() }.has_float_atomic_add, 1);
        Self { ctx, owner: std::rc::Rc::new(ContextHandle(ctx)) }
    }

    pub fn raw(&self) -> *mut dsc_ctx {
        self.ctx
    }

    /// `BufferHeap::alloc` (src/device/buffer_heap.rs:79-97): `None` when the device is exhausted.
    pub fn alloc(&mut self, bytes: usize) -> Option<BufferId> {
        let mut h: dsc_buf = 0;
        let rc = unsafe { dsc_buf_alloc(self.ctx, bytes, &mut h) };
        if rc == DSC_ERR_OOM {
            return None;
        }
        check(rc, "dsc_buf_alloc");
        Some(BufferId(h))
    }

    /// `BufferHeap::free` (src/device/buffer_heap.rs:99-104).
    pub fn free(&mut self, id: BufferId) {
        check(unsafe { dsc_buf_free(self.ctx, id.0) }, "dsc_buf_free");
    }

    /// `StagingWriter::write_slice` to completion (src/device/staging.rs:85-178).
    pub fn write(&mut self, id: BufferId, offset: usize, bytes: &[u8]) {
        check(
            unsafe { dsc_buf_write(self.ctx, id.0, offset, bytes.as_ptr() as *const c_void, bytes.len()) },
            "dsc_buf_write",
        );
    }

    /// `StagingWriter::write_zeros` and the zero fill of the unwritten tail on drop (src/device/staging.rs:125-141,181-187).
    pub fn fill_zero(&mut self, id: BufferId, offset: usize, bytes: usize) {
        check(unsafe { dsc_buf_fill_zero(self.ctx, id.0, offset, bytes) }, "dsc_buf_fill_zero");
    }

    /// `StagingReader::read_slice` to completion (src/device/staging.rs:225-302).
    pub fn read(&mut self, id: BufferId, offset: usize, out: &mut [u8]) {
        check(
            unsafe { dsc_buf_read(self.ctx, id.0, offset, out.as_mut_ptr() as *mut c_void, out.len()) },
            "dsc_buf_read",
        );
    }

    /// `FenceSet::wait_for_signal` on the latest fence (src/device/fence.rs:73-86).
    pub fn sync(&mut self) {
        check(unsafe { dsc_ctx_sync(self.ctx) }, "dsc_ctx_sync");
    }

    /// `TimestampSets::print_timings` (src/device/timestamp.rs:155-179, src/environment.rs:518-520).
    pub fn print_timings(&mut self, label: &str, top_n: usize) {
        let mut text = std::ptr::null_mut();
        check(unsafe { dsc_prof_report(self.ctx, top_n as c_int, &mut text) }, "dsc_prof_report");
        println!("{}:\n{}", label, take_string(text));
        check(unsafe { dsc_prof_reset(self.ctx) }, "dsc_prof_reset");
    }

    pub fn enable_timings(&mut self, enabled: bool) {
        check(unsafe { dsc_prof_enable(self.ctx, enabled as c_int) }, "dsc_prof_enable");
    }
}

/// A whole `Graph` handed to the library once (see `kernel_marshal::MarshalledSchedule`); `run` is what
/// `Environment::run` calls per step.
pub struct HipSchedule {
    handle: *mut dsc_schedule,
    ctx: *mut dsc_ctx,
    _owner: std::rc::Rc<ContextHandle>, // keeps the context alive until this schedule has been destroyed
}

impl HipSchedule {
    pub fn new(device: &HipDevice, desc: &dsc_schedule_desc, flags: u32) -> Self {
        let mut handle = std::ptr::null_mut();
        check(unsafe { dsc_schedule_create(device.raw(), desc, flags, &mut handle) }, "dsc_schedule_create");
        Self { handle, ctx: device.raw(), _owner: device.owner.clone() }
    }

    /// `params[slot]` = current buffer of each parameter (0 = none); updated in place (src/environment.rs:506-515).
    pub fn run(&mut self, params: &mut [dsc_buf], rand_seed: u32) {
        check(unsafe { dsc_schedule_run(self.ctx, self.handle, params.as_mut_ptr(), rand_seed) }, "dsc_schedule_run");
    }

    /// The step without device allocation: `spare[slot]` holds one more buffer per written parameter.
    pub fn run_static(&mut self, params: &mut [dsc_buf], spare: &mut [dsc_buf], rand_seed: u32) {
        assert_eq!(params.len(), spare.len());
        check(
            unsafe { dsc_schedule_run_static(self.ctx, self.handle, params.as_mut_ptr(), spare.as_mut_ptr(), rand_seed) },
            "dsc_schedule_run_static",
        );
    }

    pub fn describe(&self) -> String {
        let mut text = std::ptr::null_mut();
        check(unsafe { dsc_schedule_describe(self.handle, &mut text) }, "dsc_schedule_describe");
        take_string(text)
    }
}

impl Drop for HipSchedule {
    /// Runs before `_owner` is released (fields drop after `drop` returns), so the context is still there.
    fn drop(&mut self) {
        unsafe { dsc_schedule_destroy(self.ctx, self.handle) };
    }
}
