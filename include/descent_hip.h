/*
 * descent_hip.h -- C ABI of the MI355X (gfx950) execution backend for descent.
 *
 * This is the boundary a `src/device/hip.rs` shim binds in place of the
 * reference's Vulkan device layer and GLSL kernel dispatch.  Every entry point
 * names the reference interface it replaces (paths relative to the reference
 * repository).  All functions return a dsc_status (0 = ok); where the
 * reference panics/unwraps, this library returns an error code and keeps a
 * message retrievable through dsc_last_error().
 *
 * Conventions
 *  - plain C types only; every tensor is a dense row-major array of 32-bit
 *    words (f32, or u32 bit patterns stored in "float" buffers exactly as the
 *    reference does, kernel.rs:42-47 and kernel_common.glsl:218-220);
 *  - a context owns one HIP stream; all work of a context is stream-ordered,
 *    which replaces the full pipeline barrier the reference records after
 *    each dispatch (environment.rs:305-323);
 *  - a context is not thread-safe (the reference is `!Send`: Rc/RefCell
 *    everywhere, e.g. parameter.rs:35, device/context.rs:31).
 */
#ifndef DESCENT_HIP_H
#define DESCENT_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------ status */

typedef enum dsc_status {
    DSC_OK = 0,
    DSC_ERR_INVALID = 1,     /* bad argument / malformed descriptor (reference: assert!/panic!) */
    DSC_ERR_OOM = 2,         /* arena exhausted (reference: BufferHeap::alloc -> None, buffer_heap.rs:79-97) */
    DSC_ERR_HIP = 3,         /* a HIP runtime call failed (reference: Vulkan call .unwrap()) */
    DSC_ERR_COMPILE = 4,     /* hipRTC rejected generated source (reference: shaderc panic, kernel.rs:978-980) */
    DSC_ERR_UNSUPPORTED = 5, /* descriptor valid but outside what this backend implements */
    DSC_ERR_NO_DEVICE = 6    /* no usable GPU (reference: Context::new panics, device/context.rs:76) */
} dsc_status;

/* ------------------------------------------------------- shapes and views */

#define DSC_MAX_DIM 7 /* shape.rs:10 MAX_DIM */

/* shape.rs:40-41 `Shape` */
typedef struct dsc_shape {
    int32_t rank;               /* 1..DSC_MAX_DIM */
    int64_t dims[DSC_MAX_DIM];  /* all > 0 */
} dsc_shape;

/*
 * shape.rs:354-360 `View`: how an op reads its argument.
 *   input coordinate on axis i = in_offset[i] + sum over output axes j with
 *   map_axis[j] == i of map_step[j] * out_coord[j], clamped to
 *   [0, in_shape[i]-1] when the reachable range leaves the input
 *   (shape.rs:503-526; padding is edge-replicate, shape.rs:374-379).
 *   map_axis[j] == -1 is AxisMapping::Broadcast (shape.rs:322-325).
 */
typedef struct dsc_view {
    dsc_shape in_shape;
    int64_t in_offset[DSC_MAX_DIM];
    dsc_shape out_shape;
    int32_t map_axis[DSC_MAX_DIM];
    int64_t map_step[DSC_MAX_DIM];
} dsc_view;

/* ------------------------------------------------------ kernel descriptors */

/* kernel.rs:878-886 `GenericKernel` variants */
typedef enum dsc_kernel_kind {
    DSC_KERNEL_FILL = 0,             /* kernel.rs:146-193 */
    DSC_KERNEL_PER_ELEMENT = 1,      /* kernel.rs:196-383 */
    DSC_KERNEL_REDUCE = 2,           /* kernel.rs:560-642 */
    DSC_KERNEL_MATMUL = 3,           /* kernel.rs:386-557 + kernel_matmul.glsl */
    DSC_KERNEL_UNPAD = 4,            /* kernel.rs:645-710 */
    DSC_KERNEL_WINDOWS_TO_IMAGE = 5, /* kernel.rs:713-810 */
    DSC_KERNEL_SCATTER_ADD = 6       /* kernel.rs:813-874 */
} dsc_kernel_kind;

/* kernel.rs:8-35 `PerElementKernelOp` variants */
typedef enum dsc_pe_kind {
    DSC_PE_LOAD = 0,        /* Load{input_index} */
    DSC_PE_LITERAL_F32 = 1, /* Literal(F32): bits = value bits */
    DSC_PE_LITERAL_U32 = 2, /* Literal(U32): bits = value */
    DSC_PE_COORD = 3,       /* BuiltIn{Coord, view}: view = builtin_views[view_index] */
    DSC_PE_RAND = 4,        /* BuiltIn{Rand{uid}, view}: bits = uid */
    DSC_PE_UNARY = 5,       /* op = dsc_unary_op, args[0] */
    DSC_PE_BINARY = 6,      /* op = dsc_binary_op, args[0..2] */
    DSC_PE_SELECT = 7,      /* op = dsc_compare_mode, (args[0] OP args[1]) ? args[2] : args[3] */
    DSC_PE_GATHER = 8       /* table = inputs[input_index], index bits = args[0], axis, gather_shape */
} dsc_pe_kind;

/* op.rs:59-70 */
typedef enum dsc_unary_op {
    DSC_UN_MOV = 0, DSC_UN_NEG, DSC_UN_SQRT, DSC_UN_EXP, DSC_UN_LOG, DSC_UN_SIN, DSC_UN_COS,
    DSC_UN_FLOAT_TO_UINT, DSC_UN_UINT_TO_FLOAT
} dsc_unary_op;

/* op.rs:46-57 */
typedef enum dsc_binary_op {
    DSC_BIN_ADD = 0, DSC_BIN_SUB, DSC_BIN_MUL, DSC_BIN_DIV, DSC_BIN_POW,
    DSC_BIN_UADD, DSC_BIN_UMUL, DSC_BIN_UREM, DSC_BIN_UBITXOR
} dsc_binary_op;

/* op.rs:40-44 */
typedef enum dsc_compare_mode { DSC_CMP_EQ = 0, DSC_CMP_GT = 1 } dsc_compare_mode;
/* op.rs:28-32 */
typedef enum dsc_reduce_op { DSC_REDUCE_MAX = 0, DSC_REDUCE_SUM = 1 } dsc_reduce_op;
/* op.rs:76-80 */
typedef enum dsc_matmul_output_mode { DSC_MATMUL_BATCHES = 0, DSC_MATMUL_ROWS = 1 } dsc_matmul_output_mode;

typedef struct dsc_pe_op {
    int32_t kind;        /* dsc_pe_kind */
    int32_t op;          /* dsc_unary_op / dsc_binary_op / dsc_compare_mode */
    int32_t args[4];     /* indices of earlier ops in the list */
    uint32_t bits;       /* literal bits, or rand uid */
    int32_t input_index; /* LOAD / GATHER: which input buffer (and input view) */
    int32_t view_index;  /* COORD / RAND: index into builtin_views */
    int32_t axis;        /* GATHER */
    dsc_shape gather_shape; /* GATHER: shape of the gather node (kernel.rs:29-34) */
} dsc_pe_op;

/*
 * One kernel, equal by content to a reference `GenericKernel`; content
 * equality is the cache key exactly as `#[derive(Hash, Eq)]` is in
 * kernel.rs:1037-1056.
 *
 * Buffer binding order at launch = inputs in order, then outputs
 * (environment.rs:465-471):
 *   FILL              : [out]
 *   PER_ELEMENT       : inputs[0..n_inputs), outputs[0..n_outputs)
 *   REDUCE/UNPAD/W2I  : [input, out]
 *   MATMUL            : [a, b, out]
 *   SCATTER_ADD       : [values, indices, accumulator(in/out)]
 */
typedef struct dsc_kernel_desc {
    int32_t kind;            /* dsc_kernel_kind */
    dsc_shape shape;         /* output/node shape; FILL and PER_ELEMENT: {1,[element_count]} */
    int32_t n_inputs;        /* number of input views below */
    const dsc_view* inputs;  /* PER_ELEMENT: per input; MATMUL: {a,b}; REDUCE/UNPAD/W2I: {input};
                                SCATTER_ADD: {values, indices}; FILL: none */
    /* PER_ELEMENT only */
    int32_t n_ops;
    const dsc_pe_op* ops;
    int32_t n_outputs;
    const int32_t* outputs;  /* op index stored to each output (kernel.rs:199) */
    int32_t n_builtin_views;
    const dsc_view* builtin_views;
    /* scalar attributes */
    uint32_t fill_bits;      /* FILL: literal bits (kernel.rs:147) */
    int32_t reduce_op;       /* REDUCE */
    int32_t axis;            /* REDUCE / UNPAD / SCATTER_ADD */
    int32_t pad;             /* UNPAD */
    int32_t stride_w;        /* WINDOWS_TO_IMAGE (kernel.rs:716; tuple order is (w,h), kernel.rs:740) */
    int32_t stride_h;
    int32_t output_mode;     /* MATMUL: dsc_matmul_output_mode */
} dsc_kernel_desc;

/* ---------------------------------------------------------------- context */

typedef struct dsc_ctx dsc_ctx;
typedef struct dsc_kernel dsc_kernel;
typedef uint64_t dsc_buf; /* opaque buffer handle, 0 = none (reference: BufferId slotmap key, buffer_heap.rs:10-12) */

typedef struct dsc_caps {
    int32_t has_float_atomic_add; /* device/context.rs:28,132-138; always 1 on gfx950 */
    int32_t compute_units;
    int32_t wavefront_size;
    int64_t device_memory_bytes;
    char arch[32];                /* e.g. "gfx950" */
} dsc_caps;

/* Last error message of this thread (valid until the next failing call). */
const char* dsc_last_error(void);

/* Replaces Context::new (device/context.rs:34-164) + FenceSet/CommandBuffers/BufferHeap/StagingBuffer
 * construction in Environment::new (environment.rs:104-124): selects the device, creates the single stream. */
int dsc_ctx_create(int device_ordinal, dsc_ctx** out);
/* Replaces Drop for Environment (environment.rs:523-528): waits for the stream, frees everything. */
int dsc_ctx_destroy(dsc_ctx* ctx);
int dsc_ctx_caps(dsc_ctx* ctx, dsc_caps* out);
/* Replaces FenceSet::wait_for_signal on the latest fence (device/fence.rs:73-86). */
int dsc_ctx_sync(dsc_ctx* ctx);
/* FenceSet (device/fence.rs:21-86) as the reference uses it around command-buffer submission
 * (device/command_buffer.rs:64-123): dsc_fence_record marks everything enqueued on the context so far and returns
 * an id (next_unsignaled + the submit's signal); dsc_fence_wait blocks until that work has finished
 * (wait_for_signal); dsc_fence_query answers without blocking (1 = finished).  Ids grow by one per record; waiting
 * on an id also retires every older one of its stream.  A caller keeping two steps in flight, as the reference does,
 * records a fence after each dsc_schedule_run and waits on the one from two steps ago.  Fences need not be waited
 * for: finished ones are retired in the background once more than a thousand are outstanding, and an id that was
 * issued and is no longer tracked answers "finished". */
int dsc_fence_record(dsc_ctx* ctx, uint64_t* out_fence);
int dsc_fence_wait(dsc_ctx* ctx, uint64_t fence);
int dsc_fence_query(dsc_ctx* ctx, uint64_t fence, int* out_finished);
/* The HIP stream of the context as a hipStream_t (for event timing by a harness). */
int dsc_ctx_stream(dsc_ctx* ctx, void** out_stream);

/* ----------------------------------------------------------------- memory */

/* BufferHeap::alloc (device/buffer_heap.rs:79-97). *out = 0 and DSC_ERR_OOM when the device is exhausted. */
int dsc_buf_alloc(dsc_ctx* ctx, size_t bytes, dsc_buf* out);
/* BufferHeap::free (device/buffer_heap.rs:99-104). Stream-ordered: memory is reused only by later work. */
int dsc_buf_free(dsc_ctx* ctx, dsc_buf buf);
/* BufferHeap::info (device/buffer_heap.rs:106-110): device address and size of a live buffer. */
int dsc_buf_info(dsc_ctx* ctx, dsc_buf buf, void** out_device_ptr, size_t* out_bytes);
/* Number of live buffers and bytes handed out (heap accounting; device/heap.rs:97-346). */
int dsc_heap_stats(dsc_ctx* ctx, int64_t* out_live_buffers, int64_t* out_live_bytes, int64_t* out_arena_bytes);

/* StagingWriter::write_slice + flush (device/staging.rs:85-178): host -> device, stream-ordered after prior
 * launches; the host range may be reused as soon as the call returns. */
int dsc_buf_write(dsc_ctx* ctx, dsc_buf buf, size_t offset, const void* src, size_t bytes);
/* StagingWriter::write_zeros / zero-fill of the unwritten tail on drop (device/staging.rs:125-141,181-187). */
int dsc_buf_fill_zero(dsc_ctx* ctx, dsc_buf buf, size_t offset, size_t bytes);
/* StagingReader::read_slice to completion (device/staging.rs:225-302): device -> host, blocking. */
int dsc_buf_read(dsc_ctx* ctx, dsc_buf buf, size_t offset, void* dst, size_t bytes);

/* Overlapped parameter I/O.  The reference pushes every upload and read-back through the one queue that also runs
 * the kernels (StagingWriter / StagingReader submit on the shared command buffers, device/staging.rs:143-178,
 * 262-302), so a mini-batch upload (examples/fashion_mnist/main.rs:42-60 through Environment::writer,
 * environment.rs:160-175) serialises with the step before it.  These entry points use a second stream:
 *   dsc_buf_alloc_io                 a buffer like dsc_buf_alloc's (same handle type, same dsc_buf_free), from device
 *                                    memory set aside for uploads: nothing else is ever placed there, so what the
 *                                    memory held before is an older upload buffer and not a temporary of the step
 *                                    that is still running;
 *   dsc_host_alloc / dsc_host_free   pinned host memory that copies can use in place (no staging copy);
 *   dsc_buf_write_async              host -> device on the copy stream.  The copy waits only for the compute work that
 *                                    last used the buffer's memory, so it runs beside a step enqueued earlier when the
 *                                    buffer was not taken from memory that step used (dsc_buf_alloc_io, and allocate the
 *                                    new buffer before freeing the old one); every later launch, run or copy on the compute stream waits
 *                                    for it.  `src` inside a dsc_host_alloc range is read in place and must stay
 *                                    untouched until *out_fence has finished; any other `src` is copied through the
 *                                    staging ring before the call returns.  out_fence may be null.
 *   dsc_buf_read_async               device -> pinned host (dst must come from dsc_host_alloc) of the value that the
 *                                    work enqueued so far leaves in the buffer; the data is there once *out_fence has
 *                                    finished (dsc_fence_wait / dsc_fence_query).  The host does not block.
 * Fences of the copy stream share the id space of dsc_fence_record; waiting for one retires only older fences of the
 * same stream. */
int dsc_buf_alloc_io(dsc_ctx* ctx, size_t bytes, dsc_buf* out);
int dsc_host_alloc(dsc_ctx* ctx, size_t bytes, void** out_ptr);
int dsc_host_free(dsc_ctx* ctx, void* ptr);
int dsc_buf_write_async(dsc_ctx* ctx, dsc_buf buf, size_t offset, const void* src, size_t bytes, uint64_t* out_fence);
int dsc_buf_read_async(dsc_ctx* ctx, dsc_buf buf, size_t offset, void* dst, size_t bytes, uint64_t* out_fence);

struct dsc_schedule_desc;

/* ---------------------------------------------------------------- kernels */

/* KernelCache::module (kernel.rs:1050-1055): returns the compiled kernel for a descriptor, generating HIP
 * C++ and compiling it with hipRTC for gfx950 on first sight; later calls with an equal descriptor return
 * the same object.  The descriptor is deep-copied.  Kernels live as long as the context. */
int dsc_kernel_get(dsc_ctx* ctx, const dsc_kernel_desc* desc, dsc_kernel** out);
/* Kernel::buffer_count / group_count / label_name (kernel.rs:135-143). group_count is the reference's
 * dispatch size (what vkCmdDispatch would receive), kept for reporting; this backend picks its own grid. */
int dsc_kernel_buffer_count(const dsc_kernel* k);
int64_t dsc_kernel_reference_group_count(const dsc_kernel* k);
const char* dsc_kernel_label(const dsc_kernel* k);
/* Generated HIP source of a kernel (reference: the `println!("{}", source)` hook, kernel.rs:950). */
const char* dsc_kernel_source(const dsc_kernel* k);

/* Environment::run_kernel (environment.rs:241-324): binds `n` buffers (inputs then outputs), passes the
 * 4-byte rand seed (push constant, kernel.rs:1000-1004) and enqueues the kernel on the context's stream. */
int dsc_kernel_launch(dsc_ctx* ctx, dsc_kernel* k, const dsc_buf* bufs, int n, uint32_t rand_seed);

/* Source generation and compilation without a device (used by CPU-only tests of the code generator):
 * writes the generated source into a malloc'd string the caller releases with dsc_free_string. */
int dsc_codegen_source(const dsc_kernel_desc* desc, char** out_source);
/* Compiles the generated source for `arch` ("gfx950") with hipRTC; no GPU needed. Returns the code object
 * size through out_code_bytes. */
int dsc_codegen_compile(const dsc_kernel_desc* desc, const char* arch, size_t* out_code_bytes);
/* Plans a whole schedule (fusion included) and compiles every kernel it would launch for `arch`, without a
 * device; out_text (optional) receives the listing dsc_schedule_describe would give. */
int dsc_codegen_check_schedule(const struct dsc_schedule_desc* desc, uint32_t flags, const char* arch, char** out_text);
/* The on-disk code-object cache behind dsc_kernel_get and dsc_schedule_create (the reference keeps compiled
 * modules per process only, keyed by descriptor, kernel.rs:1037-1056; here a code object also survives the process,
 * as a file named by a hash of the generated source, the target, the compile options and the hipRTC / HIP runtime
 * versions, in $DSC_CACHE_DIR or ~/.cache/descent_amd; DSC_CACHE_DIR=off disables it).  A file is used only if its
 * header (length and checksum of the payload) matches and the payload is an AMDGPU ELF image; any other file is
 * deleted and the kernel recompiled, and so is an object the runtime refuses to load.  Process-wide counters:
 * files used, hipRTC compilations, files refused and deleted.  Any pointer may be null. */
int dsc_cache_stats(int64_t* out_hits, int64_t* out_compiles, int64_t* out_rejected);
void dsc_free_string(char* s);

/* -------------------------------------------------------------- schedules */

/*
 * A whole `Graph` (graph.rs:102-108) handed over once: the topologically sorted cluster list with the op
 * nodes each cluster reads and writes, and the parameter input/output nodes.  dsc_schedule_run then performs
 * what Environment::run does per step (environment.rs:326-516): use-count driven buffer lifetimes, lazy
 * allocation, accumulator hand-off / Fill for ScatterAdd (environment.rs:410-444), in-order launches, and
 * moving output buffers into parameters without a copy (environment.rs:506-515).
 *
 * Handing the list over as a whole is what lets the backend fuse across clusters (split-K MatMul + Reduce +
 * per-element epilogue into one MFMA kernel, window copy + Reduce(max) into one pooling kernel, ...) while
 * array.rs / graph.rs stay unchanged.
 */
typedef struct dsc_cluster_output {
    int32_t node;       /* op node id written (graph.rs:63-66 ClusterOutput.node_id) */
    int32_t copy_from;  /* InitialState::CopyFrom(node) or -1 for Undefined (graph.rs:56-60) */
    int32_t copy_from_is_literal; /* source node is Op::Literal (environment.rs:419) */
    uint32_t literal_bits;        /* its value bits */
} dsc_cluster_output;

typedef struct dsc_cluster {
    dsc_kernel_desc kernel;
    int32_t n_inputs;
    const int32_t* inputs;             /* op node ids, binding order (graph.rs:87) */
    int32_t n_outputs;
    const dsc_cluster_output* outputs; /* graph.rs:88 */
} dsc_cluster;

typedef struct dsc_param_io {
    int32_t node;   /* Input: the Op::Input node; Output: the node whose buffer becomes the parameter's */
    int32_t param;  /* caller's parameter slot: index into the `params` array of dsc_schedule_run */
} dsc_param_io;

typedef struct dsc_schedule_desc {
    int32_t n_nodes;             /* op node id bound (graph.ops.node_bound()) */
    const int64_t* node_elements;/* element count per node id (0 for absent ids) */
    int32_t n_clusters;
    const dsc_cluster* clusters; /* in clusters_sorted order (graph.rs:107) */
    int32_t n_inputs;
    const dsc_param_io* inputs;  /* Op::Input nodes (environment.rs:330-340) */
    int32_t n_outputs;
    const dsc_param_io* outputs; /* Op::Output nodes' sources (environment.rs:341-351, 506-515) */
    int32_t n_params;            /* length of the params array */
} dsc_schedule_desc;

typedef struct dsc_schedule dsc_schedule;

/* flags for dsc_schedule_create */
#define DSC_SCHEDULE_NO_FUSION 1u /* launch exactly one kernel per reference cluster (for parity tests) */
#define DSC_SCHEDULE_GRAPH_REPLAY 4u /* capture each run's launches as a HIP graph and replay it whenever a later run's
                                        buffers land on the same addresses (the Submit half of the reference's
                                        command buffer, device/command_buffer.rs:64-123, recorded once).  For the
                                        addresses to repeat, such a schedule keeps its intermediates in one region
                                        of its own and holds one spare buffer per written parameter slot: a run
                                        returns the spare as the slot's new buffer and keeps the old one as the
                                        next spare (the region and the spares go back to the heap in
                                        dsc_schedule_destroy) */
#define DSC_SCHEDULE_NO_CONV_KERNELS 2u /* keep convolutions (forward and data gradient) on the generic MatMul path
                                           (fused producers) instead of the dedicated LDS-tiled kernels (for
                                           parity tests) */

#define DSC_SCHEDULE_SPLIT_CONV_GRADS 8u /* a convolution's data gradient and filter gradient stay two kernels (the
                                           dedicated data-gradient kernel and the tall-k MatMul) instead of sharing
                                           the one that holds dC and the input tile in LDS (for parity tests) */

int dsc_schedule_create(dsc_ctx* ctx, const dsc_schedule_desc* desc, uint32_t flags, dsc_schedule** out);
/* Destroy every schedule BEFORE the context it was created on: dsc_schedule_destroy returns the schedule's replay
   region and spare buffers to that context's heap, and dsc_ctx_destroy does not know the context's schedules.  A
   schedule destroyed after its context is a use of freed memory.  (The reference has no such object: its
   Environment owns device and kernel cache together and drops them in one place, src/environment.rs:523-528.) */
int dsc_schedule_destroy(dsc_ctx* ctx, dsc_schedule* s);
/* Environment::run (environment.rs:326-516). `params[slot]` holds each parameter's current buffer (0 if
 * none) and is updated in place with the buffers the run leaves in the parameters. */
int dsc_schedule_run(dsc_ctx* ctx, dsc_schedule* s, dsc_buf* params, uint32_t rand_seed);
/*
 * dsc_schedule_run for callers that cannot allocate device memory (code under HIP-graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference, whose run allocates every
 * cluster output from the BufferHeap as it goes (environment.rs:404-444).
 *
 * Same work, same kernels and same results as dsc_schedule_run, but no hipMalloc / hipFree and no call into the
 * library's heap: every intermediate of the run is placed in a fixed array of DSC_STATIC_SCRATCH_BYTES that is part
 * of the library's device code (each GPU the library runs on holds its own copy from first use until the process
 * ends), and every parameter the run writes goes into a buffer the caller provides:
 *   params[slot]  the current buffer of every parameter, as for dsc_schedule_run;
 *   spare[slot]   for every slot the schedule writes: a caller-owned buffer, different from params[slot], of at
 *                 least the parameter's size; slots the schedule only reads are ignored (0 is fine).
 * On success the two are swapped for every written slot: params[slot] holds the new value and spare[slot] the
 * buffer the old value was in, ready to be the spare of the next call (a parameter that the run updates in place,
 * by ScatterAdd into its own buffer, keeps its buffer; its spare is left alone).  Nothing is freed.
 *
 * A run whose intermediates do not fit the array at once is refused with DSC_ERR_UNSUPPORTED before anything is
 * enqueued (the message names the size that did not fit); so are a context with per-launch timing on
 * (dsc_prof_enable creates events) and DSC_SCHEDULE_GRAPH_REPLAY schedules.  All calls on one GPU share
 * that GPU's array and it keeps the last call's contents: the schedule's own Fill launches clear what has to start
 * at zero, and two calls whose work overlaps on one GPU (two contexts, two streams) race -- finish one
 * (dsc_ctx_sync / a fence) before another context starts the next.
 */
#define DSC_STATIC_SCRATCH_BYTES (64u << 20)
int dsc_schedule_run_static(dsc_ctx* ctx, dsc_schedule* s, dsc_buf* params, dsc_buf* spare, uint32_t rand_seed);
/* Number of device kernels one run launches after fusion, and the reference cluster count. */
int dsc_schedule_launch_count(const dsc_schedule* s, int32_t* out_launches, int32_t* out_clusters);
/* Text listing of the post-fusion schedule (reference: Graph::write_dot, graph.rs:661-763). Caller releases
 * with dsc_free_string. */
int dsc_schedule_describe(const dsc_schedule* s, char** out_text);
/* Graph::write_dot_file (graph.rs:656-760), for the schedule after fusion: a graphviz digraph with one box per
 * launch (label, kernel choice, grid, algorithmic bytes, reference clusters covered), one ellipse per parameter slot
 * and one edge per buffer handed from launch to launch.  Free the text with dsc_free_string. */
int dsc_schedule_dot(const dsc_schedule* s, char** out_text);

/* ----------------------------------------------------------------- timing */

/* TimestampSets (device/timestamp.rs:196-287): when enabled every launch is bracketed by events and the
 * elapsed time is accumulated per kernel label; dsc_prof_report prints total and top-N like
 * print_timings (device/timestamp.rs:155-179, environment.rs:518-520). */
int dsc_prof_enable(dsc_ctx* ctx, int enabled);
/* Debug labels per cluster (environment.rs:452-463 wraps each dispatch in a debug-utils label named
 * Kernel::label_name): with `enabled`, every launch is wrapped in a ROCTx range named by the kernel's label, which
 * rocprofv3 --marker-trace records.  DSC_ERR_UNSUPPORTED when no ROCTx library can be loaded. */
int dsc_prof_markers(dsc_ctx* ctx, int enabled);
int dsc_prof_reset(dsc_ctx* ctx);
/* Writes a report into a malloc'd string (caller: dsc_free_string): one line per label with launches,
 * total ms, average us and the achieved GB/s or TFLOP/s against the HBM or fp32 MFMA peak, sorted by total
 * time, at most top_n lines (0 = all). */
int dsc_prof_report(dsc_ctx* ctx, int top_n, char** out_text);
/* Average duration in microseconds and launch count of all launches whose label starts with `prefix`. */
int dsc_prof_query(dsc_ctx* ctx, const char* prefix, double* out_avg_us, int64_t* out_launches);
/* Sums over the same launches: total microseconds, and the algorithmic bytes and flops those launches stand for
 * (bytes: 4 x distinct elements read, an operand read through a broadcast or window view at its own size, plus
 * elements written; flops: 2*b*M*N*K per MatMul).  The reference prints times only (device/timestamp.rs:155-179);
 * the work figures are what turns them into a fraction of the HBM or MFMA roof. */
int dsc_prof_work(dsc_ctx* ctx, const char* prefix, double* out_total_us, double* out_algo_bytes, double* out_algo_flops,
                  int64_t* out_launches);

#ifdef __cplusplus
}
#endif
#endif /* DESCENT_HIP_H */
