// extern "C" entry points declared in include/descent_hip.h.
#include "schedule.hpp"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <sstream>

using namespace dsc;

struct dsc_ctx {
    Context c;
};
struct dsc_kernel {
    Kernel k;
};
struct dsc_schedule {
    Schedule s;
};

// Device memory for the intermediates of dsc_schedule_run_static.  It is part of this library's device code, so
// every GPU the library runs on holds its own copy from the first use of the library there until the process ends,
// and using it needs no allocation.  In host code this name only stands for the array (it is what
// hipGetSymbolAddress looks up); the array's device address on a GPU is what scratch_address() stores per device.
static __device__ __align__(256) unsigned char scratch[DSC_STATIC_SCRATCH_BYTES];

namespace {

constexpr int kMaxDevices = 64;
char* g_scratch_ptr[kMaxDevices];  // per device: its copy's address, once resolved

// Resolves (once per device) the address of `device`'s copy of the scratch array.  `device` must be current.
hipError_t scratch_address(int device, char** out) {
    *out = nullptr;
    if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
    if (!g_scratch_ptr[device]) {
        void* p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) {
            (void)hipGetLastError();
            return e;
        }
        g_scratch_ptr[device] = static_cast<char*>(p);
    }
    *out = g_scratch_ptr[device];
    return hipSuccess;
}

char* dup_string(const std::string& s) {
    char* out = static_cast<char*>(std::malloc(s.size() + 1));
    if (out) std::memcpy(out, s.c_str(), s.size() + 1);
    return out;
}

#define HIP_TRY(expr)                                                                                     \
    do {                                                                                                  \
        hipError_t e_ = (expr);                                                                           \
        if (e_ != hipSuccess) return fail(DSC_ERR_HIP, std::string(#expr) + ": " + hipGetErrorString(e_)); \
    } while (0)

// Waits until staging region `r` is free again.
int staging_acquire(Context* c, int r) {
    if (c->staging_busy[r]) {
        HIP_TRY(hipEventSynchronize(c->staging_done[r]));
        c->staging_busy[r] = false;
    }
    return DSC_OK;
}

int resolve(Context* c, dsc_buf buf, size_t offset, size_t bytes, char** ptr) {
    void* p = nullptr;
    size_t size = 0;
    if (!c->heap.info(buf, &p, &size)) return fail(DSC_ERR_INVALID, "unknown buffer handle");
    if (offset > size || bytes > size - offset) return fail(DSC_ERR_INVALID, "range outside the buffer");
    *ptr = static_cast<char*>(p) + offset;
    return DSC_OK;
}

}  // namespace

extern "C" {

const char* dsc_last_error(void) { return last_error().c_str(); }

int dsc_ctx_create(int device_ordinal, dsc_ctx** out) {
    if (!out) return fail(DSC_ERR_INVALID, "null out pointer");
    *out = nullptr;
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || count <= 0) {
        (void)hipGetLastError();
        return fail(DSC_ERR_NO_DEVICE, "no HIP device available");
    }
    if (device_ordinal < 0 || device_ordinal >= count) return fail(DSC_ERR_INVALID, "device ordinal out of range");
    HIP_TRY(hipSetDevice(device_ordinal));
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, device_ordinal));
    auto ctx = new dsc_ctx();
    Context& c = ctx->c;
    c.device = device_ordinal;
    c.arch = prop.gcnArchName;
    const size_t colon = c.arch.find(':');
    if (colon != std::string::npos) c.arch = c.arch.substr(0, colon);
    c.caps.has_float_atomic_add = 1;
    c.caps.compute_units = prop.multiProcessorCount;
    c.caps.wavefront_size = prop.warpSize;
    c.caps.device_memory_bytes = (int64_t)prop.totalGlobalMem;
    std::snprintf(c.caps.arch, sizeof c.caps.arch, "%s", c.arch.c_str());
    if (c.arch != "gfx950") {
        delete ctx;
        return fail(DSC_ERR_NO_DEVICE, "device is " + std::string(prop.gcnArchName) + "; this backend is written for gfx950 only");
    }
    hipError_t e = hipStreamCreate(&c.stream);
    if (e != hipSuccess) {
        delete ctx;
        return fail(DSC_ERR_HIP, std::string("hipStreamCreate: ") + hipGetErrorString(e));
    }
    // this device's copy of the static scratch array (the device is current here); a failure only disables
    // dsc_schedule_run_static, which then reports it
    e = scratch_address(device_ordinal, &c.static_scratch);
    if (e != hipSuccess) c.static_scratch_error = std::string("hipGetSymbolAddress(scratch): ") + hipGetErrorString(e);
    {
        void* cell = nullptr;
        e = hipMalloc(&cell, 256);
        if (e != hipSuccess) {
            delete ctx;
            return fail(DSC_ERR_HIP, std::string("seed cell: ") + hipGetErrorString(e));
        }
        c.seed_cell = static_cast<uint32_t*>(cell);
    }
    for (int i = 0; i < Context::kStagingRegions; ++i) {
        void* p = nullptr;
        e = hipHostMalloc(&p, Context::kStagingBytes, hipHostMallocDefault);
        if (e == hipSuccess) e = hipEventCreateWithFlags(&c.staging_done[i], hipEventDisableTiming);
        if (e != hipSuccess) {
            delete ctx;
            return fail(DSC_ERR_HIP, std::string("staging setup: ") + hipGetErrorString(e));
        }
        c.staging[i] = static_cast<char*>(p);
    }
    *out = ctx;
    return DSC_OK;
}

int dsc_ctx_destroy(dsc_ctx* ctx) {
    if (!ctx) return DSC_OK;
    (void)hipSetDevice(ctx->c.device);
    delete ctx;
    return DSC_OK;
}

int dsc_ctx_caps(dsc_ctx* ctx, dsc_caps* out) {
    if (!ctx || !out) return fail(DSC_ERR_INVALID, "null argument");
    *out = ctx->c.caps;
    return DSC_OK;
}

int dsc_ctx_sync(dsc_ctx* ctx) {
    if (!ctx) return fail(DSC_ERR_INVALID, "null context");
    if (ctx->c.copy_stream) HIP_TRY(hipStreamSynchronize(ctx->c.copy_stream));
    HIP_TRY(hipStreamSynchronize(ctx->c.stream));
    return DSC_OK;
}

namespace {
// Records a new fence on `stream` and returns its id (0 on failure, with the error set).
uint64_t record_fence(Context* c, hipStream_t stream, bool on_copy_stream) {
    hipEvent_t ev = take_plain_event(c);
    if (!ev) {
        fail(DSC_ERR_HIP, "hipEventCreate failed");
        return 0;
    }
    const hipError_t e = hipEventRecord(ev, stream);
    if (e != hipSuccess) {
        c->fence_pool.push_back(ev);
        fail(DSC_ERR_HIP, std::string("hipEventRecord: ") + hipGetErrorString(e));
        return 0;
    }
    const uint64_t id = c->fence_next++;
    c->fences[id] = Context::Fence{ev, on_copy_stream};
    // a caller that never waits for its fences (fire-and-forget uploads) must not pile up events: past a thousand
    // known fences the finished ones among the oldest are retired (an id that is no longer known counts as finished)
    if (c->fences.size() > 1024) {
        int looked = 0;
        for (auto it = c->fences.begin(); it != c->fences.end() && looked < 64 && it->first != id; ++looked) {
            if (hipEventQuery(it->second.event) == hipSuccess) {
                c->fence_pool.push_back(it->second.event);
                it = c->fences.erase(it);
            } else {
                (void)hipGetLastError();
                ++it;
            }
        }
    }
    return id;
}

// `fence` has finished; each stream is in order, so the older fences of its stream have finished too
void retire_fences(Context* c, uint64_t fence, bool on_copy_stream) {
    for (auto it = c->fences.begin(); it != c->fences.end() && it->first <= fence;) {
        if (it->second.on_copy_stream == on_copy_stream) {
            c->fence_pool.push_back(it->second.event);
            it = c->fences.erase(it);
        } else {
            ++it;
        }
    }
}
}  // namespace

int dsc_fence_record(dsc_ctx* ctx, uint64_t* out_fence) {
    if (!ctx || !out_fence) return fail(DSC_ERR_INVALID, "null argument");
    *out_fence = record_fence(&ctx->c, ctx->c.stream, false);
    return *out_fence ? DSC_OK : DSC_ERR_HIP;
}

int dsc_fence_wait(dsc_ctx* ctx, uint64_t fence) {
    if (!ctx) return fail(DSC_ERR_INVALID, "null context");
    Context* c = &ctx->c;
    if (fence == 0 || fence >= c->fence_next) return fail(DSC_ERR_INVALID, "unknown fence id");
    auto it = c->fences.find(fence);
    if (it == c->fences.end()) return DSC_OK;  // retired
    HIP_TRY(hipEventSynchronize(it->second.event));
    retire_fences(c, fence, it->second.on_copy_stream);
    return DSC_OK;
}

int dsc_fence_query(dsc_ctx* ctx, uint64_t fence, int* out_finished) {
    if (!ctx || !out_finished) return fail(DSC_ERR_INVALID, "null argument");
    Context* c = &ctx->c;
    if (fence == 0 || fence >= c->fence_next) return fail(DSC_ERR_INVALID, "unknown fence id");
    auto it = c->fences.find(fence);
    if (it == c->fences.end()) {
        *out_finished = 1;
        return DSC_OK;
    }
    const hipError_t e = hipEventQuery(it->second.event);
    if (e == hipSuccess) {
        *out_finished = 1;
        retire_fences(c, fence, it->second.on_copy_stream);
        return DSC_OK;
    }
    if (e != hipErrorNotReady) return fail(DSC_ERR_HIP, std::string("hipEventQuery: ") + hipGetErrorString(e));
    (void)hipGetLastError();
    *out_finished = 0;
    return DSC_OK;
}

int dsc_ctx_stream(dsc_ctx* ctx, void** out_stream) {
    if (!ctx || !out_stream) return fail(DSC_ERR_INVALID, "null argument");
    *out_stream = ctx->c.stream;
    return DSC_OK;
}

int dsc_buf_alloc(dsc_ctx* ctx, size_t bytes, dsc_buf* out) {
    if (!ctx || !out) return fail(DSC_ERR_INVALID, "null argument");
    *out = ctx->c.heap.alloc(bytes);
    if (!*out) return fail(DSC_ERR_OOM, "device memory exhausted allocating " + std::to_string(bytes) + " bytes");
    return DSC_OK;
}

int dsc_buf_alloc_io(dsc_ctx* ctx, size_t bytes, dsc_buf* out) {
    if (!ctx || !out) return fail(DSC_ERR_INVALID, "null argument");
    *out = ctx->c.heap.alloc(bytes, true);
    if (!*out) return fail(DSC_ERR_OOM, "device memory exhausted allocating " + std::to_string(bytes) + " bytes");
    return DSC_OK;
}

int dsc_buf_free(dsc_ctx* ctx, dsc_buf buf) {
    if (!ctx) return fail(DSC_ERR_INVALID, "null context");
    if (!ctx->c.heap.free(buf)) return fail(DSC_ERR_INVALID, "free of an unknown or already freed buffer");
    return DSC_OK;
}

int dsc_buf_info(dsc_ctx* ctx, dsc_buf buf, void** out_device_ptr, size_t* out_bytes) {
    if (!ctx) return fail(DSC_ERR_INVALID, "null context");
    if (!ctx->c.heap.info(buf, out_device_ptr, out_bytes)) return fail(DSC_ERR_INVALID, "unknown buffer handle");
    return DSC_OK;
}

int dsc_heap_stats(dsc_ctx* ctx, int64_t* out_live_buffers, int64_t* out_live_bytes, int64_t* out_arena_bytes) {
    if (!ctx) return fail(DSC_ERR_INVALID, "null context");
    ctx->c.heap.stats(out_live_buffers, out_live_bytes, out_arena_bytes);
    return DSC_OK;
}

int dsc_buf_write(dsc_ctx* ctx, dsc_buf buf, size_t offset, const void* src, size_t bytes) {
    if (!ctx || (!src && bytes)) return fail(DSC_ERR_INVALID, "null argument");
    Context* c = &ctx->c;
    char* dst = nullptr;
    int rc = resolve(c, buf, offset, bytes, &dst);
    if (rc == DSC_OK) rc = join_copies(c);
    if (rc != DSC_OK) return rc;
    c->heap.touch(buf, ++c->work_seq);
    const char* s = static_cast<const char*>(src);
    while (bytes) {
        const int r = c->staging_next;
        c->staging_next = (r + 1) % Context::kStagingRegions;
        rc = staging_acquire(c, r);
        if (rc != DSC_OK) return rc;
        const size_t n = std::min(bytes, Context::kStagingBytes);
        std::memcpy(c->staging[r], s, n);
        HIP_TRY(hipMemcpyAsync(dst, c->staging[r], n, hipMemcpyHostToDevice, c->stream));
        HIP_TRY(hipEventRecord(c->staging_done[r], c->stream));
        c->staging_busy[r] = true;
        s += n;
        dst += n;
        bytes -= n;
    }
    return DSC_OK;
}

int dsc_buf_fill_zero(dsc_ctx* ctx, dsc_buf buf, size_t offset, size_t bytes) {
    if (!ctx) return fail(DSC_ERR_INVALID, "null context");
    char* dst = nullptr;
    int rc = resolve(&ctx->c, buf, offset, bytes, &dst);
    if (rc == DSC_OK) rc = join_copies(&ctx->c);
    if (rc != DSC_OK) return rc;
    ctx->c.heap.touch(buf, ++ctx->c.work_seq);
    if (bytes) HIP_TRY(hipMemsetAsync(dst, 0, bytes, ctx->c.stream));
    return DSC_OK;
}

int dsc_buf_read(dsc_ctx* ctx, dsc_buf buf, size_t offset, void* dst, size_t bytes) {
    if (!ctx || (!dst && bytes)) return fail(DSC_ERR_INVALID, "null argument");
    Context* c = &ctx->c;
    char* src = nullptr;
    int rc = resolve(c, buf, offset, bytes, &src);
    if (rc == DSC_OK) rc = join_copies(c);
    if (rc != DSC_OK) return rc;
    c->heap.touch(buf, ++c->work_seq);
    char* d = static_cast<char*>(dst);
    // two regions in flight: the copy into region r+1 overlaps the host memcpy out of region r
    size_t pending_n[Context::kStagingRegions] = {0, 0};
    char* pending_dst[Context::kStagingRegions] = {nullptr, nullptr};
    auto drain = [&](int r) -> int {
        if (!pending_n[r]) return DSC_OK;
        HIP_TRY(hipEventSynchronize(c->staging_done[r]));
        c->staging_busy[r] = false;
        std::memcpy(pending_dst[r], c->staging[r], pending_n[r]);
        pending_n[r] = 0;
        return DSC_OK;
    };
    int r = 0;
    while (bytes) {
        rc = drain(r);
        if (rc != DSC_OK) return rc;
        rc = staging_acquire(c, r);
        if (rc != DSC_OK) return rc;
        const size_t n = std::min(bytes, Context::kStagingBytes);
        HIP_TRY(hipMemcpyAsync(c->staging[r], src, n, hipMemcpyDeviceToHost, c->stream));
        HIP_TRY(hipEventRecord(c->staging_done[r], c->stream));
        c->staging_busy[r] = true;
        pending_n[r] = n;
        pending_dst[r] = d;
        src += n;
        d += n;
        bytes -= n;
        r = (r + 1) % Context::kStagingRegions;
    }
    for (int i = 0; i < Context::kStagingRegions; ++i) {
        rc = drain((r + i) % Context::kStagingRegions);
        if (rc != DSC_OK) return rc;
    }
    return DSC_OK;
}

int dsc_host_alloc(dsc_ctx* ctx, size_t bytes, void** out_ptr) {
    if (!ctx || !out_ptr || !bytes) return fail(DSC_ERR_INVALID, "null argument or empty allocation");
    void* p = nullptr;
    if (hipHostMalloc(&p, bytes, hipHostMallocDefault) != hipSuccess) {
        (void)hipGetLastError();
        return fail(DSC_ERR_OOM, "pinned host memory exhausted allocating " + std::to_string(bytes) + " bytes");
    }
    ctx->c.pinned[static_cast<const char*>(p)] = bytes;
    *out_ptr = p;
    return DSC_OK;
}

int dsc_host_free(dsc_ctx* ctx, void* ptr) {
    if (!ctx) return fail(DSC_ERR_INVALID, "null context");
    Context* c = &ctx->c;
    auto it = c->pinned.find(static_cast<const char*>(ptr));
    if (it == c->pinned.end()) return fail(DSC_ERR_INVALID, "not a dsc_host_alloc pointer");
    // a copy may still be reading or writing it
    if (c->copy_stream) HIP_TRY(hipStreamSynchronize(c->copy_stream));
    HIP_TRY(hipHostFree(ptr));
    c->pinned.erase(it);
    return DSC_OK;
}

namespace {
// whether [p, p + bytes) lies inside one dsc_host_alloc range
bool is_pinned(const Context* c, const void* p, size_t bytes) {
    const char* q = static_cast<const char*>(p);
    auto it = c->pinned.upper_bound(q);
    if (it == c->pinned.begin()) return false;
    --it;
    return q >= it->first && bytes <= it->second && size_t(q - it->first) <= it->second - bytes;
}

// after a copy-stream operation: the fence the caller (or only the compute stream) will wait for
int finish_copy(Context* c, uint64_t* out_fence) {
    if (out_fence) {
        *out_fence = record_fence(c, c->copy_stream, true);
        if (!*out_fence) return DSC_ERR_HIP;
        c->copies.push_back(Context::CopyInFlight{*out_fence, nullptr});
        return DSC_OK;
    }
    hipEvent_t ev = take_plain_event(c);
    if (!ev) return fail(DSC_ERR_HIP, "hipEventCreate failed");
    const hipError_t e = hipEventRecord(ev, c->copy_stream);
    if (e != hipSuccess) {
        c->fence_pool.push_back(ev);
        return fail(DSC_ERR_HIP, std::string("hipEventRecord: ") + hipGetErrorString(e));
    }
    c->copies.push_back(Context::CopyInFlight{0, ev});
    return DSC_OK;
}
}  // namespace

int dsc_buf_write_async(dsc_ctx* ctx, dsc_buf buf, size_t offset, const void* src, size_t bytes, uint64_t* out_fence) {
    if (!ctx || (!src && bytes)) return fail(DSC_ERR_INVALID, "null argument");
    Context* c = &ctx->c;
    if (out_fence) *out_fence = 0;
    char* dst = nullptr;
    int rc = resolve(c, buf, offset, bytes, &dst);
    if (rc == DSC_OK) rc = enable_async_io(c);
    // the copy may start once the compute work that last used this memory -- as this buffer, or as whatever the
    // range held before -- has finished; work enqueued earlier that does not touch it keeps running beside the copy
    if (rc == DSC_OK) rc = copy_stream_wait(c, c->heap.stamp_of(buf));
    if (rc != DSC_OK) return rc;
    if (is_pinned(c, src, bytes)) {
        if (bytes) HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, c->copy_stream));
        return finish_copy(c, out_fence);
    }
    const char* s = static_cast<const char*>(src);
    while (bytes) {
        const int r = c->staging_next;
        c->staging_next = (r + 1) % Context::kStagingRegions;
        rc = staging_acquire(c, r);
        if (rc != DSC_OK) return rc;
        const size_t n = std::min(bytes, Context::kStagingBytes);
        std::memcpy(c->staging[r], s, n);
        HIP_TRY(hipMemcpyAsync(dst, c->staging[r], n, hipMemcpyHostToDevice, c->copy_stream));
        HIP_TRY(hipEventRecord(c->staging_done[r], c->copy_stream));
        c->staging_busy[r] = true;
        s += n;
        dst += n;
        bytes -= n;
    }
    return finish_copy(c, out_fence);
}

int dsc_buf_read_async(dsc_ctx* ctx, dsc_buf buf, size_t offset, void* dst, size_t bytes, uint64_t* out_fence) {
    if (!ctx || !out_fence || (!dst && bytes)) return fail(DSC_ERR_INVALID, "null argument");
    Context* c = &ctx->c;
    *out_fence = 0;
    if (!is_pinned(c, dst, bytes)) return fail(DSC_ERR_INVALID, "dsc_buf_read_async needs a destination from dsc_host_alloc");
    char* src = nullptr;
    int rc = resolve(c, buf, offset, bytes, &src);
    if (rc == DSC_OK) rc = enable_async_io(c);
    // the value is whatever the compute work enqueued so far leaves in the buffer
    if (rc == DSC_OK) rc = copy_stream_wait(c, c->heap.stamp_of(buf));
    if (rc != DSC_OK) return rc;
    if (bytes) HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, c->copy_stream));
    return finish_copy(c, out_fence);
}

int dsc_kernel_get(dsc_ctx* ctx, const dsc_kernel_desc* desc, dsc_kernel** out) {
    if (!ctx || !desc || !out) return fail(DSC_ERR_INVALID, "null argument");
    *out = nullptr;
    std::string err = validate(*desc);
    if (!err.empty()) return fail(DSC_ERR_INVALID, err);
    int status = DSC_OK;
    Kernel* k = get_kernel(&ctx->c, FusedKernel::plain(*desc), &status);
    if (!k) return status;
    *out = reinterpret_cast<dsc_kernel*>(k);
    return DSC_OK;
}

int dsc_kernel_buffer_count(const dsc_kernel* k) { return k ? reinterpret_cast<const Kernel*>(k)->gen.n_buffers : 0; }
int64_t dsc_kernel_reference_group_count(const dsc_kernel* k) { return k ? reinterpret_cast<const Kernel*>(k)->reference_groups : 0; }
const char* dsc_kernel_label(const dsc_kernel* k) { return k ? reinterpret_cast<const Kernel*>(k)->label.c_str() : ""; }
const char* dsc_kernel_source(const dsc_kernel* k) { return k ? reinterpret_cast<const Kernel*>(k)->gen.source.c_str() : ""; }

int dsc_kernel_launch(dsc_ctx* ctx, dsc_kernel* kernel, const dsc_buf* bufs, int n, uint32_t rand_seed) {
    if (!ctx || !kernel || (!bufs && n)) return fail(DSC_ERR_INVALID, "null argument");
    Kernel* k = reinterpret_cast<Kernel*>(kernel);
    if (n != k->gen.n_buffers) return fail(DSC_ERR_INVALID, "wrong number of buffers for '" + k->label + "'");
    if (n > 256) return fail(DSC_ERR_UNSUPPORTED, "more than 256 buffers");
    void* ptrs[256];
    // every bound buffer must hold at least what the kernel addresses
    const dsc_kernel_desc& d = k->fused.main.raw();
    for (int i = 0; i < n; ++i) {
        size_t size = 0;
        if (!ctx->c.heap.info(bufs[i], &ptrs[i], &size)) return fail(DSC_ERR_INVALID, "unknown buffer handle in launch");
        size_t need = 0;
        if (i < d.n_inputs) need = (size_t)element_count(d.inputs[i].in_shape) * 4;
        else need = (size_t)element_count(d.shape) * 4;
        if (size < need) return fail(DSC_ERR_INVALID, "buffer " + std::to_string(i) + " of '" + k->label + "' is too small");
    }
    int rc = join_copies(&ctx->c);
    if (rc != DSC_OK) return rc;
    rc = launch_kernel(&ctx->c, k, ptrs, n, rand_seed);
    if (rc == DSC_OK && ctx->c.async_io)
        for (int i = 0; i < n; ++i) ctx->c.heap.touch(bufs[i], ctx->c.work_seq);
    return rc;
}

int dsc_codegen_source(const dsc_kernel_desc* desc, char** out_source) {
    if (!desc || !out_source) return fail(DSC_ERR_INVALID, "null argument");
    std::string err = validate(*desc);
    if (!err.empty()) return fail(DSC_ERR_INVALID, err);
    Generated g;
    err = generate(FusedKernel::plain(*desc), &g);
    if (!err.empty()) return fail(err.find("too large") != std::string::npos ? DSC_ERR_UNSUPPORTED : DSC_ERR_INVALID, err);
    *out_source = dup_string(g.source);
    return *out_source ? DSC_OK : fail(DSC_ERR_OOM, "host allocation failed");
}

int dsc_codegen_compile(const dsc_kernel_desc* desc, const char* arch, size_t* out_code_bytes) {
    if (!desc || !arch) return fail(DSC_ERR_INVALID, "null argument");
    std::string err = validate(*desc);
    if (!err.empty()) return fail(DSC_ERR_INVALID, err);
    Generated g;
    err = generate(FusedKernel::plain(*desc), &g);
    if (!err.empty()) return fail(err.find("too large") != std::string::npos ? DSC_ERR_UNSUPPORTED : DSC_ERR_INVALID, err);
    std::vector<char> code;
    std::string log;
    int rc = compile_source(g.source, arch, &code, &log);
    if (rc != DSC_OK) return rc;
    if (out_code_bytes) *out_code_bytes = code.size();
    return DSC_OK;
}

int dsc_codegen_check_schedule(const dsc_schedule_desc* desc, uint32_t flags, const char* arch, char** out_text) {
    if (!desc || !arch) return fail(DSC_ERR_INVALID, "null argument");
    Context offline;
    offline.offline = true;
    offline.arch = arch;
    Schedule s;
    int rc = s.build(&offline, *desc, flags);
    if (rc != DSC_OK) return rc;
    if (out_text) {
        *out_text = dup_string(s.describe());
        if (!*out_text) return fail(DSC_ERR_OOM, "host allocation failed");
    }
    return DSC_OK;
}

void dsc_free_string(char* s) { std::free(s); }

int dsc_cache_stats(int64_t* out_hits, int64_t* out_compiles, int64_t* out_rejected) {
    const CacheStats& st = cache_stats();
    if (out_hits) *out_hits = st.hits;
    if (out_compiles) *out_compiles = st.compiles;
    if (out_rejected) *out_rejected = st.rejected;
    return DSC_OK;
}

int dsc_schedule_create(dsc_ctx* ctx, const dsc_schedule_desc* desc, uint32_t flags, dsc_schedule** out) {
    if (!ctx || !desc || !out) return fail(DSC_ERR_INVALID, "null argument");
    *out = nullptr;
    auto s = new dsc_schedule();
    int rc = s->s.build(&ctx->c, *desc, flags);
    if (rc != DSC_OK) {
        delete s;
        return rc;
    }
    *out = s;
    return DSC_OK;
}

int dsc_schedule_destroy(dsc_ctx* ctx, dsc_schedule* s) {
    if (ctx && s) {
        // captured graphs may still be running, and the region they write goes back to the heap here
        if (s->s.has_captured_graphs()) (void)hipStreamSynchronize(ctx->c.stream);
        s->s.release_replay_buffers(&ctx->c);  // the region and spares of a schedule that replays graphs
    }
    delete s;
    return DSC_OK;
}

int dsc_schedule_run(dsc_ctx* ctx, dsc_schedule* s, dsc_buf* params, uint32_t rand_seed) {
    if (!ctx || !s || !params) return fail(DSC_ERR_INVALID, "null argument");
    Context* c = &ctx->c;
    int rc = join_copies(c);
    if (rc != DSC_OK) return rc;
    // memory released while the run is put together is still used by the run's launches: stamp it with a count
    // that only a mark recorded after the run covers
    ++c->work_seq;
    rc = s->s.run(c, params, rand_seed);
    if (rc != DSC_OK || !c->async_io) return rc;
    for (int i = 0; i < s->s.n_params; ++i)
        if (params[i]) c->heap.touch(params[i], c->work_seq);
    return mark_stream(c);
}

int dsc_schedule_run_static(dsc_ctx* ctx, dsc_schedule* s, dsc_buf* params, dsc_buf* spare, uint32_t rand_seed) {
    if (!ctx || !s || !params || !spare) return fail(DSC_ERR_INVALID, "null argument");
    Context* c = &ctx->c;
    if (c->offline) return fail(DSC_ERR_NO_DEVICE, "static run without a device");
    if (!c->static_scratch) return fail(DSC_ERR_HIP, "static run: the scratch array has no address on this device: " + c->static_scratch_error);
    if (c->profiling) return fail(DSC_ERR_UNSUPPORTED, "static run: per-launch timing is on (it creates events); dsc_prof_enable(ctx, 0) first");
    if (s->s.graph_replay) return fail(DSC_ERR_UNSUPPORTED, "static run: the schedule was created with DSC_SCHEDULE_GRAPH_REPLAY (instantiating a graph allocates)");
    // copies on the second stream enqueued so far come first (waits on their existing events; nothing is created)
    int rc = join_copies(c);
    if (rc != DSC_OK) return rc;
    ++c->work_seq;
    rc = s->s.run_static(c, params, spare, rand_seed, c->static_scratch, DSC_STATIC_SCRATCH_BYTES);
    if (rc != DSC_OK || !c->async_io) return rc;
    // use stamps for later uploads on the copy stream.  dsc_schedule_run also records an event here; this call leaves
    // that to the next upload that needs one (copy_stream_wait records a mark when none covers a buffer's stamp)
    for (int i = 0; i < s->s.n_params; ++i) {
        if (params[i]) c->heap.touch(params[i], c->work_seq);
        if (spare[i]) c->heap.touch(spare[i], c->work_seq);
    }
    return DSC_OK;
}

int dsc_schedule_launch_count(const dsc_schedule* s, int32_t* out_launches, int32_t* out_clusters) {
    if (!s) return fail(DSC_ERR_INVALID, "null schedule");
    if (out_launches) *out_launches = (int32_t)s->s.launches_per_run();
    if (out_clusters) *out_clusters = s->s.n_clusters;
    return DSC_OK;
}

int dsc_schedule_describe(const dsc_schedule* s, char** out_text) {
    if (!s || !out_text) return fail(DSC_ERR_INVALID, "null argument");
    *out_text = dup_string(s->s.describe());
    return *out_text ? DSC_OK : fail(DSC_ERR_OOM, "host allocation failed");
}

int dsc_schedule_dot(const dsc_schedule* s, char** out_text) {
    if (!s || !out_text) return fail(DSC_ERR_INVALID, "null argument");
    *out_text = dup_string(s->s.dot());
    return *out_text ? DSC_OK : fail(DSC_ERR_OOM, "host allocation failed");
}

int dsc_prof_markers(dsc_ctx* ctx, int enabled) {
    if (!ctx) return fail(DSC_ERR_INVALID, "null context");
    if (!enabled) {
        ctx->c.range_push = nullptr;
        ctx->c.range_pop = nullptr;
        return DSC_OK;
    }
    return load_markers(&ctx->c);
}

int dsc_prof_enable(dsc_ctx* ctx, int enabled) {
    if (!ctx) return fail(DSC_ERR_INVALID, "null context");
    ctx->c.profiling = enabled != 0;
    return DSC_OK;
}

int dsc_prof_reset(dsc_ctx* ctx) {
    if (!ctx) return fail(DSC_ERR_INVALID, "null context");
    HIP_TRY(hipStreamSynchronize(ctx->c.stream));
    for (auto& p : ctx->c.profile) {
        ctx->c.event_pool.push_back(p.start);
        ctx->c.event_pool.push_back(p.stop);
    }
    ctx->c.profile.clear();
    return DSC_OK;
}

namespace {
struct Acc {
    double ms = 0;
    int64_t n = 0;
    const Kernel* kernel = nullptr;
};
// Per compiled kernel: labels repeat (every hash-grid level scatters the same shape), kernels do not.
int collect(Context* c, std::map<const Kernel*, Acc>* by_kernel) {
    HIP_TRY(hipStreamSynchronize(c->stream));
    for (auto& p : c->profile) {
        float ms = 0.f;
        HIP_TRY(hipEventElapsedTime(&ms, p.start, p.stop));
        Acc& a = (*by_kernel)[p.kernel];
        a.ms += ms;
        a.n += 1;
        a.kernel = p.kernel;
    }
    return DSC_OK;
}
const double kHbmPeakGBs = 8000.0, kMfmaFp32PeakTflops = 157.3;
}  // namespace

int dsc_prof_report(dsc_ctx* ctx, int top_n, char** out_text) {
    if (!ctx || !out_text) return fail(DSC_ERR_INVALID, "null argument");
    std::map<const Kernel*, Acc> by_kernel;
    int rc = collect(&ctx->c, &by_kernel);
    if (rc != DSC_OK) return rc;
    std::vector<Acc> rows;
    for (auto& kv : by_kernel) rows.push_back(kv.second);
    std::sort(rows.begin(), rows.end(), [](const Acc& a, const Acc& b) { return a.ms > b.ms; });
    double total = 0;
    for (auto& r : rows) total += r.ms;
    std::ostringstream o;
    char line[512];
    std::snprintf(line, sizeof line, "total %.3f ms over %zu launches\n", total, ctx->c.profile.size());
    o << line;
    int shown = 0;
    for (auto& r : rows) {
        if (top_n > 0 && shown++ >= top_n) break;
        const double us = 1000.0 * r.ms / (double)r.n;
        const double gbs = r.kernel->gen.algo_bytes / (us * 1e-6) / 1e9;
        const double tf = r.kernel->gen.algo_flops / (us * 1e-6) / 1e12;
        // which roof bounds the kernel: the matrix units when it has at least their 20 flop per byte
        const bool mfma_bound = r.kernel->gen.algo_flops >= 20.0 * r.kernel->gen.algo_bytes;
        char roof[96];
        if (mfma_bound) std::snprintf(roof, sizeof roof, "%7.1f TFLOP/s %4.1f%% mfma", tf, 100.0 * tf / kMfmaFp32PeakTflops);
        else std::snprintf(roof, sizeof roof, "%7.0f GB/s    %4.1f%% hbm ", gbs, 100.0 * gbs / kHbmPeakGBs);
        std::snprintf(line, sizeof line, "%10.3f ms %8lld x %10.2f us  %s  %s  (%s)\n", r.ms, (long long)r.n, us, roof,
                      r.kernel->label.c_str(), r.kernel->gen.entry.c_str());
        o << line;
    }
    *out_text = dup_string(o.str());
    return *out_text ? DSC_OK : fail(DSC_ERR_OOM, "host allocation failed");
}

namespace {
int sum_prefix(Context* c, const char* prefix, Acc* sum, double* bytes, double* flops) {
    std::map<const Kernel*, Acc> by_kernel;
    int rc = collect(c, &by_kernel);
    if (rc != DSC_OK) return rc;
    const std::string pre(prefix);
    for (auto& kv : by_kernel) {
        if (kv.first->label.compare(0, pre.size(), pre) != 0) continue;
        sum->ms += kv.second.ms;
        sum->n += kv.second.n;
        if (bytes) *bytes += kv.first->gen.algo_bytes * (double)kv.second.n;
        if (flops) *flops += kv.first->gen.algo_flops * (double)kv.second.n;
    }
    return DSC_OK;
}
}  // namespace

int dsc_prof_query(dsc_ctx* ctx, const char* prefix, double* out_avg_us, int64_t* out_launches) {
    if (!ctx || !prefix) return fail(DSC_ERR_INVALID, "null argument");
    Acc sum;
    int rc = sum_prefix(&ctx->c, prefix, &sum, nullptr, nullptr);
    if (rc != DSC_OK) return rc;
    if (out_avg_us) *out_avg_us = sum.n ? 1000.0 * sum.ms / (double)sum.n : 0.0;
    if (out_launches) *out_launches = sum.n;
    return DSC_OK;
}

int dsc_prof_work(dsc_ctx* ctx, const char* prefix, double* out_total_us, double* out_algo_bytes, double* out_algo_flops,
                  int64_t* out_launches) {
    if (!ctx || !prefix) return fail(DSC_ERR_INVALID, "null argument");
    Acc sum;
    double bytes = 0, flops = 0;
    int rc = sum_prefix(&ctx->c, prefix, &sum, &bytes, &flops);
    if (rc != DSC_OK) return rc;
    if (out_total_us) *out_total_us = 1000.0 * sum.ms;
    if (out_algo_bytes) *out_algo_bytes = bytes;
    if (out_algo_flops) *out_algo_flops = flops;
    if (out_launches) *out_launches = sum.n;
    return DSC_OK;
}

}  // extern "C"
