// Device runtime behind the C ABI: context + stream, arena heap, pinned staging, hipRTC kernel cache,
// event profiler.  Replaces the reference's Vulkan device layer (src/device/*.rs).
#pragma once

#include "codegen.hpp"

#include <hip/hip_runtime.h>

#include <cstdint>
#include <deque>
#include <map>
#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

namespace dsc {

void set_error(const std::string& msg);
const std::string& last_error();
int fail(int status, const std::string& msg);

// Sub-allocator over large hipMalloc'd chunks (reference: BufferHeap over 256 MiB Vulkan chunks,
// device/buffer_heap.rs:29-110, with the free-list heap of device/heap.rs).  Best fit over an ordered set of
// free ranges, split on allocation, coalescing with both neighbours on free, 256-byte alignment.
class DeviceHeap {
  public:
    static constexpr size_t kAlign = 256;
    static constexpr size_t kChunkBytes = size_t(1) << 30;  // sized for 288 GB of HBM: few, large chunks

    ~DeviceHeap();
    static constexpr size_t kIoChunkBytes = size_t(256) << 20;
    // returns 0 when the device cannot provide the memory.  `io` buffers come from chunks of their own that no other
    // allocation uses: what an upload buffer's memory held before is then always an older upload buffer, never a
    // temporary of the step that is still running.  Uploads repeat in size, so these chunks recycle ranges by exact
    // size (the one unused longest first) and never split or merge them; a new size is cut from the unused tail.
    uint64_t alloc(size_t bytes, bool io = false);
    bool free(uint64_t handle);
    // Use stamps order the copy stream after the compute stream: `clock` points at the owner's count of operations
    // enqueued on the compute stream.  A range freed now may still be in use by any of them, so it is stamped with
    // the count; ranges that merge keep the later stamp; a buffer starts with the stamp of the range it was cut
    // from, and touch() raises it when compute work uses the buffer.  Work with a count at or below a buffer's stamp
    // has to finish before another stream may write the buffer.
    const uint64_t* clock = nullptr;
    uint64_t stamp_of(uint64_t handle) const;
    void touch(uint64_t handle, uint64_t stamp);
    bool info(uint64_t handle, void** ptr, size_t* bytes) const;
    void stats(int64_t* live, int64_t* live_bytes, int64_t* arena_bytes) const;

  private:
    struct Block {
        size_t size;
        bool is_free;
        uint64_t stamp;
    };
    struct Chunk {
        char* base = nullptr;
        size_t size = 0;
        bool io = false;
        size_t tail = 0;                 // io chunks: first byte never handed out
        std::map<size_t, Block> blocks;  // by offset
    };
    struct Live {
        int chunk;
        size_t offset;
        size_t bytes;  // requested size
        uint64_t stamp;
    };
    std::vector<Chunk> chunks_;
    std::multimap<size_t, std::pair<int, size_t>> free_by_size_[2];  // [io]: size -> (chunk, offset)
    std::unordered_map<uint64_t, Live> live_;
    uint64_t next_handle_ = 1;
    int64_t live_bytes_ = 0;

    uint64_t alloc_io(size_t bytes, size_t need);
    void add_free(int chunk, size_t offset, size_t size);
    void remove_free(int chunk, size_t offset, size_t size);
};

struct Kernel {
    FusedKernel fused;
    Generated gen;
    std::string label;
    hipModule_t module = nullptr;
    hipFunction_t function = nullptr;
    int64_t reference_groups = 0;
};

struct ProfileEntry {
    hipEvent_t start, stop;
    const Kernel* kernel;
};

struct Context {
    int device = 0;
    bool offline = false;  // no GPU: kernels are generated and compiled, never loaded or launched
    hipStream_t stream = nullptr;
    std::string arch;
    dsc_caps caps{};
    DeviceHeap heap;

    // pinned staging ring (reference: 2 x 4 MiB host-visible regions gated by fences, device/staging.rs:337-338)
    static constexpr int kStagingRegions = 2;
    static constexpr size_t kStagingBytes = size_t(16) << 20;
    char* staging[kStagingRegions] = {nullptr, nullptr};
    hipEvent_t staging_done[kStagingRegions] = {nullptr, nullptr};
    bool staging_busy[kStagingRegions] = {false, false};
    int staging_next = 0;

    // Launches take the rand seed by value.  While `seed_through_cell` is set (a schedule capturing or replaying a
    // HIP graph) they are given this one device word instead, which set_seed fills before the graph runs.
    bool seed_through_cell = false;
    uint32_t* seed_cell = nullptr;
    uint32_t seed_value = 0;
    bool seed_known = false;

    std::unordered_map<std::string, std::unique_ptr<Kernel>> kernels;  // by FusedKernel::key()

    // fences: id -> event recorded on one of the two streams; an id below `fence_next` that is no longer in the map
    // has finished (a finished fence retires the older fences of the same stream with it)
    struct Fence {
        hipEvent_t event;
        bool on_copy_stream;
    };
    std::map<uint64_t, Fence> fences;
    std::vector<hipEvent_t> fence_pool;
    uint64_t fence_next = 1;

    // Overlapped parameter I/O: uploads and read-backs on a second stream (created on first use, default priority).
    // `work_seq` counts operations enqueued on `stream`; `marks` are events recorded on `stream`, each covering every
    // operation up to a count; the copy stream waits for the mark that covers the stamp of the memory it touches.
    // `stream` waits for every copy enqueued before its next operation (`copies`).
    hipStream_t copy_stream = nullptr;
    bool async_io = false;
    uint64_t work_seq = 0, work_done = 0;
    std::deque<std::pair<uint64_t, hipEvent_t>> marks;
    struct CopyInFlight {
        uint64_t fence;   // id in `fences`, or 0
        hipEvent_t own;   // event owned by this entry when the caller asked for no fence
    };
    std::vector<CopyInFlight> copies;
    std::map<const char*, size_t> pinned;  // dsc_host_alloc ranges: base -> bytes

    // ROCTx ranges named by the kernel label around every launch (reference: debug-utils labels per cluster,
    // src/environment.rs:452-463); resolved from the ROCTx library at run time, null when off
    int (*range_push)(const char*) = nullptr;
    int (*range_pop)() = nullptr;

    // this device's copy of the library's static scratch array (dsc_schedule_run_static); null when its address
    // could not be resolved, with the reason in static_scratch_error
    char* static_scratch = nullptr;
    std::string static_scratch_error;

    bool profiling = false;
    std::vector<ProfileEntry> profile;
    std::vector<hipEvent_t> event_pool;

    Context() { heap.clock = &work_seq; }
    Context(const Context&) = delete;
    Context& operator=(const Context&) = delete;
    ~Context();
};

// Overlapped I/O plumbing (see Context::copy_stream).
int enable_async_io(Context* ctx);                  // creates the copy stream; everything enqueued so far is waited for once
int mark_stream(Context* ctx);                      // an event on `stream` that covers work_seq
int copy_stream_wait(Context* ctx, uint64_t stamp); // copy stream waits for compute work up to `stamp`
int join_copies(Context* ctx);                      // `stream` waits for the copies enqueued so far
hipEvent_t take_plain_event(Context* ctx);
int load_markers(Context* ctx);                     // resolves roctxRangePushA / roctxRangePop          // from fence_pool, or new; nullptr on failure


// Compiles (or fetches) the kernel for a fused descriptor.  Returns nullptr and sets the error on failure.
Kernel* get_kernel(Context* ctx, const FusedKernel& fk, int* status);
int launch_kernel(Context* ctx, Kernel* k, void* const* device_ptrs, int n, uint32_t rand_seed);
// Makes `rand_seed` the seed seen by launches enqueued after this call.
int set_seed(Context* ctx, uint32_t rand_seed);
// Code object for `source`: from the on-disk cache when a valid file is there (then *from_cache is set), else compiled
// with hipRTC (no device needed) and written to the cache.
int compile_source(const std::string& source, const std::string& arch, std::vector<char>* code, std::string* log, bool* from_cache = nullptr);
// Deletes the cache file of `source` (after the runtime refused to load what it held).
void drop_cached_object(const std::string& source, const std::string& arch);
// Process-wide counters of the on-disk cache: files used, hipRTC compilations, files refused and deleted.
struct CacheStats {
    int64_t hits = 0, compiles = 0, rejected = 0;
};
const CacheStats& cache_stats();

}  // namespace dsc
